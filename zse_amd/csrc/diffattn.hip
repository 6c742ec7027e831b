// Differential attention over the paged cache: two softmax maps a head over the same values.
//
//   q_t = [q1 | q2] c_t,   c_t = 1 + coef ln(floor((p_t + 1) / every) + 1)     (a query temperature)
//   s_m,j = cap tanh((q_m . k_m,j) scale / cap),   a_m = sum_j softmax(s_m)_j v_j,   m = 1, 2
//   o = a_1 - lambda a_2;   o <- o / sqrt(mean(o^2) + eps) (1 - diff)
//
// The cache keeps a key head of D channels per (key/value head, map), head 2 g + m, and one value
// head of E channels per key/value head g: both maps read the same values.
// The plain kernel: one wave per (token, query head), keys in tiles of 64 aligned to absolute
// positions with a running maximum and sum per map, so the order of every sum follows from the
// token's position alone.  Everything float.  ``zk_cache_store`` copies a step's keys and values
// as projected (no norm, no rotation) to their slots.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

#define DA_MAX 256

__device__ __forceinline__ float query_temperature(int pos, float coef, int every) {
  return every > 0 ? 1.0f + coef * logf((float)((pos + 1) / every + 1)) : 1.0f;
}

__global__ __launch_bounds__(256) void cache_store_kernel(const act_t* __restrict__ rows, int ld, int k_off, int v_off,
                                                          const int* __restrict__ slot_map, act_t* __restrict__ kcache,
                                                          act_t* __restrict__ vcache, int nk, int hd, int nv, int vd, int bs,
                                                          int v_transposed, act_t* __restrict__ q, int q_width,
                                                          const int* __restrict__ positions, float coef, int every) {
  const int t = blockIdx.x;
  if (q != nullptr) {
    // the queries of the row times the temperature of its position, in place
    const int pos = positions[t];
    const float c = pos >= 0 ? query_temperature(pos, coef, every) : 1.0f;
    if (c != 1.0f) {
      act_t* qr = q + (size_t)t * ld;
      for (int i = threadIdx.x; i < q_width; i += blockDim.x) qr[i] = from_f32<act_t>(to_f32(qr[i]) * c);
    }
  }
  const int slot = slot_map[t];
  if (slot < 0) return;
  const size_t page = slot / bs, off = slot % bs;
  const act_t* row = rows + (size_t)t * ld;
  for (int i = threadIdx.x; i < nk * hd; i += blockDim.x) {
    const int g = i / hd, d = i % hd;
    kcache[((page * nk + g) * bs + off) * hd + d] = row[k_off + i];
  }
  for (int i = threadIdx.x; i < nv * vd; i += blockDim.x) {
    const int g = i / vd, d = i % vd;
    if (v_transposed) vcache[(page * nv + g) * (size_t)vd * bs + (size_t)d * bs + off] = row[v_off + i];
    else vcache[((page * nv + g) * bs + off) * vd + d] = row[v_off + i];
  }
}

__global__ __launch_bounds__(64) void diff_attention_plain_kernel(
    const act_t* __restrict__ q, int q_stride, const act_t* __restrict__ kcache, const act_t* __restrict__ vcache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ req_of_token,
    const int* __restrict__ positions, act_t* __restrict__ out, int nh, int nkv, int D, int E, int bs, float scale,
    float softcap, int window, int v_transposed, float lambda, float diff, float eps, float coef, int every) {
  __shared__ float sq[2 * DA_MAX];
  __shared__ float sp[2][64];
  __shared__ int spage[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  act_t* o = out + ((size_t)t * nh + h) * E;
  if (pos < 0) {  // padding row
    for (int d = lane; d < E; d += 64) o[d] = from_f32<act_t>(0.f);
    return;
  }
  const int r = req_of_token[t];
  const int kvh = h / (nh / nkv);
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int* table = block_table + (size_t)r * max_blocks;
  const act_t* qr = q + (size_t)t * q_stride + (size_t)h * 2 * D;
  const float temp = query_temperature(pos, coef, every);
  for (int d = lane; d < 2 * D; d += 64) sq[d] = to_f32(qr[d]) * temp;
  __syncthreads();

  float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
  float acc[2][DA_MAX / 64] = {};
  for (int j0 = (lo / 64) * 64; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j >= lo && j <= pos;
    float s[2] = {-INFINITY, -INFINITY};
    int page = -1;
    if (valid) {
      page = table[j / bs];
#pragma unroll
      for (int mp = 0; mp < 2; mp++) {
        const act_t* kr = kcache + (((size_t)page * 2 * nkv + 2 * kvh + mp) * bs + (j % bs)) * D;
        float dot = 0.f;
        for (int d = 0; d < D; d++) dot = fmaf(sq[mp * D + d], to_f32(kr[d]), dot);
        float x = dot * scale;
        if (softcap > 0.f) x = softcap * tanhf(x / softcap);
        s[mp] = x;
      }
    }
    float corr[2];
    __syncthreads();
#pragma unroll
    for (int mp = 0; mp < 2; mp++) {
      const float m_new = fmaxf(m[mp], wave_max(s[mp]));
      const float p = valid ? expf(s[mp] - m_new) : 0.f;
      corr[mp] = expf(m[mp] - m_new);
      l[mp] = l[mp] * corr[mp] + wave_sum(p);
      m[mp] = m_new;
      sp[mp][lane] = p;
    }
    spage[lane] = page;
    __syncthreads();
#pragma unroll
    for (int c = 0; c < DA_MAX / 64; c++) {
      const int d = lane + c * 64;
      if (d < E) {
        float a0 = acc[0][c] * corr[0], a1 = acc[1][c] * corr[1];
        for (int jj = 0; jj < 64; jj++) {
          const int pg = spage[jj];
          if (pg < 0) continue;
          const size_t off = (j0 + jj) % bs;
          const size_t head_base = ((size_t)pg * nkv + kvh) * bs * E;
          const float v = to_f32(v_transposed ? vcache[head_base + (size_t)d * bs + off] : vcache[head_base + off * E + d]);
          a0 = fmaf(sp[0][jj], v, a0);
          a1 = fmaf(sp[1][jj], v, a1);
        }
        acc[0][c] = a0;
        acc[1][c] = a1;
      }
    }
  }
  const float inv0 = 1.f / l[0], inv1 = 1.f / l[1];
  float ss = 0.f;
  float res[DA_MAX / 64];
#pragma unroll
  for (int c = 0; c < DA_MAX / 64; c++) {
    const int d = lane + c * 64;
    res[c] = d < E ? acc[0][c] * inv0 - lambda * (acc[1][c] * inv1) : 0.f;
    ss = fmaf(res[c], res[c], ss);
  }
  ss = wave_sum(ss);
  const float norm = (1.0f - diff) / sqrtf(ss / (float)E + eps);
#pragma unroll
  for (int c = 0; c < DA_MAX / 64; c++) {
    const int d = lane + c * 64;
    if (d < E) o[d] = from_f32<act_t>(res[c] * norm);
  }
}

// q rows times the temperature of their positions, in place (for an attention kernel that takes
// its queries as they lie)
__global__ void query_temperature_kernel(act_t* __restrict__ q, int ld, int width, const int* __restrict__ positions,
                                         float coef, int every) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const float c = query_temperature(pos, coef, every);
  if (c == 1.0f) return;
  act_t* row = q + (size_t)t * ld;
  for (int i = threadIdx.x; i < width; i += blockDim.x) row[i] = from_f32<act_t>(to_f32(row[i]) * c);
}

// Joins two maps' outputs that an ordinary attention kernel computed as heads of their own:
// a: [T, nh, 2, E] (map 1 then map 2 of each head) -> out [T, nh, E].
__global__ __launch_bounds__(64) void diff_join_kernel(const act_t* __restrict__ a, act_t* __restrict__ out, int E,
                                                       float lambda, float diff, float eps) {
  const size_t row = (size_t)blockIdx.x * gridDim.y + blockIdx.y;
  const act_t* a1 = a + row * 2 * E;
  const act_t* a2 = a1 + E;
  float res[DA_MAX / 64];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < DA_MAX / 64; c++) {
    const int d = threadIdx.x + c * 64;
    res[c] = d < E ? to_f32(a1[d]) - lambda * to_f32(a2[d]) : 0.f;
    ss = fmaf(res[c], res[c], ss);
  }
  ss = wave_sum(ss);
  const float norm = (1.0f - diff) / sqrtf(ss / (float)E + eps);
#pragma unroll
  for (int c = 0; c < DA_MAX / 64; c++) {
    const int d = threadIdx.x + c * 64;
    if (d < E) out[row * E + d] = from_f32<act_t>(res[c] * norm);
  }
}

extern "C" {

// rows: [T, ld]; a row's nk key heads of hd begin at column k_off, its nv value heads of vd at v_off.
// kcache: [pages, nk, bs, hd]; vcache: [pages, nv, bs, vd], or [pages, nv, vd, bs] when v_transposed.
int zk_cache_store(const void* rows, int ld, int k_off, int v_off, const int* slot_map, void* kcache, void* vcache, int T,
                   int nk, int hd, int nv, int vd, int bs, int v_transposed, void* stream) {
  ZK_REQUIRE(T >= 0 && nk > 0 && nv > 0 && hd > 0 && vd > 0 && bs > 0 && slot_map != nullptr && kcache != nullptr && vcache != nullptr,
             "zk_cache_store: bad arguments");
  ZK_REQUIRE(k_off >= 0 && v_off >= 0 && ld >= k_off + nk * hd && ld >= v_off + nv * vd, "zk_cache_store: rows shorter than their heads");
  if (T == 0) return 0;
  cache_store_kernel<<<T, 256, 0, (hipStream_t)stream>>>((const act_t*)rows, ld, k_off, v_off, slot_map, (act_t*)kcache,
                                                        (act_t*)vcache, nk, hd, nv, vd, bs, v_transposed, nullptr, 0, nullptr,
                                                        0.f, 0);
  return zk_launch_status("zk_cache_store");
}

// The same, and the first q_width columns of every row (the queries) times the temperature of the
// row's position, 1 + coef ln(floor((p + 1) / every) + 1), in place: one launch for both.
int zk_cache_store_temperature(void* rows, int ld, int q_width, int k_off, int v_off, const int* positions,
                               const int* slot_map, void* kcache, void* vcache, int T, int nk, int hd, int nv, int vd, int bs,
                               int v_transposed, float coef, int every, void* stream) {
  ZK_REQUIRE(T >= 0 && nk > 0 && nv > 0 && hd > 0 && vd > 0 && bs > 0 && slot_map != nullptr && kcache != nullptr && vcache != nullptr,
             "zk_cache_store: bad arguments");
  ZK_REQUIRE(k_off >= q_width && v_off >= q_width && ld >= k_off + nk * hd && ld >= v_off + nv * vd && q_width > 0 && every > 0 &&
             positions != nullptr, "zk_cache_store: rows shorter than their heads, or queries that overlap them");
  if (T == 0) return 0;
  cache_store_kernel<<<T, 256, 0, (hipStream_t)stream>>>((const act_t*)rows, ld, k_off, v_off, slot_map, (act_t*)kcache,
                                                        (act_t*)vcache, nk, hd, nv, vd, bs, v_transposed, (act_t*)rows, q_width,
                                                        positions, coef, every);
  return zk_launch_status("zk_cache_store");
}

// q: rows q_stride apart, nh heads of [map 1 | map 2], D channels each; the cache holds 2 nkv key
// heads of D channels (head 2 g + m: map m of key/value head g) and nkv value heads of E; out: [T, nh, E].  softcap <= 0: none; window <= 0: every earlier
// key; every <= 0: no query temperature.
int zk_diff_attention_plain(const void* q, int q_stride, const void* kcache, const void* vcache, const int* block_table,
                            int max_blocks, const int* req_of_token, const int* positions, void* out, int T, int nh,
                            int nkv, int D, int E, int bs, float scale, float softcap, int window, int v_transposed,
                            float lambda, float diff, float eps, float coef, int every, void* stream) {
  ZK_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && D > 0 && E > 0 && bs > 0 && max_blocks > 0, "zk_diff_attention_plain: bad sizes");
  ZK_REQUIRE(D <= DA_MAX && E <= DA_MAX, "zk_diff_attention_plain: heads of more than 256 channels are not supported");
  ZK_REQUIRE(nh % nkv == 0 && nh <= 65535, "zk_diff_attention_plain: heads must be a multiple of kv heads");
  ZK_REQUIRE(q_stride >= nh * 2 * D, "zk_diff_attention_plain: q row stride too small");
  if (T == 0) return 0;
  dim3 grid(T, nh);
  diff_attention_plain_kernel<<<grid, 64, 0, (hipStream_t)stream>>>(
      (const act_t*)q, q_stride, (const act_t*)kcache, (const act_t*)vcache, block_table, max_blocks, req_of_token,
      positions, (act_t*)out, nh, nkv, D, E, bs, scale, softcap, window, v_transposed, lambda, diff, eps, coef, every);
  return zk_launch_status("zk_diff_attention_plain");
}

// q: [T, ld], of which the first ``width`` columns are multiplied by 1 + coef ln(floor((p + 1) / every) + 1).
int zk_query_temperature(void* q, int ld, int width, const int* positions, int T, float coef, int every, void* stream) {
  ZK_REQUIRE(T >= 0 && width > 0 && ld >= width && every > 0, "zk_query_temperature: bad sizes");
  if (T == 0) return 0;
  query_temperature_kernel<<<T, 256, 0, (hipStream_t)stream>>>((act_t*)q, ld, width, positions, coef, every);
  return zk_launch_status("zk_query_temperature");
}

// a: [T, nh, 2, E] -> out [T, nh, E]: a1 - lambda a2, unit RMS over E, times (1 - diff).
int zk_diff_join(const void* a, void* out, int T, int nh, int E, float lambda, float diff, float eps, void* stream) {
  ZK_REQUIRE(T >= 0 && nh > 0 && nh <= 65535 && E > 0 && E <= DA_MAX, "zk_diff_join: bad sizes");
  if (T == 0) return 0;
  dim3 grid(T, nh);
  diff_join_kernel<<<grid, 64, 0, (hipStream_t)stream>>>((const act_t*)a, (act_t*)out, E, lambda, diff, eps);
  return zk_launch_status("zk_diff_join");
}

}  // extern "C"

ZK_ENTER(zk_cache_store)
ZK_ENTER(zk_cache_store_temperature)
ZK_ENTER(zk_diff_attention_plain)
ZK_ENTER(zk_diff_join)
ZK_ENTER(zk_query_temperature)
