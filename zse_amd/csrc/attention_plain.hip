// Plain paged attention: one wave per (token, query head), every token of the
// step alike, whether it is a decoded token or one of a prompt portion.  Keys
// and values come only from the cache, through the request's block table.
//
//   s_j = softcap((q . k_j) * scale),   j in [lo, pos],  lo = max(0, pos - window + 1)
//   o   = sum_j softmax(s)_j v_j
//
// With ``chunk`` instead of a window, lo = floor(pos / chunk) * chunk: a query sees the keys of
// its own chunk of positions, counted from position 0.  ``unit_sink``: a sink of score 0 that has
// no value joins the denominator, exp(s_j) / (1 + sum exp(s)).
//
// Keys are visited in tiles of 64 aligned to absolute positions, with a
// running maximum and sum, so the order of every sum depends on the token's
// position alone, not on how the step was cut.  Scores, softmax and the output
// sum are float.  The reference's decode kernel has the same shape of work
// (orchestrator/kernels.py:524-671: one block per (sequence, head), block
// table walk, three passes in shared memory); its prefill kernel reads
// contiguous K/V instead (:859-958) and never applies a window (:883).
#include "common.h"

#define AP_MAX_HD 256

// MAXD: the most channels a head's queries, keys and values have (256, or 1024 for the wide rows
// of a latent cache).  sinks (may be null): float [nh], exp(sink) joins a head's denominator with
// no key and no value.  v_in_k: a value is the first vd channels of its key (no value cache).
template <int MAXD>
__global__ __launch_bounds__(64) void attention_plain_kernel(
    const act_t* __restrict__ q, int q_stride, const act_t* __restrict__ kcache,
    const act_t* __restrict__ vcache, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ req_of_token, const int* __restrict__ positions,
    act_t* __restrict__ out, int nh, int nkv, int hd, int vd, int bs, float scale, float softcap,
    int window, int v_transposed, const float* __restrict__ v_freq, int v_interleaved,
    const float* __restrict__ sinks, int v_in_k, int chunk, int unit_sink) {
  __shared__ float sq[MAXD];
  __shared__ float sp[64];
  __shared__ int spage[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  act_t* o = out + ((size_t)t * nh + h) * vd;
  if (pos < 0) {  // padding row
    for (int d = lane; d < vd; d += 64) o[d] = from_f32<act_t>(0.f);
    return;
  }
  const int r = req_of_token[t];
  const int kvh = h / (nh / nkv);
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : chunk > 0 ? pos / chunk * chunk : 0;
  const int* table = block_table + (size_t)r * max_blocks;
  const act_t* qr = q + (size_t)t * q_stride + (size_t)h * hd;
  for (int d = lane; d < hd; d += 64) sq[d] = to_f32(qr[d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[MAXD / 64] = {};
  for (int j0 = (lo / 64) * 64; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j >= lo && j <= pos;
    float s = -INFINITY;
    int page = -1;
    if (valid) {
      page = table[j / bs];
      const act_t* kr = kcache + (((size_t)page * nkv + kvh) * bs + (j % bs)) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; d++) dot = fmaf(sq[d], to_f32(kr[d]), dot);
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf on the first tile: exp(-inf) = 0
    l = l * corr + wave_sum(p);
    m = m_new;
    __syncthreads();
    sp[lane] = p;
    spage[lane] = page;
    __syncthreads();
#pragma unroll
    for (int c = 0; c < MAXD / 64; c++) {
      const int d = lane + c * 64;
      if (d < vd) {
        float a = acc[c] * corr;
        for (int jj = 0; jj < 64; jj++) {
          const int pg = spage[jj];
          if (pg < 0) continue;
          const size_t off = (j0 + jj) % bs;
          act_t v;
          if (v_in_k) {
            v = kcache[(((size_t)pg * nkv + kvh) * bs + off) * hd + d];
          } else {
            const size_t head_base = ((size_t)pg * nkv + kvh) * bs * vd;
            v = v_transposed ? vcache[head_base + (size_t)d * bs + off] : vcache[head_base + off * vd + d];
          }
          a = fmaf(sp[jj], to_f32(v), a);
        }
        acc[c] = a;
      }
    }
  }
  if (sinks != nullptr || unit_sink) {
    const float sk = sinks != nullptr ? sinks[h] : 0.f;
    const float m_new = fmaxf(m, sk);
    const float corr = expf(m - m_new);
    l = l * corr + expf(sk - m_new);
#pragma unroll
    for (int c = 0; c < MAXD / 64; c++) acc[c] *= corr;
  }
  const float inv = 1.f / l;
  if (v_freq == nullptr) {
#pragma unroll
    for (int c = 0; c < MAXD / 64; c++) {
      const int d = lane + c * 64;
      if (d < vd) o[d] = from_f32<act_t>(acc[c] * inv);
    }
    return;
  }
  // values were turned by their own positions when they were stored: the sum is turned back
  // by the query's position, pair m by -pos * v_freq[m]
  __syncthreads();
#pragma unroll
  for (int c = 0; c < MAXD / 64; c++) {
    const int d = lane + c * 64;
    if (d < vd) sq[d] = acc[c] * inv;
  }
  __syncthreads();
  const int half = vd / 2;
  for (int m2 = lane; m2 < half; m2 += 64) {
    float sn, cs, ra, rb;
    sincosf(-(float)pos * v_freq[m2], &sn, &cs);
    const int ia = v_interleaved ? 2 * m2 : m2, ib = v_interleaved ? 2 * m2 + 1 : m2 + half;
    rotate_pair(sq[ia], sq[ib], sn, cs, ra, rb);
    o[ia] = from_f32<act_t>(ra);
    o[ib] = from_f32<act_t>(rb);
  }
}

// softcap <= 0: no cap; window <= 0: every earlier key is visible.  v_transposed: V is
// cached as [page][kv head][hd][bs] instead of [page][kv head][bs][hd].
// hd: the size of a head's queries and keys; vd: of its values (the output's too).  v_freq (may
// be null): float [vd / 2], values are cached turned by their positions and the output is turned back.
// sinks (may be null): float [nh].  v_in_k: values are the first vd channels of the keys.
// chunk > 0 (without a window): a query sees the keys of its own chunk of positions only.
// unit_sink: a sink of score 0 joins every head's denominator (not together with sinks).
extern "C" int zk_attention_plain_masked(const void* q, int q_stride, const void* kcache, const void* vcache,
                                         const int* block_table, int max_blocks, const int* req_of_token,
                                         const int* positions, void* out, int T, int nh, int nkv, int hd, int vd,
                                         int bs, float scale, float softcap, int window, int v_transposed,
                                         const float* v_freq, int v_interleaved, const float* sinks, int v_in_k,
                                         int chunk, int unit_sink, void* stream) {
  ZK_REQUIRE(chunk >= 0 && (chunk == 0 || window <= 0), "zk_attention_plain: a chunk or a window, not both");
  ZK_REQUIRE(!unit_sink || sinks == nullptr, "zk_attention_plain: a unit sink or learned sinks, not both");
  ZK_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && hd > 0 && vd > 0 && bs > 0 && max_blocks > 0,
             "zk_attention_plain: bad sizes");
  ZK_REQUIRE(vd <= 1024 && (v_freq == nullptr || vd % 2 == 0), "zk_attention_plain: value size above 1024, or odd with a rotation");
  ZK_REQUIRE(nh % nkv == 0, "zk_attention_plain: heads must be a multiple of kv heads");
  ZK_REQUIRE(hd <= 1024, "zk_attention_plain: head_dim above 1024 is not supported");
  ZK_REQUIRE(nh <= 65535, "zk_attention_plain: too many heads");
  ZK_REQUIRE(q_stride >= nh * hd, "zk_attention_plain: q row stride too small");
  ZK_REQUIRE(!v_in_k || (vd <= hd && !v_transposed), "zk_attention_plain: values inside keys are no wider than the keys");
  if (T == 0) return 0;
  dim3 grid(T, nh);
  if (hd <= AP_MAX_HD && vd <= AP_MAX_HD)
    attention_plain_kernel<AP_MAX_HD><<<grid, 64, 0, (hipStream_t)stream>>>(
        (const act_t*)q, q_stride, (const act_t*)kcache, (const act_t*)vcache, block_table, max_blocks,
        req_of_token, positions, (act_t*)out, nh, nkv, hd, vd, bs, scale, softcap, window, v_transposed, v_freq,
        v_interleaved, sinks, v_in_k, chunk, unit_sink);
  else
    attention_plain_kernel<1024><<<grid, 64, 0, (hipStream_t)stream>>>(
        (const act_t*)q, q_stride, (const act_t*)kcache, (const act_t*)vcache, block_table, max_blocks,
        req_of_token, positions, (act_t*)out, nh, nkv, hd, vd, bs, scale, softcap, window, v_transposed, v_freq,
        v_interleaved, sinks, v_in_k, chunk, unit_sink);
  return zk_launch_status("zk_attention_plain");
}

extern "C" int zk_attention_plain_sink(const void* q, int q_stride, const void* kcache, const void* vcache,
                                       const int* block_table, int max_blocks, const int* req_of_token,
                                       const int* positions, void* out, int T, int nh, int nkv, int hd, int vd,
                                       int bs, float scale, float softcap, int window, int v_transposed,
                                       const float* v_freq, int v_interleaved, const float* sinks, int v_in_k,
                                       void* stream) {
  return zk_attention_plain_masked(q, q_stride, kcache, vcache, block_table, max_blocks, req_of_token, positions, out, T,
                                   nh, nkv, hd, vd, bs, scale, softcap, window, v_transposed, v_freq, v_interleaved,
                                   sinks, v_in_k, 0, 0, stream);
}

extern "C" int zk_attention_plain_ext(const void* q, int q_stride, const void* kcache, const void* vcache,
                                      const int* block_table, int max_blocks, const int* req_of_token,
                                      const int* positions, void* out, int T, int nh, int nkv, int hd, int vd,
                                      int bs, float scale, float softcap, int window, int v_transposed,
                                      const float* v_freq, int v_interleaved, void* stream) {
  ZK_REQUIRE(hd <= AP_MAX_HD && vd <= AP_MAX_HD, "zk_attention_plain: head_dim above 256 is not supported");
  return zk_attention_plain_sink(q, q_stride, kcache, vcache, block_table, max_blocks, req_of_token, positions, out, T,
                                 nh, nkv, hd, vd, bs, scale, softcap, window, v_transposed, v_freq, v_interleaved,
                                 nullptr, 0, stream);
}

extern "C" int zk_attention_plain(const void* q, int q_stride, const void* kcache, const void* vcache,
                                  const int* block_table, int max_blocks, const int* req_of_token,
                                  const int* positions, void* out, int T, int nh, int nkv, int hd,
                                  int bs, float scale, float softcap, int window, int v_transposed,
                                  void* stream) {
  return zk_attention_plain_ext(q, q_stride, kcache, vcache, block_table, max_blocks, req_of_token, positions, out, T,
                                nh, nkv, hd, hd, bs, scale, softcap, window, v_transposed, nullptr, 0, stream);
}

#include "packed_call.h"
extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
static const int attention_plain_sink_entered = zk_steplist_register(
    "zk_attention_plain_sink", zk_packed::Call<zk_attention_plain_sink>::nargs,
    (void*)zk_packed::Call<zk_attention_plain_sink>::call);
static const int attention_plain_masked_entered = zk_steplist_register(
    "zk_attention_plain_masked", zk_packed::Call<zk_attention_plain_masked>::nargs,
    (void*)zk_packed::Call<zk_attention_plain_masked>::call);
static const int attention_plain_ext_entered = zk_steplist_register(
    "zk_attention_plain_ext", zk_packed::Call<zk_attention_plain_ext>::nargs,
    (void*)zk_packed::Call<zk_attention_plain_ext>::call);
