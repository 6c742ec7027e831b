// What happens to a step's queries, keys and values between their product and the attention:
// an optional norm over each query and key head, an optional number per query head, the rotary
// encoding of queries and keys, an optional rotation of the values, and the store of keys and
// values into the paged cache.  One wave per (token, head).
//
//   q_h <- rot_p( q_h / sqrt(mean(q_h^2) + eps) * gq ) * c_h          (k likewise with gk, no c)
//   v_g <- rot'_p( v_g )
//
// rot_p turns pair (i, i + dims/2) of the first ``dims`` channels by p * inv_freq[i]; rot'_p turns
// pair m of all value channels ((m, m + E/2), or (2m, 2m + 1) when interleaved) by p * v_freq[m].
// A row of the input holds nh query heads of D, then nkv key heads of D, then nkv value heads of
// E (the last two absent when the mixer reads another one's cache).  All arithmetic is float; a
// value is rounded to the activation type once, when it is stored.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);

#define HP_MAX 256

__global__ __launch_bounds__(64) void head_prep_kernel(
    act_t* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ slot_map,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, const float* __restrict__ head_scale, float eps,
    const float* __restrict__ inv_freq, int rot_dims, const float* __restrict__ v_freq, int v_interleaved,
    act_t* __restrict__ kcache, act_t* __restrict__ vcache, int nh, int nkv, int D, int E, int bs, int v_transposed,
    const float* __restrict__ bias, float rot_scale, int qk_interleaved, int ld, int unit_norm) {
  __shared__ float buf[HP_MAX];
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;                                   // a padding row
  // ld: the distance between rows where they hold more than the heads (0: just the heads)
  const size_t width = ld > 0 ? (size_t)ld : (size_t)(nh + nkv) * D + (size_t)nkv * E;
  const int kind = head < nh ? 0 : head < nh + nkv ? 1 : 2;
  const int size = kind == 2 ? E : D;
  const size_t at = (size_t)t * width + (kind == 2 ? (size_t)(nh + nkv) * D + (size_t)(head - nh - nkv) * E : (size_t)head * D);
  const int slot = (kind != 0 && slot_map) ? slot_map[t] : -1;
  if (kind != 0 && slot < 0) return;
  float sum = 0.f;
  for (int d = lane; d < size; d += 64) {
    float x = to_f32(qkv[at + d]);
    if (bias) x += bias[at - (size_t)t * width + d];
    buf[d] = x;
    sum = fmaf(x, x, sum);
  }
  const float* gain = kind == 0 ? q_gain : kind == 1 ? k_gain : nullptr;
  if (gain != nullptr) {
    sum = wave_sum(sum);
    const float inv = 1.0f / sqrtf(sum / (float)size + eps);
    const float c = (kind == 0 && head_scale) ? head_scale[head] : 1.f;
    for (int d = lane; d < size; d += 64) buf[d] = buf[d] * inv * gain[d] * c;
  } else if (kind == 0 && head_scale) {
    const float c = head_scale[head];
    for (int d = lane; d < size; d += 64) buf[d] *= c;
  }
  __syncthreads();
  // rotation: every lane takes whole pairs, so nothing is read after another lane wrote it
  const float* freq = kind == 2 ? v_freq : inv_freq;
  const int dims = kind == 2 ? (v_freq ? E : 0) : (inv_freq ? rot_dims : 0);
  const bool inter = kind == 2 ? v_interleaved : qk_interleaved;
  const float mag = kind == 2 ? 1.0f : rot_scale;
  const int half = dims / 2;
  for (int m = lane; m < half; m += 64) {
    float sn, cs, ra, rb;
    sincosf((float)pos * freq[m], &sn, &cs);
    if (mag != 1.0f) {
      sn *= mag;
      cs *= mag;
    }
    const int ia = inter ? 2 * m : m, ib = inter ? 2 * m + 1 : m + half;
    rotate_pair(buf[ia], buf[ib], sn, cs, ra, rb);
    buf[ia] = ra;
    buf[ib] = rb;
  }
  __syncthreads();
  if (unit_norm && kind != 2) {
    // queries and keys divided by their root mean square over the head, after the rotation, no gain
    float ss = 0.f;
    for (int d = lane; d < size; d += 64) ss = fmaf(buf[d], buf[d], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)size + eps);
    for (int d = lane; d < size; d += 64) buf[d] *= inv;
  }
  if (kind == 0) {
    for (int d = lane; d < size; d += 64) qkv[at + d] = from_f32<act_t>(buf[d]);
    return;
  }
  const size_t page = slot / bs, off = slot % bs;
  if (kind == 1) {
    act_t* dst = kcache + ((page * nkv + (head - nh)) * bs + off) * D;
    for (int d = lane; d < size; d += 64) dst[d] = from_f32<act_t>(buf[d]);
  } else if (v_transposed) {
    act_t* dst = vcache + (page * nkv + (head - nh - nkv)) * (size_t)E * bs + off;
    for (int d = lane; d < size; d += 64) dst[(size_t)d * bs] = from_f32<act_t>(buf[d]);
  } else {
    act_t* dst = vcache + ((page * nkv + (head - nh - nkv)) * bs + off) * E;
    for (int d = lane; d < size; d += 64) dst[d] = from_f32<act_t>(buf[d]);
  }
}

// nkv: key/value heads held in the rows (0 for a mixer that stores none).  q_gain, k_gain,
// head_scale, inv_freq, v_freq may each be null (the step it stands for is then left out).
// bias (may be null): float, one per channel of a row, added before anything else.  rot_scale:
// multiplies the sines and cosines of queries and keys.  qk_interleaved: their pairs are
// (2i, 2i + 1) instead of (i, i + rot_dims / 2).
// ld: the distance between rows of qkv in elements where a row holds more than the heads (0: the
// heads alone).  unit_norm: queries and keys are divided by their root mean square over the head
// (with eps), after the rotation and without a gain.
extern "C" int zk_head_prep_unit(void* qkv, const int* positions, const int* slot_map, const float* q_gain,
                                 const float* k_gain, const float* head_scale, float eps, const float* inv_freq,
                                 int rot_dims, const float* v_freq, int v_interleaved, void* kcache, void* vcache, int T,
                                 int nh, int nkv, int D, int E, int bs, int v_transposed, const float* bias,
                                 float rot_scale, int qk_interleaved, int ld, int unit_norm, void* stream) {
  ZK_REQUIRE(ld == 0 || ld >= (nh + nkv) * D + nkv * E, "zk_head_prep: rows shorter than their heads");
  ZK_REQUIRE(T >= 0 && nh > 0 && nkv >= 0 && D > 0 && E > 0 && bs > 0, "zk_head_prep: bad sizes");
  ZK_REQUIRE(D <= HP_MAX && E <= HP_MAX, "zk_head_prep: heads of more than 256 channels are not supported");
  ZK_REQUIRE(inv_freq == nullptr || (rot_dims % 2 == 0 && rot_dims >= 0 && rot_dims <= D),
             "zk_head_prep: the rotated channels must be even in number and at most the head's");
  ZK_REQUIRE(v_freq == nullptr || E % 2 == 0, "zk_head_prep: rotated values need an even size");
  ZK_REQUIRE(nkv == 0 || (kcache != nullptr && vcache != nullptr && slot_map != nullptr), "zk_head_prep: no cache to store into");
  ZK_REQUIRE(nh + 2 * nkv <= 65535, "zk_head_prep: too many heads");
  if (T == 0) return 0;
  dim3 grid(T, nh + 2 * nkv);
  head_prep_kernel<<<grid, 64, 0, (hipStream_t)stream>>>((act_t*)qkv, positions, slot_map, q_gain, k_gain, head_scale, eps,
                                                         inv_freq, rot_dims, v_freq, v_interleaved, (act_t*)kcache,
                                                         (act_t*)vcache, nh, nkv, D, E, bs, v_transposed, bias, rot_scale,
                                                         qk_interleaved, ld, unit_norm);
  return zk_launch_status("zk_head_prep");
}

extern "C" int zk_head_prep_ext(void* qkv, const int* positions, const int* slot_map, const float* q_gain,
                                const float* k_gain, const float* head_scale, float eps, const float* inv_freq,
                                int rot_dims, const float* v_freq, int v_interleaved, void* kcache, void* vcache, int T,
                                int nh, int nkv, int D, int E, int bs, int v_transposed, const float* bias,
                                float rot_scale, int qk_interleaved, void* stream) {
  return zk_head_prep_unit(qkv, positions, slot_map, q_gain, k_gain, head_scale, eps, inv_freq, rot_dims, v_freq,
                           v_interleaved, kcache, vcache, T, nh, nkv, D, E, bs, v_transposed, bias, rot_scale,
                           qk_interleaved, 0, 0, stream);
}

extern "C" int zk_head_prep(void* qkv, const int* positions, const int* slot_map, const float* q_gain,
                            const float* k_gain, const float* head_scale, float eps, const float* inv_freq,
                            int rot_dims, const float* v_freq, int v_interleaved, void* kcache, void* vcache, int T,
                            int nh, int nkv, int D, int E, int bs, int v_transposed, void* stream) {
  return zk_head_prep_ext(qkv, positions, slot_map, q_gain, k_gain, head_scale, eps, inv_freq, rot_dims, v_freq,
                          v_interleaved, kcache, vcache, T, nh, nkv, D, E, bs, v_transposed, nullptr, 1.0f, 0, stream);
}

// Queries and keys whose norm runs over the whole row of heads, and values that are the keys.
//
//   q <- rot_p( (q + bq) / sqrt(mean over all nh D channels + eps) * gq ),   gq of nh D numbers
//   k <- rot_p( (k + bk) / sqrt(mean over all nkv D channels + eps) * gk )
//   v  = k + bk as projected (before norm and rotation), where ``values_are_keys``
//
// One block per token: a row holds nh query heads, then nkv key heads of D (and, without
// values_are_keys, nkv value heads of E that are stored as they are).  Float throughout, one
// rounding at the store.  In the 32-bit library the block is 256 wide whatever the step, so a row's
// sums do not depend on what else the step holds; in bfloat16 steps of up to 64 rows take 1,024 threads a row.
__global__ __launch_bounds__(1024) void row_prep_kernel(
    act_t* __restrict__ qk, int ld, const int* __restrict__ positions, const int* __restrict__ slot_map,
    const float* __restrict__ bias, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ inv_freq, int rot_dims, act_t* __restrict__ kcache, act_t* __restrict__ vcache, int nh,
    int nkv, int D, int E, int bs, int v_transposed, int values_are_keys) {
  extern __shared__ float row[];                 // [(nh + nkv) D]
  __shared__ float red[17];
  const int t = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int nq = nh * D, nk = nkv * D;
  act_t* src = qk + (size_t)t * ld;
  float sq = 0.f, sk = 0.f;
  for (int i = tid; i < nq + nk; i += nt) {
    float x = to_f32(src[i]);
    if (bias) x += bias[i];
    row[i] = x;
    if (i < nq) sq = fmaf(x, x, sq);
    else sk = fmaf(x, x, sk);
  }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  const int slot = slot_map ? slot_map[t] : -1;
  const size_t page = slot >= 0 ? slot / bs : 0, off = slot >= 0 ? slot % bs : 0;
  if (slot >= 0) {
    // the values: the keys before norm and rotation, or the row's own value heads
    const int nv = nkv * E;
    for (int i = tid; i < nv; i += nt) {
      const int g = i / E, d = i % E;
      float x;
      if (values_are_keys) x = row[nq + i];
      else {
        x = to_f32(src[nq + nk + i]);
        if (bias) x += bias[nq + nk + i];
      }
      if (v_transposed) vcache[(page * nkv + g) * (size_t)E * bs + (size_t)d * bs + off] = from_f32<act_t>(x);
      else vcache[((page * nkv + g) * bs + off) * E + d] = from_f32<act_t>(x);
    }
  }
  __syncthreads();
  if (q_gain) {
    const float inv = 1.0f / sqrtf(sq / (float)nq + eps);
    for (int i = tid; i < nq; i += nt) row[i] = row[i] * inv * q_gain[i];
  }
  if (k_gain) {
    const float inv = 1.0f / sqrtf(sk / (float)nk + eps);
    for (int i = tid; i < nk; i += nt) row[nq + i] = row[nq + i] * inv * k_gain[i];
  }
  __syncthreads();
  if (inv_freq) {
    const int half = rot_dims / 2;
    for (int i = tid; i < (nh + nkv) * half; i += nt) {
      const int head = i / half, m = i % half;
      float sn, cs, ra, rb;
      sincosf((float)pos * inv_freq[m], &sn, &cs);
      float* hp = row + head * D;
      rotate_pair(hp[m], hp[m + half], sn, cs, ra, rb);
      hp[m] = ra;
      hp[m + half] = rb;
    }
    __syncthreads();
  }
  for (int i = tid; i < nq; i += nt) src[i] = from_f32<act_t>(row[i]);
  if (slot >= 0)
    for (int i = tid; i < nk; i += nt) {
      const int g = i / D, d = i % D;
      kcache[((page * nkv + g) * bs + off) * D + d] = from_f32<act_t>(row[nq + i]);
    }
}

// qk: [T, ld], changed in place (the queries) and stored (keys, values).  bias (may be null): one
// float per channel of a row.  q_gain [nh D], k_gain [nkv D] (either may be null: no norm).
// values_are_keys: E == D and a row holds no value heads.
extern "C" int zk_row_prep(void* qk, int ld, const int* positions, const int* slot_map, const float* bias,
                           const float* q_gain, const float* k_gain, float eps, const float* inv_freq, int rot_dims,
                           void* kcache, void* vcache, int T, int nh, int nkv, int D, int E, int bs, int v_transposed,
                           int values_are_keys, void* stream) {
  ZK_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && D > 0 && E > 0 && bs > 0, "zk_row_prep: bad sizes");
  ZK_REQUIRE(!values_are_keys || E == D, "zk_row_prep: values that are keys have the keys' size");
  ZK_REQUIRE(ld >= (nh + nkv) * D + (values_are_keys ? 0 : nkv * E), "zk_row_prep: rows shorter than their heads");
  ZK_REQUIRE(inv_freq == nullptr || (rot_dims % 2 == 0 && rot_dims > 0 && rot_dims <= D),
             "zk_row_prep: the rotated channels must be even in number and at most the head's");
  ZK_REQUIRE(kcache != nullptr && vcache != nullptr && slot_map != nullptr, "zk_row_prep: no cache to store into");
  const size_t lds = (size_t)(nh + nkv) * D * sizeof(float);
  ZK_REQUIRE(lds <= 64 * 1024, "zk_row_prep: rows of more than 16384 channels are not supported");
  if (T == 0) return 0;
  static bool raised = false;
  if (!raised) {
    hipFuncSetAttribute((const void*)row_prep_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    raised = true;
  }
  const int threads = (ZSE_ACT_BF16 && T <= 64) ? 1024 : 256;
  row_prep_kernel<<<T, threads, lds, (hipStream_t)stream>>>((act_t*)qk, ld, positions, slot_map, bias, q_gain, k_gain, eps,
                                                       inv_freq, rot_dims, (act_t*)kcache, (act_t*)vcache, nh, nkv, D, E,
                                                       bs, v_transposed, values_are_keys);
  return zk_launch_status("zk_row_prep");
}

static const int row_prep_entered =
    zk_steplist_register("zk_row_prep", zk_packed::Call<zk_row_prep>::nargs, (void*)zk_packed::Call<zk_row_prep>::call);
static const int head_prep_entered =
    zk_steplist_register("zk_head_prep", zk_packed::Call<zk_head_prep>::nargs, (void*)zk_packed::Call<zk_head_prep>::call);
static const int head_prep_unit_entered = zk_steplist_register(
    "zk_head_prep_unit", zk_packed::Call<zk_head_prep_unit>::nargs, (void*)zk_packed::Call<zk_head_prep_unit>::call);
static const int head_prep_ext_entered = zk_steplist_register(
    "zk_head_prep_ext", zk_packed::Call<zk_head_prep_ext>::nargs, (void*)zk_packed::Call<zk_head_prep_ext>::call);
