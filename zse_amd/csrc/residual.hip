// Joining two sublayers that read the same norm to the float residual stream:
//
//   h <- h + (a + b + bias);    out = h / sqrt(mean(h^2) + eps) * gain     (if a next norm is given)
//
// a and b are each either activations [T, W] (parts = 0) or ``parts`` float planes [parts, T, W]
// that are added up in order (partial sums of a product that split K, or the results of
// several paths of one sublayer); either may be absent.  The sum of the sublayers is formed
// first and then added to the stream, all in float.  One block per row.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

__device__ __forceinline__ float planes_value(const void* __restrict__ p, int parts, size_t plane, size_t at) {
  if (p == nullptr) return 0.f;
  if (parts <= 0) return to_f32(((const act_t*)p)[at]);
  float x = ((const float*)p)[at];
  for (int i = 1; i < parts; i++) x += ((const float*)p)[i * plane + at];
  return x;
}

__global__ void sum_norm_kernel(float* __restrict__ h, const void* __restrict__ a, int a_parts,
                                const void* __restrict__ b, int b_parts, const float* __restrict__ bias,
                                const float* __restrict__ w_next, float eps, int unit_offset, act_t* __restrict__ out,
                                int W) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t plane = (size_t)gridDim.x * W, row = (size_t)r * W;
  float* hr = h + row;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float y = planes_value(a, a_parts, plane, row + i) + planes_value(b, b_parts, plane, row + i);
    if (bias) y += bias[i];
    const float v = hr[i] + y;
    hr[i] = v;
    ss = fmaf(v, v, ss);
  }
  if (!w_next) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)      // each thread re-reads what it wrote
    out[row + i] = from_f32<act_t>(hr[i] * inv * (unit_offset ? 1.0f + w_next[i] : w_next[i]));
}

// h <- h + (a + b + bias); out = layer_norm(h) = (h - mean) / sqrt(var + eps) * w + c, var the mean of
// the squared deviations (two passes over the row: the mean first, then the deviations)
__global__ void sum_layer_norm_kernel(float* __restrict__ h, const void* __restrict__ a, int a_parts,
                                      const void* __restrict__ b, int b_parts, const float* __restrict__ bias,
                                      const float* __restrict__ w_next, const float* __restrict__ c_next, float eps,
                                      act_t* __restrict__ out, int W) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t plane = (size_t)gridDim.x * W, row = (size_t)r * W;
  float* hr = h + row;
  float s = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = hr[i];
    if (a != nullptr || b != nullptr || bias != nullptr) {
      float y = planes_value(a, a_parts, plane, row + i) + planes_value(b, b_parts, plane, row + i);
      if (bias) y += bias[i];
      v += y;
      hr[i] = v;
    }
    s += v;
  }
  if (!w_next) return;
  const float mean = block_sum(s, red) / (float)W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {      // each thread re-reads what it wrote
    const float d = hr[i] - mean;
    ss = fmaf(d, d, ss);
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    out[row + i] = from_f32<act_t>((hr[i] - mean) * inv * w_next[i] + (c_next ? c_next[i] : 0.f));
}

// h <- h + mult * (a + b + bias); out1 = norm(h) * gain1, out2 = norm(h) * gain2: a layer whose two
// sublayers read two norms of the same stream (either output may be absent)
__global__ void sum_norm_pair_kernel(float* __restrict__ h, const void* __restrict__ a, int a_parts,
                                     const void* __restrict__ b, int b_parts, const float* __restrict__ bias, float mult,
                                     const float* __restrict__ w1, act_t* __restrict__ out1,
                                     const float* __restrict__ w2, act_t* __restrict__ out2, float eps, int unit_offset,
                                     int W) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t plane = (size_t)gridDim.x * W, row = (size_t)r * W;
  float* hr = h + row;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = hr[i];
    if (a != nullptr || b != nullptr || bias != nullptr) {
      float y = planes_value(a, a_parts, plane, row + i) + planes_value(b, b_parts, plane, row + i);
      if (bias) y += bias[i];
      v = fmaf(mult, y, v);
      hr[i] = v;
    }
    ss = fmaf(v, v, ss);
  }
  if (!w1 && !w2) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {      // each thread re-reads what it wrote
    const float x = hr[i] * inv;
    if (w1) out1[row + i] = from_f32<act_t>(x * (unit_offset ? 1.0f + w1[i] : w1[i]));
    if (w2) out2[row + i] = from_f32<act_t>(x * (unit_offset ? 1.0f + w2[i] : w2[i]));
  }
}

// out[t, :] = sum_i scale_i x_i[t, :] as one float plane; the terms are activations
__global__ void weighted_sum_kernel(const act_t* __restrict__ x0, float s0, const act_t* __restrict__ x1, float s1,
                                    const act_t* __restrict__ x2, float s2, const act_t* __restrict__ x3, float s3,
                                    float* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float y = s0 * to_f32(x0[i]);
  if (x1) y = fmaf(s1, to_f32(x1[i]), y);
  if (x2) y = fmaf(s2, to_f32(x2[i]), y);
  if (x3) y = fmaf(s3, to_f32(x3[i]), y);
  out[i] = y;
}

// y[t, :] += bias
__global__ void add_bias_kernel(act_t* __restrict__ y, const float* __restrict__ bias, int W) {
  const size_t row = (size_t)blockIdx.x * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) y[row + i] = from_f32<act_t>(to_f32(y[row + i]) + bias[i]);
}

// out[t, :] = sum of float planes, rounded once
__global__ void planes_sum_kernel(const float* __restrict__ p, int parts, act_t* __restrict__ out, int W) {
  const size_t plane = (size_t)gridDim.x * W, row = (size_t)blockIdx.x * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) out[row + i] = from_f32<act_t>(planes_value(p, parts, plane, row + i));
}

extern "C" {

int zk_sum_norm(float* h, const void* a, int a_parts, const void* b, int b_parts, const float* bias, const float* w_next,
                float eps, int unit_offset, void* out, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && a_parts >= 0 && b_parts >= 0, "zk_sum_norm: bad sizes");
  ZK_REQUIRE(w_next == nullptr || out != nullptr, "zk_sum_norm: a next norm without output");
  if (T == 0) return 0;
  // in the 32-bit library the block is always 256 wide: the order of a row's sums must not follow
  // from how many rows a step brings
  const int threads = (ZSE_ACT_BF16 && T <= 64 && W >= 1024) ? 1024 : 256;
  sum_norm_kernel<<<T, threads, 0, (hipStream_t)stream>>>(h, a, a_parts, b, b_parts, bias, w_next, eps, unit_offset,
                                                         (act_t*)out, W);
  return zk_launch_status("zk_sum_norm");
}

// As zk_sum_norm with a layer norm of the new stream: gain w_next, bias c_next (may be null).
// a, b and bias all null: the stream stays as it is and only the norm is made.
int zk_sum_layer_norm(float* h, const void* a, int a_parts, const void* b, int b_parts, const float* bias,
                      const float* w_next, const float* c_next, float eps, void* out, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && a_parts >= 0 && b_parts >= 0, "zk_sum_layer_norm: bad sizes");
  ZK_REQUIRE(w_next == nullptr || out != nullptr, "zk_sum_layer_norm: a norm without output");
  if (T == 0) return 0;
  // (in the 32-bit library the block is always 256 wide: the order of a row's sums must not follow
  // from how many rows a step brings)
  const int threads = (ZSE_ACT_BF16 && T <= 64 && W >= 1024) ? 1024 : 256;
  sum_layer_norm_kernel<<<T, threads, 0, (hipStream_t)stream>>>(h, a, a_parts, b, b_parts, bias, w_next, c_next, eps,
                                                               (act_t*)out, W);
  return zk_launch_status("zk_sum_layer_norm");
}

// As zk_sum_norm, with the sublayers' sum times ``mult`` and up to two norms of the new stream
// (w1 -> out1, w2 -> out2; either pair may be null).  a, b and bias all null: the stream stays as
// it is and only the norms are made.
int zk_sum_norm_pair(float* h, const void* a, int a_parts, const void* b, int b_parts, const float* bias, float mult,
                     const float* w1, void* out1, const float* w2, void* out2, float eps, int unit_offset, int T, int W,
                     void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && a_parts >= 0 && b_parts >= 0, "zk_sum_norm_pair: bad sizes");
  ZK_REQUIRE((w1 == nullptr || out1 != nullptr) && (w2 == nullptr || out2 != nullptr), "zk_sum_norm_pair: a norm without output");
  if (T == 0) return 0;
  const int threads = (ZSE_ACT_BF16 && T <= 64 && W >= 1024) ? 1024 : 256;
  sum_norm_pair_kernel<<<T, threads, 0, (hipStream_t)stream>>>(h, a, a_parts, b, b_parts, bias, mult, w1, (act_t*)out1, w2,
                                                              (act_t*)out2, eps, unit_offset, W);
  return zk_launch_status("zk_sum_norm_pair");
}

// out (float [T, W]) = s0 x0 + s1 x1 + s2 x2 + s3 x3 over activations [T, W]; x1..x3 may be null.
int zk_weighted_sum(const void* x0, float s0, const void* x1, float s1, const void* x2, float s2, const void* x3, float s3,
                    float* out, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && x0 != nullptr && out != nullptr, "zk_weighted_sum: bad arguments");
  if (T == 0) return 0;
  const size_t n = (size_t)T * W;
  weighted_sum_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(
      (const act_t*)x0, s0, (const act_t*)x1, s1, (const act_t*)x2, s2, (const act_t*)x3, s3, out, n);
  return zk_launch_status("zk_weighted_sum");
}

int zk_add_bias(void* y, const float* bias, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && bias != nullptr, "zk_add_bias: bad sizes");
  if (T == 0) return 0;
  add_bias_kernel<<<T, 256, 0, (hipStream_t)stream>>>((act_t*)y, bias, W);
  return zk_launch_status("zk_add_bias");
}

int zk_planes_sum(const float* planes, int parts, void* out, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && parts >= 1, "zk_planes_sum: bad sizes");
  if (T == 0) return 0;
  planes_sum_kernel<<<T, 256, 0, (hipStream_t)stream>>>(planes, parts, (act_t*)out, W);
  return zk_launch_status("zk_planes_sum");
}

}  // extern "C"

ZK_ENTER(zk_sum_norm)
ZK_ENTER(zk_sum_layer_norm)
ZK_ENTER(zk_sum_norm_pair)
ZK_ENTER(zk_weighted_sum)
ZK_ENTER(zk_add_bias)
ZK_ENTER(zk_planes_sum)
