// Several residual streams, the layer norm that reads them, and the short causal convolution
// over time that may follow the norm.
//
// The residual is S float rows per token, xs[t][s][W].  A sublayer reads a weighted sum of
// them and its result y goes back into every stream at once:
//
//   read :  u    = sum_s w_in[s] xs[s]                    (w_in absent: the plain sum)
//           out  = (u - mean(u)) / sqrt(var(u) + eps) * g + b     (var: mean squared deviation)
//   write:  xs'[r] = sum_s w_mix[s][r] xs[s] + w_out[r] y        (every r from the old xs)
//
// One kernel does a sublayer's write and the next sublayer's read, one block a token, so the
// streams are read and written once per sublayer.  S = 1 with unit weights is the ordinary
// residual sum with a layer norm.  Everything is float; y and out have the activation type.
//
// The convolution: out_t = h_t + sum_j w[c][j] h_(t - taps + 1 + j), channel by channel, rows
// before the sequence being zero.  The taps - 1 rows before a step's first token come from
// the request's state slot, which a second launch brings up to date afterwards (a launch of
// its own: the first tokens of a portion read what its last tokens would overwrite).
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

#define STREAMS_MAX 8

__global__ void replicate_kernel(const float* __restrict__ src, float* __restrict__ dst, int S, int W) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = src[(size_t)t * W + c];
    for (int s = 0; s < S; s++) dst[((size_t)t * S + s) * W + c] = v;
  }
}

// V channels a thread and pass (4 where rows are whole 16-byte pieces, else 1); the block is 256
// threads wide, or 1,024 for steps of few rows, which are bound by the latency of their loads.
template <int V>
__global__ __launch_bounds__(1024) void streams_step_kernel(
    float* __restrict__ xs, int S, const void* __restrict__ y, int y_parts, size_t y_plane,
    const float* __restrict__ w_mix, const float* __restrict__ w_out, const float* __restrict__ w_in,
    const float* __restrict__ norm_w, const float* __restrict__ norm_b, float eps, const int* __restrict__ rows,
    act_t* __restrict__ out, int W) {
  extern __shared__ float u_row[];          // W floats
  __shared__ float s_mix[STREAMS_MAX * STREAMS_MAX], s_out[STREAMS_MAX], s_in[STREAMS_MAX];
  __shared__ float scratch[17];
  const int b = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  const int t = rows ? rows[b] : b;
  if (tid < S * S && w_mix) s_mix[tid] = w_mix[tid];
  if (tid < S) {
    if (w_out) s_out[tid] = w_out[tid];
    s_in[tid] = w_in ? w_in[tid] : 1.f;
  }
  __syncthreads();
  float* x = xs + (size_t)t * S * W;
  float sum = 0.f;
  for (int c = tid * V; c < W; c += nt * V) {
    float v[STREAMS_MAX][V];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; s++)
      if (s < S) {
        if (V == 4) {
          const float4 q = *(const float4*)(x + (size_t)s * W + c);
          v[s][0] = q.x, v[s][V > 1 ? 1 : 0] = q.y, v[s][V > 2 ? 2 : 0] = q.z, v[s][V > 3 ? 3 : 0] = q.w;
        } else {
          v[s][0] = x[(size_t)s * W + c];
        }
      }
    if (y != nullptr) {
      float yv[V];
      if (y_parts > 0) {      // planes of a product that split K: added in order, rounded as the join would
        const float* p = (const float*)y + (size_t)t * W + c;
#pragma unroll
        for (int e = 0; e < V; e++) {
          float a = p[e];
          for (int k = 1; k < y_parts; k++) a += p[k * y_plane + e];
          yv[e] = to_f32(from_f32<act_t>(a));
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; e++) yv[e] = to_f32(((const act_t*)y)[(size_t)t * W + c + e]);
      }
      float nv[STREAMS_MAX][V];
#pragma unroll
      for (int r = 0; r < STREAMS_MAX; r++)
        if (r < S) {
#pragma unroll
          for (int e = 0; e < V; e++) {
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < STREAMS_MAX; s++)
              if (s < S) a = fmaf(s_mix[s * S + r], v[s][e], a);
            nv[r][e] = fmaf(s_out[r], yv[e], a);
          }
        }
#pragma unroll
      for (int r = 0; r < STREAMS_MAX; r++)
        if (r < S) {
#pragma unroll
          for (int e = 0; e < V; e++) v[r][e] = nv[r][e];
          if (V == 4) {
            *(float4*)(x + (size_t)r * W + c) = make_float4(nv[r][0], nv[r][V > 1 ? 1 : 0], nv[r][V > 2 ? 2 : 0], nv[r][V > 3 ? 3 : 0]);
          } else {
            x[(size_t)r * W + c] = nv[r][0];
          }
        }
    }
    if (out != nullptr) {
#pragma unroll
      for (int e = 0; e < V; e++) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; s++)
          if (s < S) u = fmaf(s_in[s], v[s][e], u);
        u_row[c + e] = u;
        sum += u;
      }
    }
  }
  if (out == nullptr) return;
  const float mean = block_sum(sum, scratch) / (float)W;
  float dev = 0.f;
  for (int c = tid; c < W; c += nt) {
    const float d = u_row[c] - mean;
    dev = fmaf(d, d, dev);
  }
  const float var = block_sum(dev, scratch) / (float)W;
  const float inv = 1.0f / sqrtf(var + eps);
  act_t* o = out + (size_t)b * W;
  for (int c = tid; c < W; c += nt) o[c] = from_f32<act_t>(fmaf((u_row[c] - mean) * inv, norm_w[c], norm_b ? norm_b[c] : 0.f));
}

// ---- the short convolution
// RENEW: every request of the step brings one token, so the thread of (token, channel) is the
// only one that touches its column of the state and moves it on itself.
template <bool RENEW>
__global__ void short_conv_kernel(const act_t* __restrict__ h, const float* __restrict__ w, float* __restrict__ state,
                                  int slot_words, int offset_words, const int* __restrict__ positions,
                                  const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                  const int* __restrict__ slot_of_req, act_t* __restrict__ out, int W, int taps,
                                  int ld_in, int ld_out, int residual, int act, const float* __restrict__ bias) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  if (positions[t] < 0) {             // a padding row of a captured step
    out[(size_t)t * ld_out + c] = from_f32<act_t>(0.f);
    return;
  }
  const int r = req_of_token[t];
  const int before = t - q_start[r];      // rows of this step in front of t that belong to the same request
  float* st = state + (size_t)slot_of_req[r] * slot_words + offset_words;
  const float x = to_f32(h[(size_t)t * ld_in + c]);
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; j++) {
    const int back = taps - 1 - j;
    float v;
    if (back <= before) v = to_f32(h[(size_t)(t - back) * ld_in + c]);
    else v = st[(size_t)(back - before - 1) * W + c];      // state row a holds the row a + 1 places before the step
    acc = fmaf(w[(size_t)c * taps + j], v, acc);
  }
  if (residual) acc = x + acc;
  if (act == 1) acc = acc / (1.0f + expf(-acc));      // silu
  out[(size_t)t * ld_out + c] = from_f32<act_t>(acc);
  if (RENEW) {
    for (int a = taps - 2; a > 0; a--) st[(size_t)a * W + c] = st[(size_t)(a - 1) * W + c];
    if (taps > 1) st[c] = x;
  }
}

__global__ void short_conv_state_kernel(const act_t* __restrict__ h, float* __restrict__ state, int slot_words,
                                        int offset_words, const int* __restrict__ q_start,
                                        const int* __restrict__ slot_of_req, int W, int taps, int ld_in) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int t0 = q_start[r], t1 = q_start[r + 1];
  const int n = t1 - t0;
  if (n <= 0) return;
  float* st = state + (size_t)slot_of_req[r] * slot_words + offset_words;
  // row a of the new state is the row a + 1 places before the next step: one of this step's
  // rows, or an older state row moved back by n; from the oldest on, so nothing is read after
  // it was overwritten
  for (int a = taps - 2; a >= 0; a--) {
    const float v = a < n ? to_f32(h[(size_t)(t1 - 1 - a) * ld_in + c]) : st[(size_t)(a - n) * W + c];
    st[(size_t)a * W + c] = v;
  }
}

// ---- turning pairs of channels of each head by +- position * frequency, in place
__global__ void rotate_heads_kernel(act_t* __restrict__ x, const int* __restrict__ positions,
                                    const float* __restrict__ freq, int heads, int size, int interleaved, float sign) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int half = size / 2;
  for (int it = threadIdx.x; it < heads * half; it += blockDim.x) {
    const int hd = it / half, m = it % half;
    float sn, cs;
    sincosf(sign * (float)pos * freq[m], &sn, &cs);
    act_t* p = x + ((size_t)t * heads + hd) * size;
    const int ia = interleaved ? 2 * m : m, ib = interleaved ? 2 * m + 1 : m + half;
    float ra, rb;
    rotate_pair(to_f32(p[ia]), to_f32(p[ib]), sn, cs, ra, rb);
    p[ia] = from_f32<act_t>(ra);
    p[ib] = from_f32<act_t>(rb);
  }
}

extern "C" {

int zk_replicate(const float* src, float* dst, int T, int S, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && S >= 1 && W > 0, "zk_replicate: bad sizes");
  if (T == 0) return 0;
  replicate_kernel<<<T, 256, 0, (hipStream_t)stream>>>(src, dst, S, W);
  return zk_launch_status("zk_replicate");
}

// xs: float [T, S, W], updated in place when y is given (y: [T, W] activations, or y_parts
// float planes [y_parts, T, W] to be added up).  out (may be null): the layer norm of the read,
// one row per token, or, with rows (device int32 [n_rows]), of those tokens only (y is then
// absent).  w_in null: the streams are summed with weight 1.
int zk_streams_step(float* xs, int S, const void* y, int y_parts, const float* w_mix, const float* w_out,
                    const float* w_in, const float* norm_w, const float* norm_b, float eps, const int* rows,
                    void* out, int n_rows, int T, int W, void* stream) {
  ZK_REQUIRE(S >= 1 && S <= STREAMS_MAX, "zk_streams_step: 1 to 8 streams");
  ZK_REQUIRE(T >= 0 && n_rows >= 0 && W > 0 && y_parts >= 0, "zk_streams_step: bad sizes");
  ZK_REQUIRE(y == nullptr || (w_mix != nullptr && w_out != nullptr), "zk_streams_step: a write needs its weights");
  ZK_REQUIRE(rows == nullptr || y == nullptr, "zk_streams_step: picked rows are read only");
  ZK_REQUIRE(rows != nullptr || n_rows == T, "zk_streams_step: one row per token unless rows are picked");
  ZK_REQUIRE(out == nullptr || norm_w != nullptr, "zk_streams_step: the norm needs its gain");
  ZK_REQUIRE((size_t)W * 4 <= 96 * 1024, "zk_streams_step: rows of more than 24576 channels are not supported");
  if (n_rows == 0) return 0;
  const size_t lds = out ? (size_t)W * 4 : 0;
  const bool vec = W % 4 == 0 && (uintptr_t)xs % 16 == 0;
  if (lds > 48 * 1024) {
    static bool raised = false;
    if (!raised) {
      hipFuncSetAttribute((const void*)streams_step_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
      hipFuncSetAttribute((const void*)streams_step_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
      raised = true;
    }
  }
  // in the 32-bit library the block is always 256 wide: the order of a row's sums must not follow
  // from how many rows a step brings
  const int threads = (ZSE_ACT_BF16 && n_rows <= 64) ? 1024 : 256;
  if (vec)
    streams_step_kernel<4><<<n_rows, threads, lds, (hipStream_t)stream>>>(xs, S, y, y_parts, (size_t)T * W, w_mix, w_out, w_in,
                                                                         norm_w, norm_b, eps, rows, (act_t*)out, W);
  else
    streams_step_kernel<1><<<n_rows, threads, lds, (hipStream_t)stream>>>(xs, S, y, y_parts, (size_t)T * W, w_mix, w_out, w_in,
                                                                         norm_w, norm_b, eps, rows, (act_t*)out, W);
  return zk_launch_status("zk_streams_step");
}

// h: [T, ld_in] activations, out: [T, ld_out], of which the first W channels take part; w: float
// [W, taps]; the state of request r is taps - 1 float rows of W at
// state[slot_of_req[r] * slot_words + offset_words].  residual: the input is added to the sum;
// act: 0 none, 1 silu (after the sum).
int zk_short_conv_bias(const void* h, int ld_in, const float* w, const float* state, int slot_words, int offset_words,
                       const int* positions, const int* req_of_token, const int* q_start, const int* slot_of_req,
                       void* out, int ld_out, int T, int W, int taps, int residual, int act, const float* bias,
                       void* stream) {
  ZK_REQUIRE(T >= 0 && T <= 65535 * 16 && W > 0 && taps >= 1, "zk_short_conv: bad sizes");
  ZK_REQUIRE(ld_in >= W && ld_out >= W && (act == 0 || act == 1), "zk_short_conv: bad strides or activation");
  ZK_REQUIRE(taps == 1 || (state != nullptr && slot_words >= offset_words + (taps - 1) * W),
             "zk_short_conv: the state does not fit its slot");
  if (T == 0) return 0;
  ZK_REQUIRE(T <= 65535, "zk_short_conv: more than 65535 rows");
  dim3 grid((W + 255) / 256, T);
  short_conv_kernel<false><<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)h, w, (float*)state, slot_words, offset_words,
                                                                  positions, req_of_token, q_start, slot_of_req,
                                                                  (act_t*)out, W, taps, ld_in, ld_out, residual, act, bias);
  return zk_launch_status("zk_short_conv");
}

// bias (zk_short_conv_bias; may be null): float [W], where the sum over the taps starts.
int zk_short_conv_ext(const void* h, int ld_in, const float* w, const float* state, int slot_words, int offset_words,
                      const int* positions, const int* req_of_token, const int* q_start, const int* slot_of_req,
                      void* out, int ld_out, int T, int W, int taps, int residual, int act, void* stream) {
  return zk_short_conv_bias(h, ld_in, w, state, slot_words, offset_words, positions, req_of_token, q_start, slot_of_req, out,
                            ld_out, T, W, taps, residual, act, nullptr, stream);
}

int zk_short_conv(const void* h, const float* w, const float* state, int slot_words, int offset_words,
                  const int* positions, const int* req_of_token, const int* q_start, const int* slot_of_req,
                  void* out, int T, int W, int taps, void* stream) {
  return zk_short_conv_ext(h, W, w, state, slot_words, offset_words, positions, req_of_token, q_start, slot_of_req, out, W,
                           T, W, taps, 1, 0, stream);
}

// The convolution and the renewal of the state in one launch, for steps in which every request
// brings exactly one token (T rows, T requests).
int zk_short_conv_token_bias(const void* h, int ld_in, const float* w, float* state, int slot_words, int offset_words,
                             const int* positions, const int* req_of_token, const int* q_start, const int* slot_of_req,
                             void* out, int ld_out, int T, int W, int taps, int residual, int act, const float* bias,
                             void* stream) {
  ZK_REQUIRE(T >= 0 && T <= 65535 && W > 0 && taps >= 1, "zk_short_conv_token: bad sizes");
  ZK_REQUIRE(ld_in >= W && ld_out >= W && (act == 0 || act == 1), "zk_short_conv_token: bad strides or activation");
  ZK_REQUIRE(taps == 1 || (state != nullptr && slot_words >= offset_words + (taps - 1) * W),
             "zk_short_conv_token: the state does not fit its slot");
  if (T == 0) return 0;
  dim3 grid((W + 255) / 256, T);
  short_conv_kernel<true><<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)h, w, state, slot_words, offset_words, positions,
                                                                 req_of_token, q_start, slot_of_req, (act_t*)out, W, taps,
                                                                 ld_in, ld_out, residual, act, bias);
  return zk_launch_status("zk_short_conv_token");
}

int zk_short_conv_token_ext(const void* h, int ld_in, const float* w, float* state, int slot_words, int offset_words,
                            const int* positions, const int* req_of_token, const int* q_start, const int* slot_of_req,
                            void* out, int ld_out, int T, int W, int taps, int residual, int act, void* stream) {
  return zk_short_conv_token_bias(h, ld_in, w, state, slot_words, offset_words, positions, req_of_token, q_start,
                                  slot_of_req, out, ld_out, T, W, taps, residual, act, nullptr, stream);
}

int zk_short_conv_token(const void* h, const float* w, float* state, int slot_words, int offset_words,
                        const int* positions, const int* req_of_token, const int* q_start, const int* slot_of_req,
                        void* out, int T, int W, int taps, void* stream) {
  return zk_short_conv_token_ext(h, W, w, state, slot_words, offset_words, positions, req_of_token, q_start, slot_of_req,
                                 out, W, T, W, taps, 1, 0, stream);
}

int zk_short_conv_state_ext(const void* h, int ld_in, float* state, int slot_words, int offset_words, const int* q_start,
                            const int* slot_of_req, int R, int W, int taps, void* stream) {
  ZK_REQUIRE(R >= 0 && R <= 65535 && W > 0 && taps >= 1 && ld_in >= W, "zk_short_conv_state: bad sizes");
  if (R == 0 || taps == 1) return 0;
  ZK_REQUIRE(state != nullptr && slot_words >= offset_words + (taps - 1) * W,
             "zk_short_conv_state: the state does not fit its slot");
  dim3 grid((W + 255) / 256, R);
  short_conv_state_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)h, state, slot_words, offset_words,
                                                                 q_start, slot_of_req, W, taps, ld_in);
  return zk_launch_status("zk_short_conv_state");
}

int zk_short_conv_state(const void* h, float* state, int slot_words, int offset_words, const int* q_start,
                        const int* slot_of_req, int R, int W, int taps, void* stream) {
  return zk_short_conv_state_ext(h, W, state, slot_words, offset_words, q_start, slot_of_req, R, W, taps, stream);
}

// x: [T, heads * size] activations; pair m of a head (m, m + size/2; interleaved: 2m, 2m + 1) is
// turned by sign * position * freq[m].
int zk_rotate_heads(void* x, const int* positions, const float* freq, int T, int heads, int size, int interleaved,
                    float sign, void* stream) {
  ZK_REQUIRE(T >= 0 && heads > 0 && size > 0 && size % 2 == 0 && freq != nullptr, "zk_rotate_heads: bad sizes");
  if (T == 0) return 0;
  rotate_heads_kernel<<<T, 256, 0, (hipStream_t)stream>>>((act_t*)x, positions, freq, heads, size, interleaved, sign);
  return zk_launch_status("zk_rotate_heads");
}

}  // extern "C"

ZK_ENTER(zk_replicate)
ZK_ENTER(zk_streams_step)
ZK_ENTER(zk_short_conv)
ZK_ENTER(zk_short_conv_token)
ZK_ENTER(zk_short_conv_state)
ZK_ENTER(zk_short_conv_ext)
ZK_ENTER(zk_short_conv_bias)
ZK_ENTER(zk_short_conv_token_bias)
ZK_ENTER(zk_short_conv_token_ext)
ZK_ENTER(zk_short_conv_state_ext)
ZK_ENTER(zk_rotate_heads)
