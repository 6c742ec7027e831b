// A routed feed-forward: every token goes through ``top`` of E small gated layers.
//
//   s = sigmoid(router logits),  the ``top`` largest are chosen (the lower index among equals)
//   expert e of token t sees  x' = s_e x_t  (the weight multiplies the input, not the output)
//   g = min(Wg x', limit),  u = clamp(Wu x', -limit, limit),  y = g sigmoid(1.702 g) (u + 1)
//   out_t = sum over the chosen experts, in the order they were chosen, of Wd y
//
// Variants, as parameters of the ``_ext`` entry points: scores softmax(router logits) over all experts
// instead of sigmoids; the weight on the expert's output instead of its input (out_t = sum s_e Wd y);
// y = silu(g) u instead of the clamped form.  ``zk_gate_rows`` multiplies float rows by the sigmoid
// of a number a row (a shared layer's gate).
//
// Two ways through the experts.  Few tokens (decoding): one block per (token, choice) multiplies
// the expert's rows by the token's row, and the weights stream once per choice.  Many tokens
// (bfloat16 only): the (token, choice) pairs are sorted by expert on the device, the scaled rows
// are gathered in that order, and a grouped matrix-core product runs over tiles of one expert's
// rows each; nothing comes back to the host, so a step can be written down and repeated.  Either
// way a row's sums run in an order fixed by the channel numbers, and a token's result does not
// depend on what else is in the step.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 16

__device__ __forceinline__ float clamped_swiglu(float g, float u, float limit) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
}

__device__ __forceinline__ float expert_act(float g, float u, float limit, int act) {
  return act == 1 ? g / (1.0f + expf(-g)) * u : clamped_swiglu(g, u, limit);
}

// ---- the router: one wave per token
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, int ld, int E, int top,
                                                       int* __restrict__ ids, float* __restrict__ wts, int softmax) {
  const int t = blockIdx.x, lane = threadIdx.x;
  float s[MOE_MAX_EXPERTS / 64];
  if (softmax) {
    // scores exp(z - max) / sum over all experts, in float
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / 64; i++) {
      const int e = lane + 64 * i;
      s[i] = e < E ? logits[(size_t)t * ld + e] : -INFINITY;
      mx = fmaxf(mx, s[i]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / 64; i++) {
      const int e = lane + 64 * i;
      s[i] = e < E ? expf(s[i] - mx) : 0.f;
      sum += s[i];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / 64; i++) s[i] = (lane + 64 * i) < E ? s[i] / sum : -1.f;
  } else {
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / 64; i++) {
      const int e = lane + 64 * i;
      s[i] = e < E ? 1.0f / (1.0f + expf(-logits[(size_t)t * ld + e])) : -1.f;
    }
  }
  for (int k = 0; k < top; k++) {
    float best = -2.f;
    int at = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / 64; i++)
      if (s[i] > best) {
        best = s[i];
        at = lane + 64 * i;
      }
    // the largest score of the wave, the lowest index among equals
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oa = __shfl_xor(at, o, 64);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (lane == 0) {
      ids[(size_t)t * top + k] = at;
      wts[(size_t)t * top + k] = best;
    }
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / 64; i++)
      if (lane + 64 * i == at) s[i] = -1.f;
  }
}

// Eight consecutive weights as floats (rows in whole groups of eight are read 16 bytes a lane).
__device__ __forceinline__ void load8(const float* p, float v[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const __bf16* p, float v[8]) {
  typedef __bf16 b8 __attribute__((ext_vector_type(8)));
  const b8 t = *(const b8*)p;
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = (float)t[i];
}

// A wave's sum with the steps inside a row of 16 lanes done by lane permutations of the vector unit
// (lane i with 15 - i, with 7 - i, inside the quads), the two steps across rows through local memory.
__device__ __forceinline__ float wave_sum_rows(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xf, 0xf, false));   // row_mirror
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xf, 0xf, false));   // row_half_mirror
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xf, 0xf, false));    // quad_perm [1,0,3,2]
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xf, 0xf, false));    // quad_perm [2,3,0,1]
  x += __shfl_xor(x, 16, 64);
  x += __shfl_xor(x, 32, 64);
  return x;
}

// The dot product of a weight row and a row in local memory, over a wave; the same order of sums
// whatever the step (eight channels a lane in turn where rows are whole groups of eight).
__device__ __forceinline__ float row_dot(const act_t* __restrict__ w, const float* __restrict__ x, int n, int lane) {
  float a = 0.f;
  if ((n & 7) == 0) {
    for (int i = lane * 8; i < n; i += 512) {
      float v[8];
      load8(w + i, v);
#pragma unroll
      for (int c = 0; c < 8; c++) a = fmaf(v[c], x[i + c], a);
    }
  } else {
    for (int i = lane; i < n; i += 64) a = fmaf(to_f32(w[i]), x[i], a);
  }
  return wave_sum_rows(a);
}

// ---- few tokens: y[(t, k), n] = act(Wg[e] x', Wu[e] x'), a wave per row pair
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const act_t* __restrict__ x, const int* __restrict__ ids,
                                                          const float* __restrict__ wts, const act_t* __restrict__ w_gu,
                                                          act_t* __restrict__ y, int top, int W, int F, float limit,
                                                          int rows_per_block, int act, int on_out) {
  extern __shared__ float xs[];                   // [W]
  const int pair = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int e = ids[pair];
  const float s = wts[pair];
  const int t = pair / top;
  const act_t* xr = x + (size_t)t * W;
  for (int i = tid; i < W; i += 256) xs[i] = on_out ? to_f32(xr[i]) : to_f32(from_f32<act_t>(s * to_f32(xr[i])));
  __syncthreads();
  const act_t* wg = w_gu + (size_t)e * 2 * F * W;
  const int n0 = blockIdx.y * rows_per_block;
  for (int n = n0 + wave; n < min(F, n0 + rows_per_block); n += 4) {
    const act_t* gr = wg + (size_t)n * W;
    const act_t* ur = wg + (size_t)(F + n) * W;
    const float g = row_dot(gr, xs, W, lane), u = row_dot(ur, xs, W, lane);
    if (lane == 0) y[(size_t)pair * F + n] = from_f32<act_t>(expert_act(g, u, limit, act));
  }
}

// out[t, n] = sum_k Wd[e_k][n] . y[(t, k)]
__global__ __launch_bounds__(256) void moe_down_kernel(const act_t* __restrict__ y, const int* __restrict__ ids,
                                                       const act_t* __restrict__ w_down, float* __restrict__ out,
                                                       int top, int W, int F, int rows_per_block,
                                                       const float* __restrict__ wts) {
  extern __shared__ float ys[];                   // [top][F]
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < top * F; i += 256) ys[i] = to_f32(y[(size_t)t * top * F + i]);
  __syncthreads();
  const int n0 = blockIdx.y * rows_per_block;
  for (int n = n0 + wave; n < min(W, n0 + rows_per_block); n += 4) {
    float total = 0.f;
    for (int k = 0; k < top; k++) {
      const act_t* wr = w_down + ((size_t)ids[(size_t)t * top + k] * W + n) * F;
      const float d = row_dot(wr, ys + k * F, F, lane);
      total += wts ? wts[(size_t)t * top + k] * d : d;
    }
    if (lane == 0) out[(size_t)t * W + n] = total;
  }
}

// ---- a dense layer of the same form: y = act(gu[:, :F], gu[:, F:])
__global__ void clamped_glu_kernel(const act_t* __restrict__ gu, act_t* __restrict__ y, int F, float limit) {
  const int t = blockIdx.y;
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= F) return;
  const act_t* row = gu + (size_t)t * 2 * F;
  y[(size_t)t * F + n] = from_f32<act_t>(clamped_swiglu(to_f32(row[n]), to_f32(row[F + n]), limit));
}

// ---- many tokens: sort the pairs by expert, gather the scaled rows
// One block.  order[i] = the pair at sorted place i; first[e] = the first place of expert e
// (first[E] = pairs).  Which place among its expert's a pair gets is left to chance: a row's
// result does not depend on its place.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int pairs, int E,
                                                        int* __restrict__ first, int* __restrict__ order) {
  __shared__ int count[MOE_MAX_EXPERTS + 1];
  __shared__ int cursor[MOE_MAX_EXPERTS];
  const int tid = threadIdx.x;
  for (int e = tid; e <= E; e += 1024) count[e] = 0;
  __syncthreads();
  for (int i = tid; i < pairs; i += 1024) atomicAdd(&count[ids[i] + 1], 1);
  __syncthreads();
  if (tid == 0) {
    for (int e = 0; e < E; e++) count[e + 1] += count[e];
  }
  __syncthreads();
  for (int e = tid; e <= E; e += 1024) first[e] = count[e];
  for (int e = tid; e < E; e += 1024) cursor[e] = count[e];
  __syncthreads();
  for (int i = tid; i < pairs; i += 1024) order[atomicAdd(&cursor[ids[i]], 1)] = i;
}

__global__ void moe_gather_kernel(const act_t* __restrict__ x, const int* __restrict__ order,
                                  const float* __restrict__ wts, act_t* __restrict__ xg, int top, int W) {
  const int i = blockIdx.x;
  const int pair = order[i];
  const float s = wts ? wts[pair] : 1.0f;
  const act_t* xr = x + (size_t)(pair / top) * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) xg[(size_t)i * W + c] = from_f32<act_t>(s * to_f32(xr[c]));
}

#if ZSE_ACT_BF16
// Grouped product on the matrix cores: C[i, n] = sum_k A[i, k] B[e(i)][n, k] over rows sorted by
// expert.  A block takes 64 rows of one expert and 64 columns; which expert and which rows it
// finds by walking first[] (tiles never span two experts; a tile past the last one ends at once).
// Four waves, each a 32 x 32 corner, 32 x 32 x 16 products, operands through local memory.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define GG_TM 64
#define GG_TN 64
#define GG_TK 32
#define GG_PAD 8

// mode 0: C = act(gate, up) with B = [E][2F][K], stores y[i, n] (n < F); mode 1: plain product
// with B = [E][N][K], stores float rows at out[order..] (see the launch).
template <int MODE>
__global__ __launch_bounds__(256) void moe_grouped_kernel(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                          const int* __restrict__ first, int E, int N, int K,
                                                          __bf16* __restrict__ y, float* __restrict__ out_rows,
                                                          float limit, int act) {
  __shared__ __bf16 As[GG_TM][GG_TK + GG_PAD];
  __shared__ __bf16 Bs[(MODE == 0 ? 2 : 1) * GG_TN][GG_TK + GG_PAD];
  __shared__ int tile_e, tile_row, tile_end;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) {
    // the blockIdx.x-th tile of rows, counting each expert's rows in whole tiles
    int left = blockIdx.x, e = 0, row = -1, end = 0;
    for (; e < E; e++) {
      const int lo = first[e], hi = first[e + 1];
      const int tiles = (hi - lo + GG_TM - 1) / GG_TM;
      if (left < tiles) {
        row = lo + left * GG_TM;
        end = hi;
        break;
      }
      left -= tiles;
    }
    tile_e = e;
    tile_row = row;
    tile_end = end;
  }
  __syncthreads();
  if (tile_row < 0) return;
  const int e = tile_e, row0 = tile_row, rows = min(GG_TM, tile_end - tile_row);
  const int n0 = blockIdx.y * GG_TN;
  const int wm = (wave & 1) * 32, wn = (wave >> 1) * 32;
  floatx16 acc0 = {0}, acc1 = {0};
  const __bf16* Be = B + (size_t)e * (MODE == 0 ? 2 : 1) * N * K;
  const int lr = tid >> 2, lc = (tid & 3) * 8;         // 64 rows x 4 pieces of 8
  for (int k0 = 0; k0 < K; k0 += GG_TK) {
    bf16x8 a = {0}, b = {0}, b2 = {0};
    const bool kin = k0 + lc < K;                        // K is a multiple of 8
    if (lr < rows && kin) a = *(const bf16x8*)(A + (size_t)(row0 + lr) * K + k0 + lc);
    if (n0 + lr < N && kin) {
      b = *(const bf16x8*)(Be + (size_t)(n0 + lr) * K + k0 + lc);
      if (MODE == 0) b2 = *(const bf16x8*)(Be + (size_t)(N + n0 + lr) * K + k0 + lc);
    }
    __syncthreads();
    *(bf16x8*)&As[lr][lc] = a;
    *(bf16x8*)&Bs[lr][lc] = b;
    if (MODE == 0) *(bf16x8*)&Bs[GG_TN + lr][lc] = b2;
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_TK; kk += 16) {
      const bf16x8 av = *(const bf16x8*)&As[wm + (lane & 31)][kk + (lane >> 5) * 8];
      const bf16x8 bv = *(const bf16x8*)&Bs[wn + (lane & 31)][kk + (lane >> 5) * 8];
      acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc0, 0, 0, 0);
      if (MODE == 0) {
        const bf16x8 bu = *(const bf16x8*)&Bs[GG_TN + wn + (lane & 31)][kk + (lane >> 5) * 8];
        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bu, acc1, 0, 0, 0);
      }
    }
  }
  // element i of the accumulator: row (i / 4) * 8 + (lane / 32) * 4 + i % 4, column lane % 32
  const int col = n0 + wn + (lane & 31);
#pragma unroll
  for (int i = 0; i < 16; i++) {
    const int r = wm + (i / 4) * 8 + (lane >> 5) * 4 + (i % 4);
    if (r < rows && col < N) {
      if (MODE == 0) y[(size_t)(row0 + r) * N + col] = (__bf16)expert_act(acc0[i], acc1[i], limit, act);
      else out_rows[(size_t)(row0 + r) * N + col] = acc0[i];
    }
  }
}

// out[t, :] = sum over t's choices, in their order, of the sorted rows' results
__global__ void moe_combine_kernel(const float* __restrict__ rows, const int* __restrict__ place, float* __restrict__ out,
                                   int top, int W, const float* __restrict__ wts) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float total = 0.f;
    for (int k = 0; k < top; k++) {
      const float v = rows[(size_t)place[(size_t)t * top + k] * W + c];
      total += wts ? wts[(size_t)t * top + k] * v : v;
    }
    out[(size_t)t * W + c] = total;
  }
}

__global__ void moe_place_kernel(const int* __restrict__ order, int* __restrict__ place, int pairs) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < pairs) place[order[i]] = i;
}
#endif

// rows[t, :] *= sigmoid(z[t * ld])
__global__ void gate_rows_kernel(float* __restrict__ rows, const float* __restrict__ z, int ld, int W) {
  const int t = blockIdx.x;
  const float g = 1.0f / (1.0f + expf(-z[(size_t)t * ld]));
  for (int c = threadIdx.x; c < W; c += blockDim.x) rows[(size_t)t * W + c] *= g;
}

extern "C" {

// logits: float [T, E] -> ids int32 [T, top], wts float [T, top] (the scores themselves).
// (device memory that a kernel writes is passed as void*: an ``int*`` argument means a result the
// host reads, which a launch list replaces)
// ld: the distance between rows of logits (>= E; a row may hold more than the experts' logits).
// softmax: the scores are exp(z) / sum over all experts instead of sigmoid(z).
int zk_moe_route_ext(const float* logits, int ld, void* ids, float* wts, int T, int E, int top, int softmax, void* stream) {
  ZK_REQUIRE(T >= 0 && E > 0 && top > 0 && top <= E && ld >= E, "zk_moe_route: bad sizes");
  ZK_REQUIRE(E <= MOE_MAX_EXPERTS && top <= MOE_MAX_TOP, "zk_moe_route: up to 1024 experts and 16 choices");
  if (T == 0) return 0;
  moe_route_kernel<<<T, 64, 0, (hipStream_t)stream>>>(logits, ld, E, top, (int*)ids, wts, softmax);
  return zk_launch_status("zk_moe_route");
}

int zk_moe_route(const float* logits, void* ids, float* wts, int T, int E, int top, void* stream) {
  return zk_moe_route_ext(logits, E, ids, wts, T, E, top, 0, stream);
}

// rows: float [T, W], each multiplied by sigmoid(z[t * ld]).
int zk_gate_rows(float* rows, const float* z, int ld, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && ld > 0 && rows != nullptr && z != nullptr, "zk_gate_rows: bad arguments");
  if (T == 0) return 0;
  gate_rows_kernel<<<T, 256, 0, (hipStream_t)stream>>>(rows, z, ld, W);
  return zk_launch_status("zk_gate_rows");
}

// x: [T, W]; w_gu: [E][2F][W], an expert's gate rows, then its up rows; w_down: [E][W][F].
// y: scratch [T * top, F] activations; out: float [T, W].
// act: 0 the clamped form, 1 silu(gate) up.  on_out: the weight multiplies the expert's output.
int zk_moe_experts_ext(const void* x, const int* ids, const float* wts, const void* w_gu, const void* w_down, void* y,
                       float* out, int T, int top, int W, int F, float limit, int act, int on_out, void* stream) {
  ZK_REQUIRE(T >= 0 && top > 0 && top <= MOE_MAX_TOP && W > 0 && F > 0, "zk_moe_experts: bad sizes");
  ZK_REQUIRE(T <= 65535 && (size_t)T * top <= 0x7fffffff, "zk_moe_experts: more than 65535 rows");
  ZK_REQUIRE((size_t)W * 4 <= 64 * 1024 && (size_t)top * F * 4 <= 64 * 1024, "zk_moe_experts: rows too wide for local memory");
  if (T == 0) return 0;
  const int rpb = 32;
  static bool raised = false;
  if (!raised) {
    hipFuncSetAttribute((const void*)moe_gate_up_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    hipFuncSetAttribute((const void*)moe_down_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    raised = true;
  }
  dim3 grid_up(T * top, (F + rpb - 1) / rpb);
  moe_gate_up_kernel<<<grid_up, 256, (size_t)W * 4, (hipStream_t)stream>>>((const act_t*)x, ids, wts, (const act_t*)w_gu,
                                                                          (act_t*)y, top, W, F, limit, rpb, act, on_out);
  dim3 grid(T, (W + rpb - 1) / rpb);
  moe_down_kernel<<<grid, 256, (size_t)top * F * 4, (hipStream_t)stream>>>((const act_t*)y, ids, (const act_t*)w_down, out, top,
                                                                         W, F, rpb, on_out ? wts : nullptr);
  return zk_launch_status("zk_moe_experts");
}

int zk_moe_experts(const void* x, const int* ids, const float* wts, const void* w_gu, const void* w_down, void* y,
                   float* out, int T, int top, int W, int F, float limit, void* stream) {
  return zk_moe_experts_ext(x, ids, wts, w_gu, w_down, y, out, T, top, W, F, limit, 0, 0, stream);
}

// gu: [T, 2F] -> y [T, F]
int zk_clamped_glu(const void* gu, void* y, int T, int F, float limit, void* stream) {
  ZK_REQUIRE(T >= 0 && T <= 65535 && F > 0, "zk_clamped_glu: bad sizes");
  if (T == 0) return 0;
  dim3 grid((F + 255) / 256, T);
  clamped_glu_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)gu, (act_t*)y, F, limit);
  return zk_launch_status("zk_clamped_glu");
}

#if ZSE_ACT_BF16
// The same through the grouped matrix-core product.  work: int32 [E + 1 + 2 * T * top] (first,
// order, place); xg: [T * top, W] and y: [T * top, F] bfloat16; rows: float [T * top, W].
int zk_moe_experts_grouped_ext(const void* x, const int* ids, const float* wts, const void* w_gu, const void* w_down,
                               void* work, void* xg, void* y, float* rows, float* out, int T, int E, int top, int W, int F,
                               float limit, int act, int on_out, void* stream) {
  ZK_REQUIRE(T >= 0 && top > 0 && top <= MOE_MAX_TOP && W > 0 && F > 0 && E > 0 && E <= MOE_MAX_EXPERTS,
             "zk_moe_experts_grouped: bad sizes");
  ZK_REQUIRE(W % 8 == 0 && F % 8 == 0, "zk_moe_experts_grouped: widths in whole groups of eight");
  ZK_REQUIRE(T <= 65535, "zk_moe_experts_grouped: more than 65535 rows");
  if (T == 0) return 0;
  const int pairs = T * top;
  int* first = (int*)work;
  int* order = first + E + 1;
  int* place = order + pairs;
  hipStream_t st = (hipStream_t)stream;
  moe_sort_kernel<<<1, 1024, 0, st>>>(ids, pairs, E, first, order);
  moe_place_kernel<<<(pairs + 255) / 256, 256, 0, st>>>(order, place, pairs);
  moe_gather_kernel<<<pairs, 256, 0, st>>>((const act_t*)x, order, on_out ? nullptr : wts, (act_t*)xg, top, W);
  const int tiles = (pairs + GG_TM - 1) / GG_TM + E;        // each expert may end in a tile that is not full
  dim3 g0(tiles, (F + GG_TN - 1) / GG_TN);
  moe_grouped_kernel<0><<<g0, 256, 0, st>>>((const __bf16*)xg, (const __bf16*)w_gu, first, E, F, W, (__bf16*)y, nullptr, limit, act);
  dim3 g1(tiles, (W + GG_TN - 1) / GG_TN);
  moe_grouped_kernel<1><<<g1, 256, 0, st>>>((const __bf16*)y, (const __bf16*)w_down, first, E, W, F, nullptr, rows, 0.f, 0);
  moe_combine_kernel<<<T, 256, 0, st>>>(rows, place, out, top, W, on_out ? wts : nullptr);
  return zk_launch_status("zk_moe_experts_grouped");
}

int zk_moe_experts_grouped(const void* x, const int* ids, const float* wts, const void* w_gu, const void* w_down,
                           void* work, void* xg, void* y, float* rows, float* out, int T, int E, int top, int W, int F,
                           float limit, void* stream) {
  return zk_moe_experts_grouped_ext(x, ids, wts, w_gu, w_down, work, xg, y, rows, out, T, E, top, W, F, limit, 0, 0, stream);
}
#endif

}  // extern "C"

#if ZSE_ACT_BF16
ZK_ENTER(zk_moe_experts_grouped)
ZK_ENTER(zk_moe_experts_grouped_ext)
#endif
ZK_ENTER(zk_moe_route_ext)
ZK_ENTER(zk_moe_experts_ext)
ZK_ENTER(zk_gate_rows)
ZK_ENTER(zk_moe_route)
ZK_ENTER(zk_moe_experts)
ZK_ENTER(zk_clamped_glu)
