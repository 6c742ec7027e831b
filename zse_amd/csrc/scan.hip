// The selective scan: a recurrence with N state values per channel whose decay and input follow
// from the token.
//
//   step_c = softplus(dt_c + bias_c);   A[c, n] = -exp(A_log[c, n])
//   S[c, n] <- exp(step_c A[c, n]) S[c, n] + step_c u_c B_n;   y_c = sum_n S[c, n] C_n + D_c u_c
//   out_c = y_c silu(z_c)
//
// B_n and C_n are shared by all channels of a token.  Four neighbouring lanes own a channel, each
// a share of its N state values in registers (chunks of four, dealt out in turn); the sum over n
// is joined by two lane permutations inside the quad.  A block takes 64 channels of one request
// and walks its tokens, staged in groups: B, C, the step sizes and inputs of a group are put down
// in local memory, then walked without a barrier.  Every sum runs in an order fixed by the
// state's numbering alone, so a request's values are the same bits however its tokens are cut
// into steps.  All arithmetic is float; u, B, C and z come in the activation type, dt as floats.
//
// Few requests with long portions leave most of the chip idle on such a walk, and the recurrence is
// linear in S: a portion is then cut into segments of seg_len tokens that are walked side by side,
// twice.  The first walk starts every segment from zero and keeps what it adds, L_s, and the sum
// of its step sizes, d_s; a small kernel goes through the segments in order (start_0 = S,
// start_(s+1) = exp(A d_s) start_s + L_s) and leaves every segment its starting state; the second
// walk starts from those, reads out, and its last segment stores the request's state.  The values
// differ from the plain walk's by rounding alone.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

#define SCAN_GROUP 16
#define SCAN_CHANNELS 64          // channels of a block: four lanes each

__device__ __forceinline__ float scan_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

__device__ __forceinline__ float scan_sum4(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xf, 0xf, false));    // quad_perm [1,0,3,2]
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xf, 0xf, false));    // quad_perm [2,3,0,1]
  return x;
}

// CH chunks of four state values a lane: N padded to 16 CH.
template <int CH>
__global__ __launch_bounds__(256) void selective_scan_kernel(
    const act_t* __restrict__ u, int ldu, const float* __restrict__ dt, int lddt, const float* __restrict__ dt_bias,
    const act_t* __restrict__ bc, int ldbc, int b_off, int c_off, const float* __restrict__ A_log,
    const float* __restrict__ Dv, const act_t* __restrict__ z, int ldz, float* __restrict__ state, int slot_words,
    int offset_words, const int* __restrict__ q_start, const int* __restrict__ slot_of_req, act_t* __restrict__ out,
    int inner, int N, int mode, int seg_len, int nseg, float* __restrict__ seg_state, float* __restrict__ seg_steps) {
  constexpr int NPAD = 16 * CH, GRP = SCAN_GROUP;
  __shared__ __attribute__((aligned(16))) float Bs[GRP][NPAD];
  __shared__ __attribute__((aligned(16))) float Cs[GRP][NPAD];
  __shared__ float steps[GRP][SCAN_CHANNELS];
  __shared__ float us[GRP][SCAN_CHANNELS];
  __shared__ float zs[GRP][SCAN_CHANNELS];         // the gate going in, the gated read-out coming back
  // mode 0: the plain walk, nseg == 1.  mode 1: a segment from zero, its sum and step sizes kept.
  // mode 2: a segment from its starting state, read out.
  const int r = blockIdx.x / nseg, seg = blockIdx.x - r * nseg;
  const int ch0 = blockIdx.y * SCAN_CHANNELS, tid = threadIdx.x;
  const int col = tid >> 2, j = tid & 3, c = ch0 + col;
  int t0 = q_start[r], t1 = q_start[r + 1];
  if (t1 <= t0) return;
  bool last_seg = true;
  if (mode != 0) {
    const int segs = (t1 - t0 + seg_len - 1) / seg_len;
    last_seg = seg == segs - 1;
    if (seg >= segs || (mode == 1 && last_seg)) return;        // nothing follows the last segment
    t0 += seg * seg_len;
    t1 = min(t1, t0 + seg_len);
  }
  const bool live = c < inner;
  const bool readout = mode != 1;
  float* Sreq = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)(live ? c : 0) * N;
  float* Sseg = mode != 0 ? seg_state + ((size_t)blockIdx.x * inner + (live ? c : 0)) * N : nullptr;
  const float* S = mode == 2 ? Sseg : Sreq;
  float step_sum = 0.f;
  float s[4 * CH], a[4 * CH];
#pragma unroll
  for (int i = 0; i < CH; i++)
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int n = 4 * (j + 4 * i) + q;
      const bool in = live && n < N;
      s[4 * i + q] = (in && mode != 1) ? S[n] : 0.f;
      a[4 * i + q] = in ? -expf(A_log[(size_t)c * N + n]) : 0.f;
    }
  const float dskip = live ? Dv[c] : 0.f;
  for (int c0 = t0; c0 < t1; c0 += GRP) {
    const int n_tok = min(GRP, t1 - c0);
    __syncthreads();
    for (int i = tid; i < n_tok * NPAD; i += 256) {
      const int tt = i / NPAD, n = i % NPAD;
      const act_t* row = bc + (size_t)(c0 + tt) * ldbc;
      Bs[tt][n] = n < N ? to_f32(row[b_off + n]) : 0.f;
      Cs[tt][n] = n < N ? to_f32(row[c_off + n]) : 0.f;
    }
    for (int i = tid; i < n_tok * SCAN_CHANNELS; i += 256) {
      const int tt = i / SCAN_CHANNELS, cc = i % SCAN_CHANNELS;
      const bool in = ch0 + cc < inner;
      steps[tt][cc] = in ? scan_softplus(dt[(size_t)(c0 + tt) * lddt + ch0 + cc] + dt_bias[ch0 + cc]) : 0.f;
      us[tt][cc] = in ? to_f32(u[(size_t)(c0 + tt) * ldu + ch0 + cc]) : 0.f;
      zs[tt][cc] = in ? to_f32(z[(size_t)(c0 + tt) * ldz + ch0 + cc]) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < n_tok; tt++) {
      const float st = steps[tt][col], x = us[tt][col];
      const float sx = st * x;
      const float4* B4 = (const float4*)Bs[tt] + j;
      const float4* C4 = (const float4*)Cs[tt] + j;
      float acc0 = 0.f, acc1 = 0.f;
      step_sum += st;
#pragma unroll
      for (int i = 0; i < CH; i++) {
        const float4 b = B4[4 * i];
        s[4 * i] = fmaf(expf(st * a[4 * i]), s[4 * i], sx * b.x);
        s[4 * i + 1] = fmaf(expf(st * a[4 * i + 1]), s[4 * i + 1], sx * b.y);
        s[4 * i + 2] = fmaf(expf(st * a[4 * i + 2]), s[4 * i + 2], sx * b.z);
        s[4 * i + 3] = fmaf(expf(st * a[4 * i + 3]), s[4 * i + 3], sx * b.w);
      }
      if (!readout) continue;
#pragma unroll
      for (int i = 0; i < CH; i++) {
        const float4 cv = C4[4 * i];
        acc0 = fmaf(s[4 * i], cv.x, acc0);
        acc1 = fmaf(s[4 * i + 1], cv.y, acc1);
        acc0 = fmaf(s[4 * i + 2], cv.z, acc0);
        acc1 = fmaf(s[4 * i + 3], cv.w, acc1);
      }
      const float y = scan_sum4(acc0 + acc1) + dskip * x;
      // the walk touches no global memory: a channel's gate waits in local memory, and its
      // result takes the gate's place (the channel's four lanes are in one wave)
      if (j == 0) {
        const float zz = zs[tt][col];
        zs[tt][col] = y * (zz / (1.0f + expf(-zz)));
      }
    }
    __syncthreads();
    if (!readout) continue;
    for (int i = tid; i < n_tok * SCAN_CHANNELS; i += 256) {
      const int tt = i / SCAN_CHANNELS, cc = i % SCAN_CHANNELS;
      if (ch0 + cc < inner) out[(size_t)(c0 + tt) * inner + ch0 + cc] = from_f32<act_t>(zs[tt][cc]);
    }
  }
  if (mode == 1 && live && j == 0) seg_steps[(size_t)blockIdx.x * inner + c] = step_sum;
  float* Sto = mode == 1 ? Sseg : Sreq;
  if (live && (mode != 2 || last_seg)) {
#pragma unroll
    for (int i = 0; i < CH; i++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int n = 4 * (j + 4 * i) + q;
        if (n < N) Sto[n] = s[4 * i + q];
      }
  }
}

// Through a request's segments in order: what a segment added from zero gives way to the state
// it starts from.  One thread an element of S; the last segment adds nothing here (it stores the
// request's state itself, after its second walk).
__global__ __launch_bounds__(256) void scan_segments_kernel(
    float* __restrict__ seg_state, const float* __restrict__ seg_steps, const float* __restrict__ A_log,
    const float* __restrict__ state, int slot_words, int offset_words, const int* __restrict__ q_start,
    const int* __restrict__ slot_of_req, int seg_len, int nseg, int inner, int N) {
  const int r = blockIdx.y;
  const int n_tok = q_start[r + 1] - q_start[r];
  if (n_tok <= 0) return;
  const int segs = (n_tok + seg_len - 1) / seg_len;
  const size_t per = (size_t)inner * N;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= per) return;
  const size_t c = i / N;
  const float a = -expf(A_log[i]);
  float cur = state[(size_t)slot_of_req[r] * slot_words + offset_words + i];
  float* ss = seg_state + (size_t)r * nseg * per + i;
  const float* sd = seg_steps + (size_t)r * nseg * inner + c;
  for (int sg = 0; sg < segs; sg++) {
    const bool more = sg + 1 < segs;
    const float added = more ? ss[(size_t)sg * per] : 0.f;
    const float decay = more ? expf(a * sd[(size_t)sg * inner]) : 0.f;
    ss[(size_t)sg * per] = cur;
    cur = fmaf(decay, cur, added);
  }
}

extern "C" {

// u: [T, ldu] activations, ``inner`` channels (after the convolution and silu).  dt: float [T, lddt],
// one per channel before bias and softplus; dt_bias: float [inner].  bc: [T, ldbc] activations with
// B_n at column b_off and C_n at c_off (N each).  A_log: float [inner, N]; Dv: float [inner].
// z: [T, ldz] activations, the output gate before its silu.  state: request r's S [inner, N] lies at
// state[slot_of_req[r] * slot_words + offset_words].  out: [T, inner].  Requests are rows
// [q_start[r], q_start[r + 1]).
int zk_selective_scan(const void* u, int ldu, const float* dt, int lddt, const float* dt_bias, const void* bc, int ldbc,
                      int b_off, int c_off, const float* A_log, const float* Dv, const void* z, int ldz, float* state,
                      int slot_words, int offset_words, const int* q_start, const int* slot_of_req, void* out, int T,
                      int R, int inner, int N, int max_q_len, int seg_len, float* seg_state, float* seg_steps,
                      void* stream) {
  ZK_REQUIRE(T >= 0 && R >= 0 && inner > 0 && N > 0, "zk_selective_scan: bad sizes");
  ZK_REQUIRE(N <= 128, "zk_selective_scan: up to 128 state values a channel");
  ZK_REQUIRE(ldu >= inner && lddt >= inner && ldz >= inner && ldbc >= b_off + N && ldbc >= c_off + N && b_off >= 0 && c_off >= 0,
             "zk_selective_scan: rows too short");
  ZK_REQUIRE(state != nullptr && (long long)slot_words >= (long long)offset_words + (long long)inner * N,
             "zk_selective_scan: the state does not fit its slot");
  if (R == 0 || T == 0) return 0;
  const int blocks = (inner + SCAN_CHANNELS - 1) / SCAN_CHANNELS;
  ZK_REQUIRE(blocks <= 65535, "zk_selective_scan: too many channels");
  // segments: seg_state float [R * nseg, inner * N], seg_steps float [R * nseg, inner], nseg as below
  const bool segmented = seg_len > 0 && seg_state != nullptr && seg_steps != nullptr && max_q_len > seg_len;
  const int nseg = segmented ? (max_q_len + seg_len - 1) / seg_len : 1;
  ZK_REQUIRE((long long)R * nseg <= 0x7fffffffLL / 2, "zk_selective_scan: too many segments");
  dim3 grid(R * nseg, blocks);
#define LAUNCH(C, MODE)                                                                                               \
  selective_scan_kernel<C><<<grid, 256, 0, (hipStream_t)stream>>>(                                                   \
      (const act_t*)u, ldu, dt, lddt, dt_bias, (const act_t*)bc, ldbc, b_off, c_off, A_log, Dv, (const act_t*)z, ldz, \
      state, slot_words, offset_words, q_start, slot_of_req, (act_t*)out, inner, N, MODE, seg_len, nseg, seg_state,   \
      seg_steps)
#define WALK(MODE)                                                                                                    \
  do {                                                                                                                \
    if (N <= 16) LAUNCH(1, MODE);                                                                                     \
    else if (N <= 32) LAUNCH(2, MODE);                                                                                \
    else if (N <= 64) LAUNCH(4, MODE);                                                                                \
    else LAUNCH(8, MODE);                                                                                             \
  } while (0)
  if (segmented) {
    WALK(1);
    dim3 sg((unsigned)(((size_t)inner * N + 255) / 256), R);
    scan_segments_kernel<<<sg, 256, 0, (hipStream_t)stream>>>(seg_state, seg_steps, A_log, state, slot_words,
                                                              offset_words, q_start, slot_of_req, seg_len, nseg, inner, N);
    WALK(2);
  } else {
    WALK(0);
  }
#undef WALK
#undef LAUNCH
  return zk_launch_status("zk_selective_scan");
}

}  // extern "C"

ZK_ENTER(zk_selective_scan)
