// Gated linear attention: a recurrent mixer with a matrix state S [D, E] per head whose rows
// decay each at its own rate.
//
//   S <- diag(alpha_t) S + k_t v_t^T;   o_t = S^T q_t
//
// with q_t scaled by D^(-1/2), alpha_t = sigmoid(z_t + bias)^(1/tau) = exp(logsigmoid(z_t + bias) / tau)
// per key channel, and the read-out divided by its root mean square over E, times a gain [E] and
// silu(g_t).
//
// The recurrence never mixes value channels: column e of S and o depends on column e alone.  DS
// neighbouring lanes own one column of S, each a share of its rows in registers (row chunks of
// four, dealt out in turn), and walk the tokens of their request; the sum over the rows (S^T q)
// is joined across the lanes by lane permutations inside the wave, no local memory and no
// barrier.  q_t, k_t and alpha_t are read from local memory, every column at the same
// addresses.  Tokens are staged in groups: the block loads q, k of a group and makes its decays,
// walks it, then norms and gates the group's read-outs (a head whose value channels span several
// blocks leaves that to a second kernel).  Every sum runs in an order fixed by the channel
// numbers alone, so a request's values are the same bits however its tokens are cut into steps.
// All arithmetic is float; q, k, v, g come in the activation type, z as floats.
//
// Few requests with long portions leave most of the chip idle on such a walk, and the recurrence is
// linear in S: a portion is then cut into segments of seg_len tokens that are walked side by side,
// twice.  The first walk starts every segment from zero and keeps what it adds, L_s, and the
// product of its decays, P_s; a small kernel goes through the segments in order (start_0 = S,
// start_(s+1) = diag(P_s) start_s + L_s) and leaves every segment its starting state; the second
// walk starts from those, reads out, and its last segment stores the request's state.  The sums
// are the same, grouped by segments, so the values differ from the plain walk's by rounding alone.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

#define GLA_GROUP 16
#define GLA_COLS 128              // the most value channels a block takes
#define GLA_COLS_LONG 16          // and what it takes when portions are long: more blocks, a head over more compute units

// The sum of x over the 8 lanes that share a column: lane i with 7 - i, then inside the quads.
__device__ __forceinline__ float gla_sum8(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xf, 0xf, false));   // row_half_mirror
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xf, 0xf, false));    // quad_perm [1,0,3,2]
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xf, 0xf, false));    // quad_perm [2,3,0,1]
  return x;
}
__device__ __forceinline__ float gla_sum16(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xf, 0xf, false));   // row_mirror
  return gla_sum8(x);
}

// log(sigmoid(x)) = min(x, 0) - log(1 + exp(-|x|))
__device__ __forceinline__ float log_sigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// DS lanes share a column (8 or 16), each holds CH chunks of four rows of S (4 CH DS rows in all, D
// padded with zeros).  raw (may be null): float [T, H * E], the read-outs before their norm, for a
// head that spans several blocks.
template <int CH, int DS>
__global__ __launch_bounds__(1024) void gla_kernel(
    const act_t* __restrict__ qkv, int ld, int k_off, int v_off, const act_t* __restrict__ g, int ldg,
    const float* __restrict__ z, int ldz, const float* __restrict__ z_bias, float inv_tau,
    const float* __restrict__ gain, float* __restrict__ state, int slot_words, int offset_words,
    const int* __restrict__ q_start, const int* __restrict__ slot_of_req, act_t* __restrict__ out,
    float* __restrict__ raw, int H, int D, int E, float eps, float q_scale, int COLS, int mode, int seg_len, int nseg,
    float* __restrict__ seg_state, float* __restrict__ seg_decay, int decays_ready) {
  constexpr int DMAX = 4 * CH * DS, RD = 4 * CH, GRP = GLA_GROUP;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;                                 // [GRP][DMAX]
  float* ks = qs + GRP * DMAX;                     // [GRP][DMAX]
  float* as = ks + GRP * DMAX;                     // [GRP][DMAX]: the decays
  float* ov = as + GRP * DMAX;                     // [GRP][COLS]: v going in, the read-out coming back
  float* prod = ov + GRP * COLS;                   // [DMAX]: the product of a segment's decays (mode 1)
  // mode 0: the plain walk, nseg == 1.  mode 1: a segment from zero, its sum and decays kept.
  // mode 2: a segment from its starting state, read out.
  const int r = blockIdx.x / nseg, seg = blockIdx.x - r * nseg;
  const int h = blockIdx.y, e0 = blockIdx.z * COLS, tid = threadIdx.x, nt = blockDim.x;
  const int lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
  const int col = tid / DS, j = tid % DS, e = e0 + col;
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
  const bool live = e < E;
  const bool readout = mode != 1;
  const int cols = min(COLS, E - e0);
  float* S = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)h * D * E;
  float* Sseg = mode != 0 ? seg_state + ((size_t)blockIdx.x * H + h) * D * E : nullptr;
  const float* Sfrom = mode == 2 ? Sseg : S;
  float s[RD];
#pragma unroll
  for (int i = 0; i < CH; i++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const int d = 4 * (j + DS * i) + c;
      s[4 * i + c] = (mode != 1 && live && d < D) ? Sfrom[(size_t)d * E + e] : 0.f;
    }
  if (mode == 1)
    for (int d = tid; d < DMAX; d += nt) prod[d] = 1.f;
  for (int c0 = t0; c0 < t1; c0 += GRP) {
    const int n = min(GRP, t1 - c0);
    __syncthreads();
    for (int i = tid; i < n * DMAX; i += nt) {
      const int tt = i / DMAX, d = i % DMAX;
      const act_t* row = qkv + (size_t)(c0 + tt) * ld + (size_t)h * D;
      const bool in = d < D;
      if (readout) qs[i] = in ? to_f32(row[d]) * q_scale : 0.f;
      ks[i] = in ? to_f32(row[k_off + d]) : 0.f;
      // padding rows of S stay zero whatever their decay
      const float zz = in ? z[(size_t)(c0 + tt) * ldz + (size_t)h * D + d] : 0.f;
      as[i] = !in ? 0.f : decays_ready ? zz : expf(log_sigmoid_f(zz + z_bias[(size_t)h * D + d]) * inv_tau);
    }
    for (int i = tid; i < n * COLS; i += nt) {
      const int tt = i / COLS, c = i % COLS;
      ov[i] = c < cols ? to_f32(qkv[(size_t)(c0 + tt) * ld + v_off + (size_t)h * E + e0 + c]) : 0.f;
    }
    __syncthreads();
    if (mode == 1 && blockIdx.z == 0)
      for (int d = tid; d < DMAX; d += nt) {
        float pr = prod[d];
        for (int tt = 0; tt < n; tt++) pr *= as[tt * DMAX + d];
        prod[d] = pr;
      }
    // the walk: no barrier.  What the next token needs (its k, decays and v) is asked for before this
    // token's arithmetic.
    float4 kn[CH], an[CH];
    float vn;
    {
      const float4* k4 = (const float4*)ks + j;
      const float4* a4 = (const float4*)as + j;
#pragma unroll
      for (int i = 0; i < CH; i++) {
        kn[i] = k4[DS * i];
        an[i] = a4[DS * i];
      }
      vn = ov[col];
    }
    for (int tt = 0; tt < n; tt++) {
      const float4* q4 = (const float4*)(qs + tt * DMAX) + j;
      const float vt = vn;
      float4 kk[CH], aa[CH], qq[CH];
#pragma unroll
      for (int i = 0; i < CH; i++) {
        kk[i] = kn[i];
        aa[i] = an[i];
        qq[i] = q4[DS * i];
      }
      if (tt + 1 < n) {
        const float4* k4 = (const float4*)(ks + (tt + 1) * DMAX) + j;
        const float4* a4 = (const float4*)(as + (tt + 1) * DMAX) + j;
#pragma unroll
        for (int i = 0; i < CH; i++) {
          kn[i] = k4[DS * i];
          an[i] = a4[DS * i];
        }
        vn = ov[(tt + 1) * COLS + col];
      }
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
      for (int i = 0; i < CH; i++) {
        s[4 * i] = fmaf(s[4 * i], aa[i].x, kk[i].x * vt);
        s[4 * i + 1] = fmaf(s[4 * i + 1], aa[i].y, kk[i].y * vt);
        s[4 * i + 2] = fmaf(s[4 * i + 2], aa[i].z, kk[i].z * vt);
        s[4 * i + 3] = fmaf(s[4 * i + 3], aa[i].w, kk[i].w * vt);
      }
      if (!readout) continue;
#pragma unroll
      for (int i = 0; i < CH; i++) {
        a0 = fmaf(s[4 * i], qq[i].x, a0);
        a1 = fmaf(s[4 * i + 1], qq[i].y, a1);
        a2 = fmaf(s[4 * i + 2], qq[i].z, a2);
        a3 = fmaf(s[4 * i + 3], qq[i].w, a3);
      }
      const float o = DS == 16 ? gla_sum16((a0 + a1) + (a2 + a3)) : gla_sum8((a0 + a1) + (a2 + a3));
      // a column's v of this token was read (by its lanes, all in one wave) before the read-out
      // takes its place
      if (j == 0) ov[tt * COLS + col] = o;
    }
    __syncthreads();
    if (!readout) continue;
    if (raw != nullptr) {                          // the head spans several blocks: its norm comes later
      for (int i = tid; i < n * COLS; i += nt) {
        const int tt = i / COLS, c = i % COLS;
        if (c < cols) raw[((size_t)(c0 + tt) * H + h) * E + e0 + c] = ov[i];
      }
      continue;
    }
    for (int tt = wave; tt < n; tt += nw) {        // unit RMS over the head's read-out, gain, gate
      float ss = 0.f;
      for (int c = lane; c < E; c += 64) ss = fmaf(ov[tt * COLS + c], ov[tt * COLS + c], ss);
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)E + eps);
      const act_t* gr = g + (size_t)(c0 + tt) * ldg + (size_t)h * E;
      act_t* orow = out + ((size_t)(c0 + tt) * H + h) * E;
      for (int c = lane; c < E; c += 64) {
        const float gg = to_f32(gr[c]);
        orow[c] = from_f32<act_t>(ov[tt * COLS + c] * inv * gain[c] * (gg / (1.0f + expf(-gg))));
      }
    }
  }
  if (mode == 1 && blockIdx.z == 0)                // written by the threads that made them
    for (int d = tid; d < D; d += nt) seg_decay[((size_t)blockIdx.x * H + h) * D + d] = prod[d];
  float* Sto = mode == 1 ? Sseg : S;
  if (live && (mode != 2 || last_seg)) {
#pragma unroll
    for (int i = 0; i < CH; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int d = 4 * (j + DS * i) + c;
        if (d < D) Sto[(size_t)d * E + e] = s[4 * i + c];
      }
  }
}

// The decays of a step with long portions, made once where every block of a head and both walks
// of a segment would make them again: z <- sigmoid(z + bias)^(1 / tau), the very expression of the walk.
__global__ __launch_bounds__(256) void gla_decays_kernel(float* __restrict__ z, int ldz, const float* __restrict__ z_bias,
                                                         float inv_tau, int T, int HD) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)T * HD) return;
  const size_t t = i / HD, c = i - t * HD;
  float* at = z + t * ldz + c;
  *at = expf(log_sigmoid_f(*at + z_bias[c]) * inv_tau);
}

// Through a request's segments in order: what a segment added from zero gives way to the state
// it starts from.  One thread an element of S; the last segment adds nothing here (it stores the
// request's state itself, after its second walk).
__global__ __launch_bounds__(256) void gla_segments_kernel(
    float* __restrict__ seg_state, const float* __restrict__ seg_decay, const float* __restrict__ state, int slot_words,
    int offset_words, const int* __restrict__ q_start, const int* __restrict__ slot_of_req, int seg_len, int nseg,
    int H, int D, int E) {
  const int r = blockIdx.y;
  const int n_tok = q_start[r + 1] - q_start[r];
  if (n_tok <= 0) return;
  const int segs = (n_tok + seg_len - 1) / seg_len;
  const size_t per = (size_t)H * D * E;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= per) return;
  const size_t hd = i / E;                         // h * D + d
  float cur = state[(size_t)slot_of_req[r] * slot_words + offset_words + i];
  float* ss = seg_state + (size_t)r * nseg * per + i;
  const float* pd = seg_decay + (size_t)r * nseg * H * D + hd;
  for (int sg = 0; sg < segs; sg++) {
    const bool more = sg + 1 < segs;
    const float added = more ? ss[(size_t)sg * per] : 0.f;
    const float decay = more ? pd[(size_t)sg * H * D] : 0.f;
    ss[(size_t)sg * per] = cur;
    cur = fmaf(decay, cur, added);
  }
}

// One wave per (token, head): out = raw / sqrt(mean(raw^2) + eps) * gain * silu(g).
__global__ __launch_bounds__(64) void gla_finish_kernel(const float* __restrict__ raw, const act_t* __restrict__ g, int ldg,
                                                        const float* __restrict__ gain, const int* __restrict__ positions,
                                                        act_t* __restrict__ out, int H, int E, float eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* rr = raw + ((size_t)t * H + h) * E;
  act_t* orow = out + ((size_t)t * H + h) * E;
  if (positions[t] < 0) {                          // a padding row of a captured step
    for (int c = lane; c < E; c += 64) orow[c] = from_f32<act_t>(0.f);
    return;
  }
  float ss = 0.f;
  for (int c = lane; c < E; c += 64) ss = fmaf(rr[c], rr[c], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)E + eps);
  const act_t* gr = g + (size_t)t * ldg + (size_t)h * E;
  for (int c = lane; c < E; c += 64) {
    const float gg = to_f32(gr[c]);
    orow[c] = from_f32<act_t>(rr[c] * inv * gain[c] * (gg / (1.0f + expf(-gg))));
  }
}

extern "C" {

// qkv: [T, ld] activations: H query heads of D at column 0, H key heads at k_off, H value heads of E
// at v_off.  g: [T, ldg], H heads of E (the output gate before its silu).  z: float [T, ldz], H heads
// of D (the decays before bias, sigmoid and root; overwritten with the decays where the step is walked in
// segments); z_bias: float [H * D]; gain: float [E].
// state: request r's S [H, D, E] lies at state[slot_of_req[r] * slot_words + offset_words].
// out: [T, H * E].  Requests are rows [q_start[r], q_start[r + 1]).  raw: float scratch [T, H * E],
// used by heads that span several blocks (may be null: a head of up to 128 value channels then
// stays in one block whatever the step); positions: [T].  max_q_len: the longest portion of the
// step: with long portions a block takes 16 value channels, so that a head's walk spreads over
// more compute units.
int zk_gla(const void* qkv, int ld, int k_off, int v_off, const void* g, int ldg, float* z, int ldz,
           const float* z_bias, float tau, const float* gain, float* state, int slot_words, int offset_words,
           const int* q_start, const int* slot_of_req, const int* positions, void* out, float* raw, int T, int R,
           int max_q_len, int H, int D, int E, float eps, int seg_len, float* seg_state, float* seg_decay, void* stream) {
  ZK_REQUIRE(T >= 0 && R >= 0 && H > 0 && D > 0 && E > 0 && tau > 0.f, "zk_gla: bad sizes");
  ZK_REQUIRE(D <= 256, "zk_gla: up to 256 query/key channels a head");
  ZK_REQUIRE(H <= 65535 && (E + GLA_COLS_LONG - 1) / GLA_COLS_LONG <= 65535, "zk_gla: too many heads or value channels");
  ZK_REQUIRE(state != nullptr && slot_words >= offset_words + H * D * E, "zk_gla: the state does not fit its slot");
  ZK_REQUIRE(ldz >= H * D && z != nullptr && z_bias != nullptr, "zk_gla: the decays' rows are too short");
  const bool scratch = raw != nullptr && positions != nullptr;
  if (R == 0 || T == 0) return 0;
  const int DMAX = D <= 32 ? 32 : D <= 64 ? 64 : D <= 128 ? 128 : 256;
  const int DS = DMAX == 256 ? 16 : 8;
  const bool spread = scratch && max_q_len > GLA_GROUP && E > GLA_COLS_LONG;
  const int per_block = spread ? GLA_COLS_LONG : DS == 16 ? GLA_COLS / 2 : GLA_COLS;
  ZK_REQUIRE(E <= per_block || scratch, "zk_gla: a head that spans several blocks needs scratch");
  const int blocks_e = (E + per_block - 1) / per_block;
  const int unit = 64 / DS;                                             // columns of a wave
  const int cols = E < per_block ? (E + unit - 1) / unit * unit : per_block;
  const int threads = cols * DS;
  const size_t lds = (size_t)GLA_GROUP * (3 * DMAX + cols) * sizeof(float) + DMAX * sizeof(float);
  // segments: seg_state float [R * nseg, H * D * E], seg_decay float [R * nseg, H * D], nseg as below
  const bool segmented = seg_len > 0 && seg_state != nullptr && seg_decay != nullptr && max_q_len > seg_len;
  ZK_REQUIRE(seg_len <= 0 || seg_len % GLA_GROUP == 0, "zk_gla: segments of whole groups of tokens");
  const int nseg = segmented ? (max_q_len + seg_len - 1) / seg_len : 1;
  ZK_REQUIRE((long long)R * nseg <= 0x7fffffffLL / 2, "zk_gla: too many segments");
  dim3 grid(R * nseg, H, blocks_e);
  float* raw_arg = blocks_e > 1 ? raw : nullptr;
  const float q_scale = 1.0f / sqrtf((float)D);
#define LAUNCH(C, L, MODE)                                                                                        \
  gla_kernel<C, L><<<grid, threads, lds, (hipStream_t)stream>>>(                                                  \
      (const act_t*)qkv, ld, k_off, v_off, (const act_t*)g, ldg, z, ldz, z_bias, 1.0f / tau, gain, state,        \
      slot_words, offset_words, q_start, slot_of_req, (act_t*)out, raw_arg, H, D, E, eps, q_scale, cols, MODE,   \
      seg_len, nseg, seg_state, seg_decay, segmented ? 1 : 0)
#define WALK(MODE)                                                                                                \
  do {                                                                                                            \
    if (DMAX == 32) LAUNCH(1, 8, MODE);                                                                           \
    else if (DMAX == 64) LAUNCH(2, 8, MODE);                                                                      \
    else if (DMAX == 128) LAUNCH(4, 8, MODE);                                                                     \
    else LAUNCH(4, 16, MODE);                                                                                     \
  } while (0)
  if (segmented) {
    // z is the caller's scratch: its rows become the decays themselves
    gla_decays_kernel<<<(unsigned)(((size_t)T * H * D + 255) / 256), 256, 0, (hipStream_t)stream>>>(z, ldz, z_bias, 1.0f / tau,
                                                                                                   T, H * D);
    WALK(1);
    dim3 sg((unsigned)(((size_t)H * D * E + 255) / 256), R);
    gla_segments_kernel<<<sg, 256, 0, (hipStream_t)stream>>>(seg_state, seg_decay, state, slot_words, offset_words,
                                                             q_start, slot_of_req, seg_len, nseg, H, D, E);
    WALK(2);
  } else {
    WALK(0);
  }
#undef WALK
#undef LAUNCH
  if (blocks_e > 1) {
    dim3 fg(T, H);
    gla_finish_kernel<<<fg, 64, 0, (hipStream_t)stream>>>(raw, (const act_t*)g, ldg, gain, positions, (act_t*)out, H, E, eps);
  }
  return zk_launch_status("zk_gla");
}

}  // extern "C"

ZK_ENTER(zk_gla)
