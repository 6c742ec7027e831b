// Attention over one latent row per token.
//
// A token leaves c = rms_norm(first C channels of its down-projection) * gain and one rotated key
// part of R channels; head h's key would be [Wuk_h c, rotated part] and its value Wuv_h c.  Only
// [c, rotated part] is cached (one "key head" of C + R channels).  Because
//     q_plain . (Wuk_h c) = (Wuk_h^T q_plain) . c      and      sum_j p_j (Wuv_h c_j) = Wuv_h (sum_j p_j c_j)
// a query head becomes [Wuk_h^T q_plain, q_rotated] (C + R channels), attends to the cached rows
// as keys and to their first C channels as values, and the result goes through Wuv_h.  The two
// per-head products are ``zk_heads_linear``; ``zk_latent_prep`` norms, rotates and stores.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

// One block per (token, head or latent).  Heads: the rotated part of the query goes, rotated, to
// qa[t, head, C:].  The latent (blockIdx.y == H): the normed c and the rotated key part go to
// the cache row of the token's slot.
__global__ __launch_bounds__(256) void latent_prep_kernel(
    const act_t* __restrict__ qd, int ld, const act_t* __restrict__ down, int ldd, const int* __restrict__ positions,
    const int* __restrict__ slot_map, const float* __restrict__ gain, float eps, const float* __restrict__ freq,
    float rot_scale, int interleaved, act_t* __restrict__ qa, act_t* __restrict__ kcache, int H, int D, int R, int C,
    int bs) {
  __shared__ float red[17];
  const int t = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int half = R / 2;
  if (head < H) {
    const act_t* src = qd + (size_t)t * ld + (size_t)head * (D + R) + D;
    act_t* dst = qa + ((size_t)t * H + head) * (C + R) + C;
    for (int m = tid; m < half; m += 256) {
      float sn, cs, ra, rb;
      sincosf((float)pos * freq[m], &sn, &cs);
      sn *= rot_scale;
      cs *= rot_scale;
      const int ia = interleaved ? 2 * m : m, ib = interleaved ? 2 * m + 1 : m + half;
      rotate_pair(to_f32(src[ia]), to_f32(src[ib]), sn, cs, ra, rb);
      dst[ia] = from_f32<act_t>(ra);
      dst[ib] = from_f32<act_t>(rb);
    }
    return;
  }
  const int slot = slot_map[t];
  if (slot < 0) return;
  const act_t* src = down + (size_t)t * ldd;
  act_t* dst = kcache + (size_t)slot * (C + R);           // one key head: row (page * bs + offset)
  float ss = 0.f;
  for (int i = tid; i < C; i += 256) {
    const float x = to_f32(src[i]);
    ss = fmaf(x, x, ss);
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)C + eps);
  for (int i = tid; i < C; i += 256) dst[i] = from_f32<act_t>(to_f32(src[i]) * inv * gain[i]);
  for (int m = tid; m < half; m += 256) {
    float sn, cs, ra, rb;
    sincosf((float)pos * freq[m], &sn, &cs);
    sn *= rot_scale;
    cs *= rot_scale;
    const int ia = interleaved ? 2 * m : m, ib = interleaved ? 2 * m + 1 : m + half;
    rotate_pair(to_f32(src[C + ia]), to_f32(src[C + ib]), sn, cs, ra, rb);
    dst[C + ia] = from_f32<act_t>(ra);
    dst[C + ib] = from_f32<act_t>(rb);
  }
}

// out[t, h, n] = sum_k x[t, h, k] w_h(n, k);  w_h(n, k) = w[(h K + k) N + n] (kn) or w[(h N + n) K + k].
// A block: 32 tokens x 64 columns of one head; a thread: 8 tokens of one column.
#define HL_TT 32
#define HL_TK 32
template <bool KN>
__global__ __launch_bounds__(256) void heads_linear_kernel(const act_t* __restrict__ x, int ldx, int x_head,
                                                           const act_t* __restrict__ w, act_t* __restrict__ out, int ldo,
                                                           int o_head, int T, int K, int N) {
  __shared__ float xs[HL_TT][HL_TK + 1];
  __shared__ float ws[HL_TK][64 + 1];
  const int h = blockIdx.y, t0 = blockIdx.x * HL_TT, n0 = blockIdx.z * 64;
  const int tid = threadIdx.x, tx = tid & 63, ty = tid >> 6;
  const act_t* wh = w + (size_t)h * K * N;
  float acc[8] = {};
  for (int k0 = 0; k0 < K; k0 += HL_TK) {
    __syncthreads();
    for (int i = tid; i < HL_TT * HL_TK; i += 256) {
      const int tt = i / HL_TK, kk = i % HL_TK;
      xs[tt][kk] = (t0 + tt < T && k0 + kk < K) ? to_f32(x[(size_t)(t0 + tt) * ldx + (size_t)h * x_head + k0 + kk]) : 0.f;
    }
    for (int i = tid; i < HL_TK * 64; i += 256) {
      int kk, nn;
      if (KN) {
        kk = i / 64;
        nn = i % 64;
      } else {
        nn = i / HL_TK;
        kk = i % HL_TK;
      }
      const bool in = k0 + kk < K && n0 + nn < N;
      ws[kk][nn] = in ? to_f32(KN ? wh[(size_t)(k0 + kk) * N + n0 + nn] : wh[(size_t)(n0 + nn) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < HL_TK; kk++) {
      const float wv = ws[kk][tx];
#pragma unroll
      for (int j = 0; j < 8; j++) acc[j] = fmaf(xs[ty * 8 + j][kk], wv, acc[j]);
    }
  }
  if (n0 + tx < N) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int t = t0 + ty * 8 + j;
      if (t < T) out[(size_t)t * ldo + (size_t)h * o_head + n0 + tx] = from_f32<act_t>(acc[j]);
    }
  }
}

// The same for steps of few tokens: a thread per column n, a block per (token, head, 64 columns);
// the sum over k runs in the same order as in the tiled kernel, so a row's values are the same
// bits whichever of the two computes it.
template <bool KN>
__global__ __launch_bounds__(64) void heads_linear_few_kernel(const act_t* __restrict__ x, int ldx, int x_head,
                                                              const act_t* __restrict__ w, act_t* __restrict__ out, int ldo,
                                                              int o_head, int K, int N) {
  extern __shared__ float xrow[];                    // [K]
  const int t = blockIdx.x, h = blockIdx.y, n = blockIdx.z * 64 + threadIdx.x;
  const act_t* xr = x + (size_t)t * ldx + (size_t)h * x_head;
  for (int k = threadIdx.x; k < K; k += 64) xrow[k] = to_f32(xr[k]);
  __syncthreads();
  if (n >= N) return;
  const act_t* wh = w + (size_t)h * K * N;
  float acc = 0.f;
  if (KN) {
    for (int k = 0; k < K; k++) acc = fmaf(xrow[k], to_f32(wh[(size_t)k * N + n]), acc);
  } else {
    const act_t* wr = wh + (size_t)n * K;
    for (int k = 0; k < K; k++) acc = fmaf(xrow[k], to_f32(wr[k]), acc);
  }
  out[(size_t)t * ldo + (size_t)h * o_head + n] = from_f32<act_t>(acc);
}

extern "C" {

// qd: [T, ld]: H query heads of D + R, then C + R of the down-projection.  qa: [T, H, C + R], of
// which this writes [.., C:].  kcache: [pages, 1, bs, C + R].  freq: float [R / 2].
// q: [T, ldq], H query heads of D + R; down: [T, ldd], C + R of the down-projection, wherever the
// two lie.
int zk_latent_prep_ext(const void* q, int ldq, const void* down, int ldd, const int* positions, const int* slot_map,
                       const float* gain, float eps, const float* freq, float rot_scale, int interleaved, void* qa,
                       void* kcache, int T, int H, int D, int R, int C, int bs, void* stream) {
  ZK_REQUIRE(T >= 0 && H > 0 && D > 0 && R >= 0 && R % 2 == 0 && C > 0 && bs > 0, "zk_latent_prep: bad sizes");
  ZK_REQUIRE(ldq >= H * (D + R) && ldd >= C + R, "zk_latent_prep: rows too short");
  ZK_REQUIRE(H < 65535 && (R == 0 || freq != nullptr), "zk_latent_prep: too many heads, or no frequencies");
  if (T == 0) return 0;
  dim3 grid(T, H + 1);
  latent_prep_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)q, ldq, (const act_t*)down, ldd, positions, slot_map,
                                                            gain, eps, freq, rot_scale, interleaved, (act_t*)qa,
                                                            (act_t*)kcache, H, D, R, C, bs);
  return zk_launch_status("zk_latent_prep");
}

int zk_latent_prep(const void* qd, int ld, const int* positions, const int* slot_map, const float* gain, float eps,
                   const float* freq, float rot_scale, int interleaved, void* qa, void* kcache, int T, int H, int D,
                   int R, int C, int bs, void* stream) {
  ZK_REQUIRE(H > 0 && D > 0 && R >= 0 && C > 0 && ld >= H * (D + R) + C + R, "zk_latent_prep: rows too short");
  return zk_latent_prep_ext(qd, ld, (const act_t*)qd + (size_t)H * (D + R), ld, positions, slot_map, gain, eps, freq,
                            rot_scale, interleaved, qa, kcache, T, H, D, R, C, bs, stream);
}

// x: head h of token t at x[t * ldx + h * x_head], K channels; out likewise with ldo, o_head, N.
// w: [H][K][N] when w_kn, else [H][N][K].
int zk_heads_linear(const void* x, int ldx, int x_head, const void* w, int w_kn, void* out, int ldo, int o_head, int T,
                    int H, int K, int N, void* stream) {
  ZK_REQUIRE(T >= 0 && H > 0 && K > 0 && N > 0, "zk_heads_linear: bad sizes");
  ZK_REQUIRE(H <= 65535 && (N + 63) / 64 <= 65535, "zk_heads_linear: too many heads or columns");
  if (T == 0) return 0;
  if (T <= 16 && K <= 8192) {
    dim3 few(T, H, (N + 63) / 64);
    if (w_kn)
      heads_linear_few_kernel<true><<<few, 64, (size_t)K * 4, (hipStream_t)stream>>>((const act_t*)x, ldx, x_head, (const act_t*)w,
                                                                                    (act_t*)out, ldo, o_head, K, N);
    else
      heads_linear_few_kernel<false><<<few, 64, (size_t)K * 4, (hipStream_t)stream>>>((const act_t*)x, ldx, x_head, (const act_t*)w,
                                                                                     (act_t*)out, ldo, o_head, K, N);
    return zk_launch_status("zk_heads_linear");
  }
  dim3 grid((T + HL_TT - 1) / HL_TT, H, (N + 63) / 64);
  if (w_kn)
    heads_linear_kernel<true><<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)x, ldx, x_head, (const act_t*)w,
                                                                     (act_t*)out, ldo, o_head, T, K, N);
  else
    heads_linear_kernel<false><<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)x, ldx, x_head, (const act_t*)w,
                                                                      (act_t*)out, ldo, o_head, T, K, N);
  return zk_launch_status("zk_heads_linear");
}

}  // extern "C"

ZK_ENTER(zk_latent_prep)
ZK_ENTER(zk_latent_prep_ext)
ZK_ENTER(zk_heads_linear)

#if ZSE_ACT_BF16
// ---- the attention itself on the matrix cores (bfloat16)
// Every head of a token reads the same cached rows, so the rows of the first product are
// (token, head) pairs: row i of a request's step is head i % H of its token i / H.  A block takes
// up to 128 such rows (a wave 32 of them) and walks the keys in tiles of 32 that all its waves
// share through local memory, once as they lie (for S^T = K Q^T) and once transposed (their first
// C channels are the values: O^T += V^T P^T).  Both products keep a row in a fixed lane (column =
// lane % 32), so the running maximum and sum are per-lane numbers, and the weights a lane holds
// after the first product are its operand of the second: the order of the keys in that product
// is permuted to match (slots e < 4 of lane half h are keys 4h + e, slots e >= 4 keys 8 + 4h + e - 4).
// Few rows behind long contexts: the keys are cut into ranges over blockIdx.z, every block
// leaves (max, sum, O) of its range and a second kernel joins them; the sink enters there.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));

#define LA_ROWS 128
#define LA_VT_LD 40

template <int DT>
__global__ __launch_bounds__(256) void latent_attn_kernel(
    const __bf16* __restrict__ qa, const __bf16* __restrict__ kcache, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, const float* __restrict__ sinks,
    __bf16* __restrict__ out, float* __restrict__ part, int H, int HD, int C, int HDP, int bs, float scale, int splits,
    int split_keys, int window, int wide) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int LDK = HDP + 8;
  __bf16* Ks = (__bf16*)smem;                       // [32][LDK]
  __bf16* Vt = Ks + 32 * LDK;                       // [DT * 32][LA_VT_LD]
  __bf16* Qs = Vt + DT * 32 * LA_VT_LD;             // [LA_ROWS][LDK]
  const int r = blockIdx.y, split = blockIdx.z;
  const int t0 = q_start[r], n_q = q_start[r + 1] - t0;
  if (n_q <= 0) return;
  const int rows = n_q * H, row0 = blockIdx.x * LA_ROWS;
  if (row0 >= rows) return;
  const int ctx = ctx_len[r];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 31, lh = lane >> 5;
  const int pieces = HDP / 8;
  const int* table = block_table + (size_t)r * max_blocks;
  const int staged = min(LA_ROWS, (rows - row0 + 31) / 32 * 32);      // the rows of waves that have any
  for (int i = tid; i < staged * pieces; i += 256) {
    const int row = i / pieces, c8 = (i % pieces) * 8;
    bf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row0 + row < rows && c8 < HD) v = *(const bf16x8_t*)(qa + ((size_t)t0 * H + row0 + row) * HD + c8);
    *(bf16x8_t*)(Qs + row * LDK + c8) = v;
  }
  const int wrow = row0 + wave * 32 + lr;
  const int my_pos = wrow < rows ? ctx - n_q + wrow / H : -1;
  // with a window a row sees the keys [my_lo, my_pos]; the block begins at the tile that holds the
  // first key of its first row (pages before it may have gone back to the pool: the table names none)
  const int my_lo = window > 0 ? max(my_pos - window + 1, 0) : 0;
  const int block_lo = window > 0 ? max(ctx - n_q + row0 / H - window + 1, 0) / 32 * 32 : 0;
  const bool wave_live = row0 + wave * 32 < rows;
  const int last_row = min(rows, row0 + LA_ROWS) - 1;
  // the ranges of a split count from the block's first tile
  const int k_begin = block_lo + split * split_keys;
  const int k_end = min(ctx - n_q + last_row / H + 1, block_lo + (split + 1) * split_keys);      // exclusive
  float m = -INFINITY, l = 0.f;
  floatx16_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) o[dt][e] = 0.f;
  // a tile's pieces travel from memory into registers while the tile before it is multiplied
  constexpr int PRE = 5;                               // 16-byte pieces a thread carries: 32 x HDP / 8 / 256 <= 5 (HDP <= 320)
  bf16x8_t nxt[PRE];
  auto fetch = [&](int key0) {
#pragma unroll
    for (int u = 0; u < PRE; u++) {
      // consecutive threads take consecutive keys of one column of pieces: the transposed copy is
      // then written to consecutive addresses
      const int i = tid + u * 256;
      const int kk = i & 31, c8 = (i >> 5) * 8, key = key0 + kk;
      bf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (i < 32 * pieces && key < k_end && c8 < HD) {
        const int page = table[key / bs];
        if (page >= 0) v = *(const bf16x8_t*)(kcache + ((size_t)page * bs + key % bs) * HD + c8);
      }
      nxt[u] = v;
    }
  };
  if (k_begin < k_end) fetch(k_begin);
  for (int key0 = k_begin; key0 < k_end; key0 += 32) {
    __syncthreads();                                 // the last tile has been used (and Q is in place)
#pragma unroll
    for (int u = 0; u < PRE; u++) {
      const int i = tid + u * 256;
      if (i < 32 * pieces) {
        const int kk = i & 31, c8 = (i >> 5) * 8;
        const bf16x8_t v = nxt[u];
        *(bf16x8_t*)(Ks + kk * LDK + c8) = v;
        if (c8 < DT * 32) {
#pragma unroll
          for (int j = 0; j < 8; j++) Vt[(c8 + j) * LA_VT_LD + kk] = (c8 + j < C) ? v[j] : (__bf16)0.f;
        }
      }
    }
    __syncthreads();
    if (key0 + 32 < k_end) fetch(key0 + 32);
    if (!wave_live) continue;
    floatx16_t s;
#pragma unroll
    for (int e = 0; e < 16; e++) s[e] = 0.f;
    const __bf16* ka = Ks + lr * LDK + lh * 8;
    const __bf16* qb = Qs + (wave * 32 + lr) * LDK + lh * 8;
    for (int ks = 0; ks < HDP / 16; ks++)
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)(ka + ks * 16), *(const bf16x8_t*)(qb + ks * 16), s, 0, 0, 0);
    float mt = -INFINITY;
#pragma unroll
    for (int e = 0; e < 16; e++) {
      const int key = key0 + (e / 4) * 8 + lh * 4 + (e % 4);
      const bool seen = key <= my_pos && key >= my_lo && key < k_end;
      s[e] = seen ? s[e] * scale : -INFINITY;
      mt = fmaxf(mt, s[e]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m, mt);
    const float corr = (m_new == -INFINITY) ? 1.f : __expf(m - m_new);
    float p[16], ps = 0.f;
#pragma unroll
    for (int e = 0; e < 16; e++) {
      p[e] = (s[e] == -INFINITY) ? 0.f : __expf(s[e] - m_new);
      ps += p[e];
    }
    ps += __shfl_xor(ps, 32, 64);
    l = l * corr + ps;
    m = m_new;
    bf16x8_t pb0, pb1, pr0, pr1;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      pb0[e] = (__bf16)p[e];
      pb1[e] = (__bf16)p[8 + e];
    }
    if (wide) {
      // a weight meets the values as two bfloat16 numbers: its rounded value and what the rounding left
#pragma unroll
      for (int e = 0; e < 8; e++) {
        pr0[e] = (__bf16)(p[e] - (float)pb0[e]);
        pr1[e] = (__bf16)(p[8 + e] - (float)pb1[e]);
      }
    }
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
#pragma unroll
      for (int e = 0; e < 16; e++) o[dt][e] *= corr;
      const __bf16* vr = Vt + (dt * 32 + lr) * LA_VT_LD + 4 * lh;
      const bf16x4_t a0 = *(const bf16x4_t*)vr, a1 = *(const bf16x4_t*)(vr + 8);
      const bf16x4_t a2 = *(const bf16x4_t*)(vr + 16), a3 = *(const bf16x4_t*)(vr + 24);
      bf16x8_t va, vb;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        va[e] = a0[e];
        va[4 + e] = a1[e];
        vb[e] = a2[e];
        vb[4 + e] = a3[e];
      }
      o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb0, o[dt], 0, 0, 0);
      o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vb, pb1, o[dt], 0, 0, 0);
      if (wide) {
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pr0, o[dt], 0, 0, 0);
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vb, pr1, o[dt], 0, 0, 0);
      }
    }
  }
  if (!wave_live || wrow >= rows) return;
  const size_t grow = (size_t)t0 * H + wrow;          // the row's number in the step
  if (splits > 1) {
    const int CP = DT * 32;
    float* pr = part + (grow * splits + split) * (size_t)(CP + 2);
    if (lh == 0) {
      pr[0] = m;
      pr[1] = l;
    }
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int e = 0; e < 16; e++) pr[2 + dt * 32 + (e / 4) * 8 + lh * 4 + (e % 4)] = o[dt][e];
    return;
  }
  if (sinks != nullptr) {
    const float sk = sinks[wrow % H];
    const float m_new = fmaxf(m, sk);
    const float corr = __expf(m - m_new);
    l = l * corr + __expf(sk - m_new);
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int e = 0; e < 16; e++) o[dt][e] *= corr;
  }
  const float inv = 1.f / l;
  __bf16* orow = out + grow * C;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) {
      const int d = dt * 32 + (e / 4) * 8 + lh * 4 + (e % 4);
      if (d < C) orow[d] = (__bf16)(o[dt][e] * inv);
    }
}

// One block per row of the step: joins the ranges' (max, sum, O), adds the sink.
__global__ __launch_bounds__(256) void latent_join_kernel(const float* __restrict__ part, const float* __restrict__ sinks,
                                                          const int* __restrict__ positions, __bf16* __restrict__ out, int H,
                                                          int C, int CP, int splits) {
  __shared__ float wgt[64];
  __shared__ float inv_den;
  const size_t row = blockIdx.x;
  __bf16* orow = out + row * C;
  if (positions[row / H] < 0) {                      // a padding row of a captured step
    for (int c = threadIdx.x; c < C; c += blockDim.x) orow[c] = (__bf16)0.f;
    return;
  }
  const float* pr = part + row * splits * (size_t)(CP + 2);
  if (threadIdx.x < 64) {                            // one wave: the ranges' weights exp(m_s - M) and the denominator
    const int s = threadIdx.x;
    const float ms = s < splits ? pr[(size_t)s * (CP + 2)] : -INFINITY;
    const float ls = s < splits ? pr[(size_t)s * (CP + 2) + 1] : 0.f;
    const float sk = sinks ? sinks[row % H] : -INFINITY;
    const float M = fmaxf(wave_max(ms), sk);
    const float w = ms > -INFINITY ? __expf(ms - M) : 0.f;
    const float den = wave_sum(ls * w) + (sinks ? __expf(sk - M) : 0.f);
    wgt[s] = w;
    if (s == 0) inv_den = 1.f / den;
  }
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float acc = 0.f;
    for (int s = 0; s < splits; s++) acc = fmaf(pr[(size_t)s * (CP + 2) + 2 + c], wgt[s], acc);
    orow[c] = (__bf16)(acc * inv_den);
  }
}

extern "C" {

// Whether the matrix-core kernel takes rows of HD channels of which the first C are values.
int zk_latent_attention_bf16_supports(int HD, int C, int bs) {
  return HD % 8 == 0 && HD <= 320 && C <= 256 && C <= HD && bs > 0;
}

// Floats of workspace that let a step of T tokens cut its keys into up to ``splits`` ranges.
size_t zk_latent_attention_bf16_workspace(int T, int H, int C, int splits) {
  const int CP = C <= 64 ? 64 : C <= 128 ? 128 : 256;
  return (size_t)T * H * splits * (CP + 2) * sizeof(float);
}

// qa: [T, H, HD] queries carried over to the cached rows' channels; kcache: [pages, 1, bs, HD];
// out: [T, H, C].  Request r holds rows [q_start[r], q_start[r + 1]) and ends at position
// ctx_len[r] - 1.  max_q_len, max_ctx: the longest portion and context of the step (they size
// the grid).  work: float scratch of work_bytes (may be null: no ranges).
// window > 0: a row at position p sees the keys [max(0, p - window + 1), p] only.  wide: the softmax's
// weights keep 16 bits of mantissa in the product with the values (two bfloat16 numbers a weight).
int zk_latent_attention_bf16_window(const void* qa, const void* kcache, const int* block_table, int max_blocks,
                                    const int* q_start, const int* ctx_len, const int* positions, const float* sinks,
                                    void* out, void* work, size_t work_bytes, int T, int R, int max_q_len, int max_ctx, int H,
                                    int HD, int C, int bs, float scale, int window, int wide, void* stream) {
  ZK_REQUIRE(T >= 0 && R >= 0 && H > 0 && max_q_len > 0 && max_ctx > 0 && max_blocks > 0, "zk_latent_attention_bf16: bad sizes");
  ZK_REQUIRE(zk_latent_attention_bf16_supports(HD, C, bs), "zk_latent_attention_bf16: rows of up to 320 channels in eights, up to 256 of them values");
  ZK_REQUIRE(R <= 65535, "zk_latent_attention_bf16: too many requests");
  if (T == 0 || R == 0) return 0;
  const int HDP = (HD + 15) / 16 * 16;
  const int DT = C <= 64 ? 2 : C <= 128 ? 4 : 8;
  const int groups = (int)(((size_t)max_q_len * H + LA_ROWS - 1) / LA_ROWS);
  int splits = 1;
  const int blocks = groups * R;
  // the keys a block walks: with a window, those of its rows' windows (and the tile they begin in)
  const int keys = window > 0 ? min(max_ctx, window + (LA_ROWS + H - 1) / H + 32) : max_ctx;
  if (blocks < 128 && work != nullptr) {
    // (with a window, ranges that lie before it are empty: only those over the window's keys count)
    splits = (256 + blocks - 1) / blocks;
    splits = min(splits, (keys + 127) / 128);
    splits = min(splits, 64);
    while (splits > 1 && zk_latent_attention_bf16_workspace(T, H, C, splits) > work_bytes) splits--;
    splits = max(splits, 1);
  }
  const int split_keys = splits == 1 ? 0x40000000 : ((keys + splits - 1) / splits + 31) / 32 * 32;
  const size_t lds = ((size_t)32 * (HDP + 8) + (size_t)DT * 32 * LA_VT_LD + (size_t)LA_ROWS * (HDP + 8)) * sizeof(__bf16);
  dim3 grid(groups, R, splits);
  hipStream_t st = (hipStream_t)stream;
#define LA_LAUNCH(N)                                                                                                   \
  do {                                                                                                                 \
    static bool raised = false;                                                                                        \
    if (!raised) {                                                                                                     \
      hipFuncSetAttribute((const void*)latent_attn_kernel<N>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
      raised = true;                                                                                                   \
    }                                                                                                                  \
    latent_attn_kernel<N><<<grid, 256, lds, st>>>((const __bf16*)qa, (const __bf16*)kcache, block_table, max_blocks,   \
                                                  q_start, ctx_len, sinks, (__bf16*)out, (float*)work, H, HD, C, HDP,  \
                                                  bs, scale, splits, split_keys, window, wide);                        \
  } while (0)
  if (DT == 2) LA_LAUNCH(2);
  else if (DT == 4) LA_LAUNCH(4);
  else LA_LAUNCH(8);
#undef LA_LAUNCH
  if (splits > 1)
    latent_join_kernel<<<T * H, 256, 0, st>>>((const float*)work, sinks, positions, (__bf16*)out, H, C, DT * 32, splits);
  return zk_launch_status("zk_latent_attention_bf16");
}

int zk_latent_attention_bf16(const void* qa, const void* kcache, const int* block_table, int max_blocks,
                             const int* q_start, const int* ctx_len, const int* positions, const float* sinks, void* out,
                             void* work, size_t work_bytes, int T, int R, int max_q_len, int max_ctx, int H, int HD, int C,
                             int bs, float scale, void* stream) {
  return zk_latent_attention_bf16_window(qa, kcache, block_table, max_blocks, q_start, ctx_len, positions, sinks, out, work,
                                         work_bytes, T, R, max_q_len, max_ctx, H, HD, C, bs, scale, 0, 0, stream);
}

}  // extern "C"

ZK_ENTER(zk_latent_attention_bf16)
ZK_ENTER(zk_latent_attention_bf16_window)
#endif
