// An embedding of token pairs added to the embedded rows.
//
//   x_t += pair[(prev_t * mul_prev + token_t * mul_cur) mod buckets]      (row ``buckets`` for a
//                                                                           sequence's first token)
//
// prev_t is the token before t in its sequence.  Inside a step it is the step's own token t - 1;
// for the first token that a request brings it is the last token of the step before, which the
// request keeps in its state slot (one int32).  ``zk_prev_token`` reads that word for every request
// of the step and puts the request's last token of this step in its place: one thread a request
// does both, so nothing is read after another thread wrote it.  The sum is float.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

__global__ void prev_token_kernel(const int* __restrict__ tokens, const int* __restrict__ q_start,
                                  const int* __restrict__ slot_of_req, int* __restrict__ state, size_t slot_words,
                                  size_t word, int* __restrict__ prev_first, int R) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= R) return;
  const int a = q_start[r], b = q_start[r + 1];
  if (b <= a) {                        // a padding request
    prev_first[r] = 0;
    return;
  }
  int* p = state + (size_t)slot_of_req[r] * slot_words + word;
  prev_first[r] = *p;
  *p = tokens[b - 1];
}

__global__ void add_pair_rows_kernel(float* __restrict__ out, const act_t* __restrict__ table,
                                     const int* __restrict__ tokens, const int* __restrict__ positions,
                                     const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                     const int* __restrict__ prev_first, int buckets, long long mul_prev,
                                     long long mul_cur, int H) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  long long row = buckets;             // a sequence's first token (and padding rows, whose result nobody reads)
  if (pos > 0) {
    const int r = req_of_token[t];
    const long long prev = t > q_start[r] ? tokens[t - 1] : prev_first[r];
    row = (prev * mul_prev + (long long)tokens[t] * mul_cur) % buckets;
    if (row < 0) row += buckets;
  }
  const act_t* src = table + (size_t)row * H;
  float* dst = out + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] += to_f32(src[i]);
}

extern "C" {

// state: the runner's state slots as 32-bit words, ``slot_words`` a slot; ``word``: where in a slot
// the previous token lies.  prev_first: int32 [R], the token before each request's first of this step.
int zk_prev_token(const int* tokens, const int* q_start, const int* slot_of_req, void* state, size_t slot_words,
                  size_t word, void* prev_first, int R, void* stream) {
  ZK_REQUIRE(R >= 0 && state != nullptr && prev_first != nullptr && word < slot_words, "zk_prev_token: bad arguments");
  if (R == 0) return 0;
  prev_token_kernel<<<(R + 63) / 64, 64, 0, (hipStream_t)stream>>>(tokens, q_start, slot_of_req, (int*)state, slot_words, word,
                                                                  (int*)prev_first, R);
  return zk_launch_status("zk_prev_token");
}

// out: float [T, H]; table: [buckets + 1, H] in the storage type, row-major.
int zk_add_pair_rows(float* out, const void* table, const int* tokens, const int* positions, const int* req_of_token,
                     const int* q_start, const void* prev_first, int buckets, int mul_prev, int mul_cur, int T, int H,
                     void* stream) {
  ZK_REQUIRE(T >= 0 && H > 0 && buckets > 0, "zk_add_pair_rows: bad sizes");
  if (T == 0) return 0;
  add_pair_rows_kernel<<<T, 256, 0, (hipStream_t)stream>>>(out, (const act_t*)table, tokens, positions, req_of_token, q_start,
                                                          (const int*)prev_first, buckets, mul_prev, mul_cur, H);
  return zk_launch_status("zk_add_pair_rows");
}

}  // extern "C"

ZK_ENTER(zk_prev_token)
ZK_ENTER(zk_add_pair_rows)
