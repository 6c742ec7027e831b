// Element by element: an activation without a gate, and a gate on the heads of a mixer.
//
//   zk_unary_act:   out = act(x)                        act 0: max(x, 0)^2
//   zk_gate_heads:  o <- o * sigmoid(g)                 g read from rows of another width; one g
//                                                       for every ``per`` channels (a number a head)
//
// Arithmetic is float; one rounding to the activation type at the store.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

__global__ void unary_act_kernel(const act_t* __restrict__ x, act_t* __restrict__ out, size_t n, int act) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float v = fmaxf(to_f32(x[i]), 0.f);
  out[i] = from_f32<act_t>(v * v);
}

__global__ void gate_heads_kernel(act_t* __restrict__ o, const act_t* __restrict__ g, int ldg, int W, int per) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= W) return;
  const float z = to_f32(g[(size_t)t * ldg + i / per]);
  const size_t at = (size_t)t * W + i;
  o[at] = from_f32<act_t>(to_f32(o[at]) / (1.0f + expf(-z)));
}

extern "C" {

// x, out: n activations.  act: 0 = the square of relu.
int zk_unary_act(const void* x, void* out, size_t n, int act, void* stream) {
  ZK_REQUIRE(act == 0, "zk_unary_act: unknown activation");
  if (n == 0) return 0;
  ZK_REQUIRE((n + 255) / 256 < 2147483647ull, "zk_unary_act: too many elements");
  unary_act_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>((const act_t*)x, (act_t*)out, n, act);
  return zk_launch_status("zk_unary_act");
}

// o: [T, W] activations, multiplied in place by sigmoid(g[t, i]); g: rows ldg apart.
// per: the channels that share one gate value (1: a value a channel; a head's size: a value a head).
int zk_gate_heads_per(void* o, const void* g, int ldg, int T, int W, int per, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && per > 0 && W % per == 0 && ldg >= W / per && g != nullptr, "zk_gate_heads: bad sizes");
  ZK_REQUIRE(T <= 65535, "zk_gate_heads: more than 65535 rows");
  if (T == 0) return 0;
  dim3 grid((W + 255) / 256, T);
  gate_heads_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((act_t*)o, (const act_t*)g, ldg, W, per);
  return zk_launch_status("zk_gate_heads");
}

int zk_gate_heads(void* o, const void* g, int ldg, int T, int W, void* stream) {
  return zk_gate_heads_per(o, g, ldg, T, W, 1, stream);
}

}  // extern "C"

ZK_ENTER(zk_unary_act)
ZK_ENTER(zk_gate_heads)
ZK_ENTER(zk_gate_heads_per)
