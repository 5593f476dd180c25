// A mixture of experts' router and the weighting of the experts' middle activations.
//
// route_kernel: a wave per token.  From the router's logits z [T, E] (32-bit sums of the projection) plus a bias
// it picks the `top` largest (of equal logits the lower index), takes the softmax over the picked logits only, and
// writes a dense row of weights [E]: the picked experts' weights, zero elsewhere.  All in 32-bit.
//
// scale_columns_kernel: y[t, e F + j] = x[t, e F + j] * w[t, e] for rows made of E parts of F columns: the experts'
// middle activations side by side, each multiplied by its expert's weight of that token (a zero for an expert that
// the token does not use), so that one down projection over all parts gives the weighted sum of the experts.
#include "common.h"
#include "alice_hip.h"

namespace {

constexpr int MAX_EXPERTS = 1024;

__global__ __launch_bounds__(64) void route_kernel(const float* __restrict__ z, const float* __restrict__ bias, float* __restrict__ w,
                                                   int E, int top) {
  __shared__ float zs[MAX_EXPERTS];
  __shared__ float ws[MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) {
    zs[e] = z[(size_t)t * E + e] + (bias ? bias[e] : 0.f);
    ws[e] = 0.f;
  }
  __syncthreads();
  float first = 0.f, sum = 0.f;
  for (int n = 0; n < top; ++n) {
    float best = -INFINITY;
    int at = E;
    for (int e = lane; e < E; e += 64)
      if (ws[e] == 0.f && (zs[e] > best || (zs[e] == best && e < at))) { best = zs[e]; at = e; }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oa = __shfl_xor(at, o, 64);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (at >= E) break;                                // (only if every logit is NaN)
    if (n == 0) first = best;
    const float p = expf(best - first);                // the first pick is the largest: exponents are never positive
    sum += p;
    __syncthreads();
    if (lane == 0) ws[at] = p;
    __syncthreads();
  }
  const float inv = sum > 0.f ? 1.f / sum : 0.f;
  for (int e = lane; e < E; e += 64) w[(size_t)t * E + e] = ws[e] * inv;
}

template <typename TI, typename TO>
__global__ void scale_columns_kernel(const TI* __restrict__ x, const float* __restrict__ w, TO* __restrict__ y, long n, int E, int F) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long t = i / ((long)E * F);
    const int e = (int)((i / F) % E);
    store_f32(y, (size_t)i, load_f32(x, (size_t)i) * w[t * E + e]);
  }
}

}  // namespace

extern "C" int alice_route_topk(const float* z, const float* bias, float* w, int T, int E, int top, hipStream_t stream) {
  ALICE_CHECK(z && w, "route_topk: a pointer is missing");
  ALICE_CHECK(T >= 0 && E >= 1 && E <= MAX_EXPERTS && top >= 1 && top <= E, "route_topk: 1 <= top <= experts <= %d", MAX_EXPERTS);
  if (T == 0) return 0;
  route_kernel<<<T, 64, 0, stream>>>(z, bias, w, E, top);
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_scale_columns(const void* x, int x_dtype, const float* w, void* y, int y_dtype, int T, int E, int F,
                                   hipStream_t stream) {
  ALICE_CHECK(x && w && y && dtype_ok(x_dtype) && dtype_ok(y_dtype), "scale_columns: a pointer is missing or a dtype is unknown");
  ALICE_CHECK(T >= 0 && E >= 1 && F >= 1, "scale_columns: bad sizes");
  const long n = (long)T * E * F;
  if (n == 0) return 0;
  const int blocks = (int)((n + 255) / 256 < (1L << 20) ? (n + 255) / 256 : (1L << 20));      // beyond that a thread takes several elements
#define GO(TI, TO) scale_columns_kernel<TI, TO><<<blocks, 256, 0, stream>>>((const TI*)x, w, (TO*)y, n, E, F)
  if (x_dtype == DT_F32 && y_dtype == DT_F32) GO(float, float);
  else if (x_dtype == DT_F32) GO(float, bf16_t);
  else if (y_dtype == DT_F32) GO(bf16_t, float);
  else GO(bf16_t, bf16_t);
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}
