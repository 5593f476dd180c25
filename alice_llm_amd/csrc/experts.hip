// A mixture of experts' router and the weighting of the experts' middle activations.
//
// route_kernel: a wave per token.  From the router's logits z [T, E] (32-bit sums of the projection) plus a bias
// it picks the `top` largest (of equal logits the lower index), takes the softmax over the picked logits only, and
// writes a dense row of weights [E]: the picked experts' weights, zero elsewhere.  All in 32-bit.
//
// scale_columns_kernel: y[t, e F + j] = x[t, e F + j] * w[t, e] for rows made of E parts of F columns: the experts'
// middle activations side by side, each multiplied by its expert's weight of that token (a zero for an expert that
// the token does not use), so that one down projection over all parts gives the weighted sum of the experts.
//
// The grouped products (bfloat16, weights in the matrix cores' fragment layout): the (token, expert) pairs of a step are
// put in the order of their experts, every expert's run padded to whole tiles of 64 rows (route_groups_kernel: one
// block counts, places and labels; which row is whose is device data, so a launch depends on sizes only).  A block of
// expert_gate_up_kernel takes one tile of rows, all of one expert, and 128 of that expert's middle columns: each of its
// four waves holds 32 columns of the gate and of the up matrix against the tile's four row fragments, gathered from the
// tokens' rows, and writes act(gate) * up * routing weight, rounded once.  expert_down_kernel is the same walk over
// the expert's slice of the inner dimension of the side-by-side down matrices; expert_combine_kernel adds a token's
// rows.  Only the experts that tokens chose are read, and each row meets only its own expert.
#include "linear_mfma.h"

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

constexpr int GROUP_TILE = 64;      // rows of a tile: four row fragments of 16

// One block.  w: [T, E] routing weights (zero: not chosen).  row_token / row_weight [R]: the pairs in expert order, every
// expert's run padded to whole tiles (token -1, weight 0); tile_expert [R / 64] (-1: no rows); token_rows [T, top]:
// where each token's rows went (-1: fewer than top).
__global__ __launch_bounds__(1024) void route_groups_kernel(const float* __restrict__ w, int T, int E, int top, int R,
                                                            int* __restrict__ row_token, float* __restrict__ row_weight,
                                                            int* __restrict__ tile_expert, int* __restrict__ token_rows) {
  __shared__ int cnt[MAX_EXPERTS], fill[MAX_EXPERTS], off[MAX_EXPERTS + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += blockDim.x) cnt[e] = fill[e] = 0;
  __syncthreads();
  for (long i = tid; i < (long)T * E; i += blockDim.x)
    if (w[i] > 0.f) atomicAdd(&cnt[i % E], 1);
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = at;
      at += (cnt[e] + GROUP_TILE - 1) / GROUP_TILE * GROUP_TILE;
    }
    off[E] = at;
  }
  __syncthreads();
  for (int r = tid; r < R; r += blockDim.x) {
    row_token[r] = -1;
    row_weight[r] = 0.f;
  }
  for (int t = tid; t < R / GROUP_TILE; t += blockDim.x) {
    const int r = t * GROUP_TILE;
    int e = -1;
    if (r < off[E]) {
      int lo = 0, hi = E - 1;                       // the last expert whose run starts at or before r and is not empty there
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (off[mid] <= r) lo = mid; else hi = mid - 1;
      }
      e = lo;
    }
    tile_expert[t] = e;
  }
  __syncthreads();
  for (int t = tid; t < T; t += blockDim.x) {
    int j = 0;
    for (int e = 0; e < E && j < top; ++e) {
      const float x = w[(size_t)t * E + e];
      if (x > 0.f) {
        const int r = off[e] + atomicAdd(&fill[e], 1);
        row_token[r] = t;
        row_weight[r] = x;
        token_rows[(size_t)t * top + j++] = r;
      }
    }
    for (; j < top; ++j) token_rows[(size_t)t * top + j] = -1;
  }
}

// mid[r, f] = act(gate_e x[token r]) * (up_e x[token r]) * weight r, for the tile's expert e; wf: the fragment layout of
// [all gates; all ups] ([2 E F, W]); mid: [R, F] bfloat16.  A wave takes CW tiles of 16 columns against the tile's four
// row fragments: 4 + 2 CW loads for 8 CW products a k-tile.
template <int CW>
__global__ __launch_bounds__(256) void expert_gate_up_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wf,
                                                             const int* __restrict__ row_token, const float* __restrict__ row_weight,
                                                             const int* __restrict__ tile_expert, bf16_t* __restrict__ mid,
                                                             int W, int F, int E, float epi) {
  constexpr int RS = GROUP_TILE / 16;
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
  const int f0 = (blockIdx.y * 4 + wave) * 16 * CW;
  if (f0 >= F) return;
  const int KT = (W + 31) / 32;
  const bf16_t *wg[CW], *wu[CW];
#pragma unroll
  for (int j = 0; j < CW; ++j) {
    const int f = min(f0 + j * 16, F - 16);           // (a tile beyond the expert's columns repeats the last one; it is not stored)
    wg[j] = wf + (size_t)((e * F + f) / 16) * KT * 512 + lane * 8;
    wu[j] = wf + (size_t)(((size_t)E * F + (size_t)e * F + f) / 16) * KT * 512 + lane * 8;
  }
  const bf16_t* xr[RS];
  const int r0 = blockIdx.x * GROUP_TILE;
#pragma unroll
  for (int s = 0; s < RS; ++s) xr[s] = x + (size_t)max(row_token[r0 + s * 16 + c], 0) * W;     // (a padded row reads token 0's; its weight is 0)
  f32x4 ag[CW][RS], au[CW][RS];
#pragma unroll
  for (int j = 0; j < CW; ++j)
#pragma unroll
    for (int s = 0; s < RS; ++s) ag[j][s] = au[j][s] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int kt = 0; kt < KT; ++kt) {
    const int k = min(kt * 32 + g * 8, W - 8);       // a row's last, partial k-tile: the weights are zero there
    u32x4 b[RS], a_g[CW], a_u[CW];
#pragma unroll
    for (int j = 0; j < CW; ++j) {
      a_g[j] = *reinterpret_cast<const u32x4*>(wg[j] + (size_t)kt * 512);
      a_u[j] = *reinterpret_cast<const u32x4*>(wu[j] + (size_t)kt * 512);
    }
#pragma unroll
    for (int s = 0; s < RS; ++s) b[s] = *reinterpret_cast<const u32x4*>(xr[s] + k);
#pragma unroll
    for (int j = 0; j < CW; ++j)
#pragma unroll
      for (int s = 0; s < RS; ++s) {
        ag[j][s] = mfma16(a_g[j], b[s], ag[j][s]);
        au[j][s] = mfma16(a_u[j], b[s], au[j][s]);
      }
  }
#pragma unroll
  for (int s = 0; s < RS; ++s) {
    const int r = r0 + s * 16 + c;
    const float wr = row_weight[r];
#pragma unroll
    for (int j = 0; j < CW; ++j) {
      if (f0 + j * 16 >= F) continue;
      f32x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = wr == 0.f ? 0.f : gated_act(ag[j][s][i], au[j][s][i], epi, false) * wr;
      store4(mid, (size_t)r * F, f0 + j * 16 + g * 4, F, o);
    }
  }
}

// out[r, n] = sum_f mid[r, f] down_e[n, f] for the tile's expert e; wf: the fragment layout of the down matrices side
// by side ([W, E F]); out: [R, W] float32.  A wave takes CW tiles of 16 outputs against the tile's four row fragments.
template <int CW>
__global__ __launch_bounds__(256) void expert_down_kernel(const bf16_t* __restrict__ mid, const bf16_t* __restrict__ wf,
                                                          const int* __restrict__ tile_expert, float* __restrict__ out,
                                                          int W, int F, int E) {
  constexpr int RS = GROUP_TILE / 16;
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
  const int n0 = (blockIdx.y * 4 + wave) * 16 * CW;
  if (n0 >= W) return;
  const int KT = (E * F + 31) / 32, kt0 = e * F / 32, kts = F / 32;      // F is a multiple of 32: an expert's k-tiles are its own
  const int n_tiles = (W + 15) / 16;
  const bf16_t* wd[CW];
#pragma unroll
  for (int j = 0; j < CW; ++j) wd[j] = wf + ((size_t)min(n0 / 16 + j, n_tiles - 1) * KT + kt0) * 512 + lane * 8;
  const int r0 = blockIdx.x * GROUP_TILE;
  const bf16_t* mr[RS];
#pragma unroll
  for (int s = 0; s < RS; ++s) mr[s] = mid + (size_t)(r0 + s * 16 + c) * F + g * 8;
  f32x4 acc[CW][RS];
#pragma unroll
  for (int j = 0; j < CW; ++j)
#pragma unroll
    for (int s = 0; s < RS; ++s) acc[j][s] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int kt = 0; kt < kts; ++kt) {
    u32x4 a[CW], b[RS];
#pragma unroll
    for (int j = 0; j < CW; ++j) a[j] = *reinterpret_cast<const u32x4*>(wd[j] + (size_t)kt * 512);
#pragma unroll
    for (int s = 0; s < RS; ++s) b[s] = *reinterpret_cast<const u32x4*>(mr[s] + kt * 32);
#pragma unroll
    for (int j = 0; j < CW; ++j)
#pragma unroll
      for (int s = 0; s < RS; ++s) acc[j][s] = mfma16(a[j], b[s], acc[j][s]);
  }
#pragma unroll
  for (int j = 0; j < CW; ++j) {
    if (n0 + j * 16 >= W) continue;
#pragma unroll
    for (int s = 0; s < RS; ++s) store4(out, (size_t)(r0 + s * 16 + c) * W, n0 + j * 16 + g * 4, W, acc[j][s]);
  }
}

// y[t, c] = the sum of the token's rows of `rows` [R, W]
__global__ void expert_combine_kernel(const float* __restrict__ rows, const int* __restrict__ token_rows, float* __restrict__ y,
                                      int W, int top) {
  const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  float s = 0.f;
  for (int j = 0; j < top; ++j) {
    const int r = token_rows[(size_t)t * top + j];
    if (r >= 0) s += rows[(size_t)r * W + c];
  }
  y[(size_t)t * W + c] = s;
}

}  // namespace

// Rows that the grouped products of a step of T tokens need: every pair and every expert's padding, in whole tiles.
extern "C" long alice_expert_rows(int T, int E, int top) {
  return ((long)T * top + (long)E * (GROUP_TILE - 1) + GROUP_TILE - 1) / GROUP_TILE * GROUP_TILE;
}

// The routed feed-forward by grouped products, see the top of the file.  x: [T, W] bfloat16; weights: [T, E] float32 of
// alice_route_topk; gate_up, down: fragment layouts of [2 E F, W] and [W, E F]; y: [T, W] float32.  Workspaces for
// R = alice_expert_rows(T, E, top): ints [2 R + R / 64 + T top] (row_token, tile_expert, token_rows; the row weights
// share the ints' buffer as floats), mid [R, F] bfloat16, rows [R, W] float32.
extern "C" int alice_expert_products(const void* x, const float* weights, const void* gate_up, const void* down, float* y, int* ints,
                                     void* mid, float* rows, int T, int W, int F, int E, int top, float epi, hipStream_t stream) {
  ALICE_CHECK(x && weights && gate_up && down && y && ints && mid && rows, "expert_products: a pointer is missing");
  ALICE_CHECK(T >= 1 && E >= 1 && E <= MAX_EXPERTS && top >= 1 && top <= E, "expert_products: 1 <= top <= experts <= %d", MAX_EXPERTS);
  ALICE_CHECK(W >= 8 && W % 8 == 0 && F >= 32 && F % 32 == 0, "expert_products: the width must be a multiple of 8 and the experts' a multiple of 32");
  const long R = alice_expert_rows(T, E, top);
  ALICE_CHECK(R / GROUP_TILE <= 2147483647L / 2 && (long)T * E < (1L << 40), "expert_products: too many rows for one launch");
  int* row_token = ints;
  float* row_weight = reinterpret_cast<float*>(ints + R);
  int* tile_expert = ints + 2 * R;
  int* token_rows = tile_expert + R / GROUP_TILE;
  route_groups_kernel<<<1, 1024, 0, stream>>>(weights, T, E, top, (int)R, row_token, row_weight, tile_expert, token_rows);
  ALICE_LAUNCH_CHECK();
  dim3 g1((unsigned)(R / GROUP_TILE), ceil_div(F, 128));
  expert_gate_up_kernel<2><<<g1, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)gate_up, row_token, row_weight, tile_expert,
                                                (bf16_t*)mid, W, F, E, epi);
  ALICE_LAUNCH_CHECK();
  dim3 g2((unsigned)(R / GROUP_TILE), ceil_div(W, 256));
  expert_down_kernel<4><<<g2, 256, 0, stream>>>((const bf16_t*)mid, (const bf16_t*)down, tile_expert, rows, W, F, E);
  ALICE_LAUNCH_CHECK();
  dim3 g3(T, ceil_div(W, 256));
  expert_combine_kernel<<<g3, 256, 0, stream>>>(rows, token_rows, y, W, top);
  ALICE_LAUNCH_CHECK();
  return 0;
}

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
