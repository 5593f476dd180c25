// From the rows of a fused q | k | v (| ...) projection to the attention kernels' operands, for mixers whose
// projections have biases, whose rotation pairs neighbouring dimensions, covers a part of the head, or also
// turns the values: bias add, rotation, q out, k and v into their places of the paged cache (row-major pages).
//
// The rows come in float32 (the projection's sums, nothing rounded on the way) or in the activation dtype; the
// outputs are in the activation dtype TO.  Pairing: interleaved (2i, 2i + 1) or halves (i, i + R/2) over the
// rotated width R <= d of q and k heads; the pair (u, v) at position p becomes (u cos a - v sin a,
// v cos a + u sin a), a = p * f_i, from tables [positions, R/2].  With value tables [positions, dv/2] every value
// head is turned the same way over all its dv dimensions by its own position (the attention kernel turns the
// head's output back by the query's position).
//
// With norm weights the q columns (all heads together) and the k columns (likewise) are each divided by their root
// mean square over the whole projection, eps inside the root, and multiplied by a weight of that length, after the
// bias and before the rotation; projection_rms_kernel finds the two factors of every token first, in 32-bit.
#include "common.h"
#include "alice_hip.h"
#include "kv_layout.h"

namespace {

// inv[t, part] = 1 / sqrt(mean over the part's columns of (row + bias)^2 + eps); part 0: the q columns [0, n_q),
// part 1: the k columns [n_q, n_q + n_k).
template <typename TI>
__global__ __launch_bounds__(256) void projection_rms_kernel(const TI* __restrict__ rows, int row_w, const float* __restrict__ bias,
                                                             float* __restrict__ inv, int n_q, int n_k, float eps) {
  __shared__ float red[17];
  const int t = blockIdx.x, part = blockIdx.y;
  const int c0 = part ? n_q : 0, n = part ? n_k : n_q;
  const TI* row = rows + (size_t)t * row_w;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    float x = load_f32(row, (size_t)c0 + c);
    if (bias) x += bias[c0 + c];
    ss = fmaf(x, x, ss);
  }
  ss = block_sum(ss, red);
  if (threadIdx.x == 0) inv[(size_t)t * 2 + part] = 1.f / sqrtf(ss / (float)n + eps);
}

template <typename TI, typename TO>
__global__ void qkv_prepare_kernel(const TI* __restrict__ rows, int row_w, const float* __restrict__ bias,
                                   const float* __restrict__ norm_w, const float* __restrict__ inv_rms,
                                   TO* __restrict__ q_out, TO* __restrict__ k_pool, TO* __restrict__ v_pool,
                                   const float* __restrict__ cos_t, const float* __restrict__ sin_t, int R, int interleaved,
                                   const float* __restrict__ vcos, const float* __restrict__ vsin,
                                   const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                   const int* __restrict__ block_table, int bt_stride, int nH, int nKV, int d, int dv,
                                   int page_size, int n_pages) {
  const int t = blockIdx.x, h = blockIdx.y;
  const int pos = positions[t];
  const TI* row = rows + (size_t)t * row_w;
  const int tp = pos % page_size;
  int page = -1;
  if (k_pool) {
    page = block_table[(size_t)seq_of_token[t] * bt_stride + pos / page_size];
    if (page < 0 || page >= n_pages) page = -1;
  }
  if (h < nH + nKV) {
    const bool is_q = h < nH;
    if (!is_q && page < 0) return;
    const size_t col0 = (size_t)h * d;                         // k heads follow the q heads
    TO* dst = is_q ? q_out + ((size_t)t * nH + h) * d
                   : k_pool + (((size_t)page * nKV + (h - nH)) * page_size + tp) * d;
    const int half = R >> 1;
    const float inv = norm_w ? inv_rms[(size_t)t * 2 + (is_q ? 0 : 1)] : 1.f;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      const int e0 = interleaved ? 2 * i : i, e1 = interleaved ? 2 * i + 1 : i + half;
      float x0 = load_f32(row, col0 + e0), x1 = load_f32(row, col0 + e1);
      if (bias) { x0 += bias[col0 + e0]; x1 += bias[col0 + e1]; }
      if (norm_w) { x0 = x0 * inv * norm_w[col0 + e0]; x1 = x1 * inv * norm_w[col0 + e1]; }
      float y0, y1;
      rotate_pair(x0, x1, cos_t[(size_t)pos * half + i], sin_t[(size_t)pos * half + i], y0, y1);
      store_f32(dst, e0, y0);
      store_f32(dst, e1, y1);
    }
    for (int e = R + threadIdx.x; e < d; e += blockDim.x) {
      float x = load_f32(row, col0 + e);
      if (bias) x += bias[col0 + e];
      if (norm_w) x = x * inv * norm_w[col0 + e];
      store_f32(dst, e, x);
    }
  } else if (page >= 0) {
    const int hv = h - nH - nKV;
    const size_t col0 = (size_t)(nH + nKV) * d + (size_t)hv * dv;
    TO* dst = v_pool + (((size_t)page * nKV + hv) * page_size + tp) * dv;
    if (vcos) {
      const int half = dv >> 1;
      for (int i = threadIdx.x; i < half; i += blockDim.x) {
        const int e0 = interleaved ? 2 * i : i, e1 = interleaved ? 2 * i + 1 : i + half;
        float x0 = load_f32(row, col0 + e0), x1 = load_f32(row, col0 + e1);
        if (bias) { x0 += bias[col0 + e0]; x1 += bias[col0 + e1]; }
        float y0, y1;
        rotate_pair(x0, x1, vcos[(size_t)pos * half + i], vsin[(size_t)pos * half + i], y0, y1);
        store_f32(dst, e0, y0);
        store_f32(dst, e1, y1);
      }
    } else {
      for (int e = threadIdx.x; e < dv; e += blockDim.x) {
        float x = load_f32(row, col0 + e);
        if (bias) x += bias[col0 + e];
        store_f32(dst, e, x);
      }
    }
  }
}

// x[t, c] += (a ? a[t, c] : 0) + (v ? v[c] : 0)
__global__ void add_rows_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ v, long n, int W) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float s = x[i];
  if (a) s += a[i];
  if (v) s += v[i % W];
  x[i] = s;
}

}  // namespace

extern "C" int alice_qkv_prepare(const void* rows, int rows_dtype, int row_width, const float* bias, void* q_out, void* k_pool,
                                 void* v_pool, int out_dtype, const float* cos_t, const float* sin_t, int rotary_dim,
                                 int interleaved, const float* vcos, const float* vsin, const int* positions,
                                 const int* seq_of_token, const int* block_table, int bt_stride, int T, int nH, int nKV,
                                 int d, int dv, int page_size, int n_pages, const float* norm_w, float norm_eps, float* inv_rms,
                                 hipStream_t stream) {
  ALICE_CHECK(dtype_ok(rows_dtype) && dtype_ok(out_dtype), "qkv_prepare: unknown dtype");
  ALICE_CHECK(norm_w == nullptr || (inv_rms != nullptr && norm_eps > 0.f), "qkv_prepare: the projection norm needs its workspace and a positive eps");
  ALICE_CHECK(rows_dtype == DT_F32 || rows_dtype == out_dtype, "qkv_prepare: rows are float32 or in the outputs' dtype");
  ALICE_CHECK(T >= 0 && nH >= 1 && nKV >= 0 && d >= 1 && dv >= 1, "qkv_prepare: bad sizes T=%d nH=%d nKV=%d d=%d dv=%d", T, nH, nKV, d, dv);
  ALICE_CHECK(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0, "qkv_prepare: rotated width %d must be even and at most %d", rotary_dim, d);
  ALICE_CHECK((cos_t == nullptr) == (sin_t == nullptr) && (rotary_dim == 0 || cos_t != nullptr), "qkv_prepare: a rotated width needs both tables");
  ALICE_CHECK((vcos == nullptr) == (vsin == nullptr) && (vcos == nullptr || dv % 2 == 0), "qkv_prepare: turning the values needs both tables and an even size");
  ALICE_CHECK((k_pool == nullptr) == (v_pool == nullptr), "qkv_prepare: key and value pools must come together");
  ALICE_CHECK(k_pool == nullptr || (block_table && seq_of_token && page_size > 0 && n_pages > 0 && nKV >= 1 && bt_stride > 0),
              "qkv_prepare: a cache write needs the block table, the token-to-sequence map and the page geometry");
  ALICE_CHECK(row_width >= (nH + (k_pool ? nKV : 0)) * d + (k_pool ? nKV * dv : 0), "qkv_prepare: rows of %d elements are too short for the heads", row_width);
  ALICE_CHECK(nH + 2 * nKV <= 65535, "qkv_prepare: too many heads for one launch");
  if (T == 0) return 0;
  dim3 grid(T, nH + (k_pool ? 2 * nKV : 0));
  const int threads = 64;
  if (norm_w) {
    dim3 g0(T, k_pool ? 2 : 1);
    if (rows_dtype == DT_F32) projection_rms_kernel<float><<<g0, 256, 0, stream>>>((const float*)rows, row_width, bias, inv_rms, nH * d, k_pool ? nKV * d : 0, norm_eps);
    else projection_rms_kernel<bf16_t><<<g0, 256, 0, stream>>>((const bf16_t*)rows, row_width, bias, inv_rms, nH * d, k_pool ? nKV * d : 0, norm_eps);
    ALICE_LAUNCH_CHECK();
  }
#define GO(TI, TO)                                                                                                          \
  qkv_prepare_kernel<TI, TO><<<grid, threads, 0, stream>>>((const TI*)rows, row_width, bias, norm_w, inv_rms, (TO*)q_out, (TO*)k_pool, (TO*)v_pool, \
      cos_t, sin_t, rotary_dim, interleaved, vcos, vsin, positions, seq_of_token, block_table, bt_stride, nH, nKV, d, dv, page_size, n_pages)
  if (rows_dtype == DT_F32 && out_dtype == DT_F32) GO(float, float);
  else if (rows_dtype == DT_F32) GO(float, bf16_t);
  else GO(bf16_t, bf16_t);
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_add_rows(float* x, const float* a, const float* v, int T, int W, hipStream_t stream) {
  ALICE_CHECK(x && T >= 0 && W >= 1, "add_rows: bad arguments");
  const long n = (long)T * W;
  if (n == 0 || (!a && !v)) return 0;
  add_rows_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(x, a, v, n, W);
  ALICE_LAUNCH_CHECK();
  return 0;
}
