// Latent attention: every head's keys and values are linear maps of one latent row a token, so only that row
// [c (rank R) | kr (rotated part, r)] is cached, as the one "kv head" of a row-major page, and the maps move to the
// query's side:  score_h(i, j) = scale * ((Uk_h^T q_h,plain(i)) . c(j) + q_h,rot(i) . kr(j)),
// out_h(i) = Uv_h sum_j w_h(i, j) c(j).  Attention is then one shared key of R + r dimensions whose first R
// dimensions are also the value; all heads of a token read the same rows.
//
// Kernels of this file:
//   alice_latent_prepare     from the float32 rows [a | c' | kr'] of the fused down projection: a / rms(a) * wa to the
//                            query latent (activation dtype), c' / rms(c') * wc and kr' rotated in pairs (2i, 2i + 1)
//                            into the token's cache row
//   alice_heads_linear       a matrix a head: y[t, h, 0:n] = M_h x[t, h, 0:k] (M given transposed, [H, k, n]), with
//                            an optional tail y[t, h, n:n+r] = x[t, h, k:k+r] rotated by the token's position
//   alice_latent_attention   softmax attention of [T, H, R + r] queries over the cached rows, causal with an optional
//                            window, 32-bit arithmetic, any sizes; a block a (token, head)
#include "common.h"
#include "alice_hip.h"
#include "kv_layout.h"

namespace {

constexpr int PREP_THREADS = 256;

template <typename TO>
__global__ __launch_bounds__(PREP_THREADS) void latent_prepare_kernel(
    const float* __restrict__ rows, int row_w, int A, int R, int r, const float* __restrict__ wa,
    const float* __restrict__ wc, float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int bt_stride, int page_size, int n_pages, TO* __restrict__ a_out, TO* __restrict__ k_pool) {
  __shared__ float red[17];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* row = rows + (size_t)t * row_w;
  float s = 0.f;
  for (int i = tid; i < A; i += PREP_THREADS) s = fmaf(row[i], row[i], s);
  const float inv_a = 1.f / sqrtf(block_sum(s, red) / (float)A + eps);
  for (int i = tid; i < A; i += PREP_THREADS) store_f32(a_out + (size_t)t * A, i, row[i] * inv_a * wa[i]);
  if (!k_pool) return;
  const int pos = positions[t];
  const int page = block_table[(size_t)seq_of_token[t] * bt_stride + pos / page_size];
  if (page < 0 || page >= n_pages) return;
  TO* dst = k_pool + ((size_t)page * page_size + pos % page_size) * (R + r);
  s = 0.f;
  for (int i = tid; i < R; i += PREP_THREADS) s = fmaf(row[A + i], row[A + i], s);
  const float inv_c = 1.f / sqrtf(block_sum(s, red) / (float)R + eps);
  for (int i = tid; i < R; i += PREP_THREADS) store_f32(dst, i, row[A + i] * inv_c * wc[i]);
  const int half = r >> 1;
  for (int i = tid; i < half; i += PREP_THREADS) {
    float y0, y1;
    rotate_pair(row[A + R + 2 * i], row[A + R + 2 * i + 1], cos_t[(size_t)pos * half + i], sin_t[(size_t)pos * half + i], y0, y1);
    store_f32(dst, R + 2 * i, y0);
    store_f32(dst, R + 2 * i + 1, y1);
  }
}

// ---------------------------------------------------------------------------------------- a matrix a head

constexpr int HL_THREADS = 256;
constexpr int HL_TOKENS = 8;

// A block: HL_TOKENS tokens of one head and 256 outputs.  The tokens' inputs wait in LDS as float32; a thread owns
// one output column and walks down the transposed matrix, whose rows are contiguous over the outputs.
template <typename TX, typename TW, typename TY>
__global__ __launch_bounds__(HL_THREADS) void heads_linear_kernel(
    const TX* __restrict__ x, long x_row, int x_head, const TW* __restrict__ wt, TY* __restrict__ y, long y_row, int y_head,
    int T, int n, int k, int r, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions) {
  extern __shared__ float xs[];                       // [HL_TOKENS][k]
  const int t0 = blockIdx.x * HL_TOKENS, h = blockIdx.y, tid = threadIdx.x;
  const int nt = min(HL_TOKENS, T - t0);
  for (int i = tid; i < HL_TOKENS * k; i += HL_THREADS) {
    const int tt = i / k, e = i % k;
    xs[i] = tt < nt ? load_f32(x + (size_t)(t0 + tt) * x_row + (size_t)h * x_head, e) : 0.f;
  }
  __syncthreads();
  const int c = blockIdx.z * HL_THREADS + tid;
  if (c < n) {
    const TW* w = wt + (size_t)h * k * n + c;
    float acc[HL_TOKENS];
#pragma unroll
    for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = 0.f;
    for (int e = 0; e < k; ++e) {
      const float wv = load_f32(w, (size_t)e * n);
#pragma unroll
      for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = fmaf(xs[tt * k + e], wv, acc[tt]);
    }
#pragma unroll
    for (int tt = 0; tt < HL_TOKENS; ++tt)
      if (tt < nt) store_f32(y + (size_t)(t0 + tt) * y_row + (size_t)h * y_head, c, acc[tt]);
  }
  if (r > 0 && blockIdx.z == 0) {                     // the rotated tail, pairs (2i, 2i + 1)
    const int half = r >> 1;
    for (int i = tid; i < nt * half; i += HL_THREADS) {
      const int tt = i / half, p = i % half, t = t0 + tt;
      const TX* src = x + (size_t)t * x_row + (size_t)h * x_head + k;
      const int pos = positions[t];
      float y0, y1;
      rotate_pair(load_f32(src, 2 * p), load_f32(src, 2 * p + 1), cos_t[(size_t)pos * half + p], sin_t[(size_t)pos * half + p], y0, y1);
      TY* dst = y + (size_t)t * y_row + (size_t)h * y_head + n;
      store_f32(dst, 2 * p, y0);
      store_f32(dst, 2 * p + 1, y1);
    }
  }
}

// ---------------------------------------------------------------------------------------- attention, 32-bit arithmetic

constexpr int LA_THREADS = 256;
constexpr int LA_CHUNK = 1024;
constexpr int LA_COLS = 4;                           // value columns a thread: R <= LA_COLS * LA_THREADS

template <typename T, bool FULL>
__global__ __launch_bounds__(LA_THREADS) void latent_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pool, T* __restrict__ out, const int* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ block_table, int bt_stride, int nH, int R, int r,
    int page_size, float scale, int window, int DG) {
  extern __shared__ float lds[];                      // q [R + r], then the partial outputs [G][R]
  __shared__ float sc[LA_CHUNK];
  __shared__ float red[17];
  const int D = R + r;
  float* qs = lds;
  float* part = lds + D;
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int pos = positions[t];
  const int* bt = block_table + (size_t)seq_of_token[t] * bt_stride;
  const int start = window > 0 ? max(0, pos + 1 - window) : 0;
  const int n_keys = pos + 1 - start;
  const T* qrow = q + ((size_t)t * nH + h) * D;
  for (int i = tid; i < D; i += LA_THREADS) qs[i] = load_f32(qrow, i);
  __syncthreads();
  const int G = LA_THREADS / DG, g = tid / DG, j = tid % DG;
  float acc[LA_COLS];
#pragma unroll
  for (int c = 0; c < LA_COLS; ++c) acc[c] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  for (int c0 = 0; c0 < n_keys; c0 += LA_CHUNK) {
    const int n = min(LA_CHUNK, n_keys - c0);
    float lmax = -INFINITY;
    for (int i = tid; i < n; i += LA_THREADS) {
      const int kp = start + c0 + i;
      const T* krow = k_pool + ((size_t)bt[kp / page_size] * page_size + kp % page_size) * D;
      float s = 0.f;
      for (int e = 0; e < D; ++e) s = fmaf(qs[e], load_f32(krow, e), s);
      s *= scale;
      sc[i] = s;
      lmax = fmaxf(lmax, s);
    }
    const float m_new = fmaxf(m_run, block_max(lmax, red));
    const float corr = (m_run == -INFINITY) ? 0.f : (FULL ? expf(m_run - m_new) : __expf(m_run - m_new));
    float lsum = 0.f;
    for (int i = tid; i < n; i += LA_THREADS) {
      const float p = FULL ? expf(sc[i] - m_new) : __expf(sc[i] - m_new);
      sc[i] = p;
      lsum += p;
    }
    l_run = l_run * corr + block_sum(lsum, red);      // the barriers inside also publish sc[]
    m_run = m_new;
#pragma unroll
    for (int c = 0; c < LA_COLS; ++c) acc[c] *= corr;
    for (int i = g; i < n; i += G) {
      const int kp = start + c0 + i;
      const T* vrow = k_pool + ((size_t)bt[kp / page_size] * page_size + kp % page_size) * D;
      const float p = sc[i];
#pragma unroll
      for (int c = 0; c < LA_COLS; ++c)
        if (j + c * DG < R) acc[c] = fmaf(p, load_f32(vrow, j + c * DG), acc[c]);
    }
    __syncthreads();                                   // sc[] is rewritten by the next chunk
  }
#pragma unroll
  for (int c = 0; c < LA_COLS; ++c)
    if (j + c * DG < R) part[(size_t)g * R + j + c * DG] = acc[c];
  __syncthreads();
  for (int e = tid; e < R; e += LA_THREADS) {
    float o = 0.f;
    for (int gg = 0; gg < G; ++gg) o += part[(size_t)gg * R + e];
    store_f32(out + ((size_t)t * nH + h) * R, e, o / l_run);
  }
}

}  // namespace

extern "C" int alice_latent_prepare(const float* rows, int row_width, int q_rank, int kv_rank, int rot_dim,
                                    const float* w_q, const float* w_kv, float eps, const float* cos_t, const float* sin_t,
                                    const int* positions, const int* seq_of_token, const int* block_table, int bt_stride,
                                    int page_size, int n_pages, void* q_latent, void* k_pool, int out_dtype, int T,
                                    hipStream_t stream) {
  ALICE_CHECK(dtype_ok(out_dtype), "latent_prepare: unknown dtype %d", out_dtype);
  ALICE_CHECK(rows && w_q && w_kv && q_latent && positions, "latent_prepare: missing arguments");
  ALICE_CHECK(T >= 0 && q_rank >= 1 && kv_rank >= 1 && rot_dim >= 0 && rot_dim % 2 == 0,
              "latent_prepare: bad sizes q_rank=%d kv_rank=%d rot_dim=%d", q_rank, kv_rank, rot_dim);
  ALICE_CHECK(row_width >= q_rank + kv_rank + rot_dim, "latent_prepare: rows of %d elements are too short", row_width);
  ALICE_CHECK(rot_dim == 0 || (cos_t && sin_t), "latent_prepare: a rotated part needs both tables");
  ALICE_CHECK(k_pool == nullptr || (block_table && seq_of_token && page_size > 0 && n_pages > 0 && bt_stride > 0),
              "latent_prepare: a cache write needs the block table, the token-to-sequence map and the page geometry");
  ALICE_CHECK(eps > 0.f, "latent_prepare: eps must be positive");
  if (T == 0) return 0;
  DISPATCH_DTYPE(out_dtype, TO, {
    latent_prepare_kernel<TO><<<T, PREP_THREADS, 0, stream>>>(rows, row_width, q_rank, kv_rank, rot_dim, w_q, w_kv, eps, cos_t,
        sin_t, positions, seq_of_token, block_table, bt_stride, page_size, n_pages, (TO*)q_latent, (TO*)k_pool);
  });
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_heads_linear(const void* x, int x_dtype, long x_row, int x_head, const void* wt, int w_dtype, void* y,
                                  int y_dtype, long y_row, int y_head, int T, int H, int n, int k, int rot_dim,
                                  const float* cos_t, const float* sin_t, const int* positions, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(x_dtype) && dtype_ok(w_dtype) && dtype_ok(y_dtype), "heads_linear: unknown dtype");
  ALICE_CHECK(x && wt && y && T >= 0 && H >= 1 && H <= 65535 && n >= 1 && k >= 1, "heads_linear: bad sizes T=%d H=%d n=%d k=%d", T, H, n, k);
  ALICE_CHECK(rot_dim >= 0 && rot_dim % 2 == 0 && (rot_dim == 0 || (cos_t && sin_t && positions)),
              "heads_linear: a rotated tail is even and needs both tables and the positions");
  ALICE_CHECK(x_head >= k + rot_dim && y_head >= n + rot_dim && x_row >= (long)(H - 1) * x_head + k + rot_dim &&
              y_row >= (long)(H - 1) * y_head + n + rot_dim, "heads_linear: the heads do not fit the rows");
  ALICE_CHECK((size_t)HL_TOKENS * k * sizeof(float) <= 64 * 1024, "heads_linear: inner size %d is beyond this kernel", k);
  ALICE_CHECK(ceil_div(n, HL_THREADS) <= 65535, "heads_linear: too many outputs a head (%d)", n);
  if (T == 0) return 0;
  const dim3 grid(ceil_div(T, HL_TOKENS), H, ceil_div(n, HL_THREADS));
  const size_t lds = (size_t)HL_TOKENS * k * sizeof(float);
#define GO(TX, TW, TY)                                                                                                   \
  heads_linear_kernel<TX, TW, TY><<<grid, HL_THREADS, lds, stream>>>((const TX*)x, x_row, x_head, (const TW*)wt, (TY*)y, y_row, \
      y_head, T, n, k, rot_dim, cos_t, sin_t, positions)
  const int code = x_dtype * 4 + w_dtype * 2 + y_dtype;
  switch (code) {
    case 0: GO(float, float, float); break;
    case 1: GO(float, float, bf16_t); break;
    case 2: GO(float, bf16_t, float); break;
    case 3: GO(float, bf16_t, bf16_t); break;
    case 4: GO(bf16_t, float, float); break;
    case 5: GO(bf16_t, float, bf16_t); break;
    case 6: GO(bf16_t, bf16_t, float); break;
    default: GO(bf16_t, bf16_t, bf16_t); break;
  }
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_latent_attention(const void* q, int dtype, const void* k_pool, void* out, const int* positions,
                                      const int* seq_of_token, const int* block_table, int bt_stride, int T, int nH,
                                      int kv_rank, int rot_dim, int page_size, float scale, int window,
                                      int full_precision, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(dtype), "latent_attention: unknown dtype %d", dtype);
  ALICE_CHECK(q && k_pool && out && positions && seq_of_token && block_table, "latent_attention: missing arguments");
  ALICE_CHECK(T >= 0 && nH >= 1 && nH <= 65535 && kv_rank >= 1 && rot_dim >= 0, "latent_attention: bad sizes");
  ALICE_CHECK(kv_rank <= LA_COLS * LA_THREADS, "latent_attention: latent size %d is beyond %d, the range of this kernel", kv_rank,
              LA_COLS * LA_THREADS);
  ALICE_CHECK(page_size > 0 && bt_stride > 0 && window >= 0, "latent_attention: bad page geometry or window");
  if (T == 0) return 0;
  int DG = 1;
  while (DG < kv_rank && DG < LA_THREADS) DG <<= 1;
  const int G = LA_THREADS / DG;
  const size_t lds = ((size_t)(kv_rank + rot_dim) + (size_t)G * kv_rank) * sizeof(float);
  ALICE_CHECK(lds <= 56 * 1024, "latent_attention: sizes beyond this kernel's LDS");
  const dim3 grid(T, nH);
  DISPATCH_DTYPE(dtype, TT, {
    if (full_precision)
      latent_attention_kernel<TT, true><<<grid, LA_THREADS, lds, stream>>>((const TT*)q, (const TT*)k_pool, (TT*)out, positions,
          seq_of_token, block_table, bt_stride, nH, kv_rank, rot_dim, page_size, scale, window, DG);
    else
      latent_attention_kernel<TT, false><<<grid, LA_THREADS, lds, stream>>>((const TT*)q, (const TT*)k_pool, (TT*)out, positions,
          seq_of_token, block_table, bt_stride, nH, kv_rank, rot_dim, page_size, scale, window, DG);
  });
  ALICE_LAUNCH_CHECK();
  return 0;
}
