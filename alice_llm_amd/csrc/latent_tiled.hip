// Latent attention on the matrix cores, prompts and single tokens alike.  In the form with the per-head maps on the
// query's side every head of a token attends over the same cached rows [c (R) | kr (r)], whose first R numbers are
// the value as well: one "kv head" of D = R + r dimensions for all heads.  So the query rows of a sequence are laid
// out flat, row = (token - first token) * heads + head, and a block of four waves takes 64 consecutive rows, a wave
// 16 of them: a staged block of 32 keys serves as many heads of as few tokens as possible (all 16 heads of four
// tokens with 16 heads; a single token's heads are one wave's rows).
//
// A wave computes the transposed score tile S^T = K Q^T with v_mfma_f32_16x16x32_bf16 (keys are the rows, the
// wave's 16 query rows the columns), so that a lane holds eight scores of ONE query row: maximum and sum are
// four-lane affairs, and the rounded weights are, as they stand, the second operand of O^T = V^T P^T.  The keys lie
// in LDS twice, row-major for the first product and transposed (its first DVP dimensions) for the second, in the
// key order in which the score tiles leave the matrix instruction.  Key blocks that no row of the block sees are
// not visited.  With splits > 1 (single tokens: few rows, many keys) block z of a row group takes every splits-th
// run of key blocks and leaves (sum of weighted rows, maximum, sum of weights) for alice_latent_merge.
// bfloat16 operands, 32-bit scores, softmax and sums.  D and R are multiples of 8, D at most 640.
//
// SINGLE: a step of single tokens with at most 16 heads.  A sequence's rows are then one tile of 16, and the four
// waves share it instead of three standing by: each takes every fourth 32-dimension slice of the score product (the
// partial tiles meet in LDS, and every wave does the same softmax on the sum) and every fourth 16-row tile of the
// transposed output.  A wave's key fragments of its slices come straight from memory in fragment order (16 bytes a
// lane: eight consecutive dimensions of one key), every element loaded once by one lane, so the row-major copy of the
// keys in LDS is left out, and the transposed copy of the next step is written from these same registers: a row is
// read from memory once.  A wave holds a quarter of the query and of the output.  Several blocks then fit a CU, and
// one block's walk from page table to rows is covered by the others' arithmetic.
#include "common.h"
#include "alice_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mfma32(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

struct LatentArgs {
  const bf16_t* q;        // [T, nH, D]
  const bf16_t* pool;     // [pages, 1, page, D]
  bf16_t* out;            // [T, nH, R]
  float* part;            // [splits, T nH, R + 2] where splits > 1
  const int* positions;
  const int* cu_seqlens;
  const int* block_table;
  int bt_stride, n_seqs, nH, R, r, page_size, page_shift;
  float scale;
  int window, splits;
  long rows_total;
};

constexpr int KT = 32;        // keys a step
constexpr int VPAD = 40;      // row length of the transposed rows in LDS (32 keys and a pad against bank conflicts)
constexpr int ROWS = 64;      // query rows a block

template <int DP, int DVP, bool SINGLE>
__global__ __launch_bounds__(256) void latent_tiled_kernel(LatentArgs a) {
  constexpr int KS = DP / 32, ET = DVP / 16;
  constexpr int KSW = SINGLE ? (KS + 3) / 4 : KS, ETW = SINGLE ? (ET + 3) / 4 : ET;      // slices and tiles a wave
  constexpr int KROW = DP + 8;
  constexpr int NKC = DP / 64, NVC = DVP / 64;          // 16-byte pieces a thread moves a step, for each of the two copies
  extern __shared__ __align__(16) unsigned char lds_raw[];
  constexpr size_t KS_BYTES = SINGLE ? 0 : (size_t)KT * KROW * sizeof(bf16_t);                       // SINGLE keeps no row-major copy
  bf16_t (*Ks)[KROW] = reinterpret_cast<bf16_t (*)[KROW]>(lds_raw);                                  // [KT][KROW]
  bf16_t (*Vt)[VPAD] = reinterpret_cast<bf16_t (*)[VPAD]>(lds_raw + KS_BYTES);                       // [DVP][VPAD]
  f32x4* Sp = reinterpret_cast<f32x4*>(lds_raw + KS_BYTES + (size_t)DVP * VPAD * sizeof(bf16_t));    // SINGLE: [4][2][64]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, g = lane >> 4;
  const int D = a.R + a.r, R = a.R, nH = a.nH;

  // which 64 rows: the blocks are dealt to the sequences in order, ceil(tokens * heads / 64) each; the last rows of a
  // sequence have the most keys and go first
  int idx = gridDim.x - 1 - blockIdx.x, seq = -1, b = 0, n_rows = 0;
  if (SINGLE) {                                          // a block a sequence, its one token's heads the rows
    idx = 0;
    seq = blockIdx.x;
    b = a.cu_seqlens[seq];
    n_rows = nH;
  } else {
    for (int s = 0; s < a.n_seqs; ++s) {
      const int sb = a.cu_seqlens[s], se = a.cu_seqlens[s + 1], nt = ((se - sb) * nH + ROWS - 1) / ROWS;
      if (idx < nt) {
        seq = s;
        b = sb;
        n_rows = (se - sb) * nH;
        break;
      }
      idx -= nt;
    }
  }
  if (seq < 0) return;
  const int rho0 = idx * ROWS, nq = min(ROWS, n_rows - rho0);
  const int* bt = a.block_table + (size_t)seq * a.bt_stride;
  const int t_first = b + rho0 / nH, t_last = b + (rho0 + nq - 1) / nH;
  const int p_first = a.positions[t_first], p_last = p_first + (t_last - t_first);
  const int rr = SINGLE ? c : wave * 16 + c;             // SINGLE: every wave has the same 16 rows
  const bool valid = rr < nq;
  const bool wave_on = SINGLE || wave * 16 < nq;
  const int rho = rho0 + (valid ? rr : 0);
  const int tq = b + rho / nH;
  const int qpos = p_first + (tq - t_first);
  const size_t grow = (size_t)b * nH + rho;              // the row in q and out
  const int lo_q = a.window > 0 ? qpos + 1 - a.window : 0;
  const int lo = a.window > 0 ? max(0, p_first + 1 - a.window) : 0;
  const int t_lo = lo / KT, t_hi = p_last / KT;
  const int z = blockIdx.y;
  // this block's steps: z, z + splits, ... of the key blocks t_lo .. t_hi
  const int n_all = t_hi - t_lo + 1;
  const int n_steps = n_all > z ? (n_all - z + a.splits - 1) / a.splits : 0;

  u32x4 qf[KSW];                                         // SINGLE: the slices wave, wave + 4, ...
#pragma unroll
  for (int i = 0; i < KSW; ++i) {
    const int ks = SINGLE ? wave + 4 * i : i, dim = ks * 32 + g * 8;
    qf[i] = u32x4{0u, 0u, 0u, 0u};
    if (ks < KS && dim < D) qf[i] = *reinterpret_cast<const u32x4*>(a.q + grow * D + dim);
  }

  auto row_of = [&](int kp) -> size_t {
    const int pi = a.page_shift >= 0 ? kp >> a.page_shift : kp / a.page_size;
    const int sl = a.page_shift >= 0 ? kp & (a.page_size - 1) : kp % a.page_size;
    return (size_t)bt[pi] * a.page_size + sl;
  };
  // A step's 32 keys lie in one page where pages are a power of two of at least 32 positions, so the page is looked
  // up once a block and step, by a load that does not depend on the lane, a step ahead of the rows' loads
  auto page_of = [&](int step) -> int {
    return a.page_shift >= 5 ? bt[((t_lo + z + step * a.splits) * KT) >> a.page_shift] : -1;
  };
  auto row_in = [&](int pg, int kp) -> size_t {
    return pg >= 0 ? (size_t)pg * a.page_size + (kp & (a.page_size - 1)) : row_of(kp);
  };
  u32x4 pk[SINGLE ? 1 : NKC], pv[SINGLE ? 1 : NVC];
  u32x4 kfr[SINGLE ? KSW : 1][2];                        // SINGLE: the key fragments of the wave's slices
  auto fetch_keys = [&](int step, int pg) {              // SINGLE: lane (c, g) takes key c of each tile, dimensions g * 8 ..
    const int key0 = (t_lo + z + step * a.splits) * KT;
#pragma unroll
    for (int i = 0; i < (SINGLE ? KSW : 0); ++i) {
      const int ks = wave + 4 * i, dim = ks * 32 + g * 8;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const int kp = key0 + mt * 16 + c;
        kfr[i][mt] = u32x4{0u, 0u, 0u, 0u};
        if (ks < KS && dim < D && kp <= p_last && kp >= lo) kfr[i][mt] = *reinterpret_cast<const u32x4*>(a.pool + row_in(pg, kp) * D + dim);
      }
    }
  };
  auto fetch = [&](int step, int pg) {
    const int key0 = (t_lo + z + step * a.splits) * KT;
#pragma unroll
    for (int n = 0; n < (SINGLE ? 0 : NKC); ++n) {
      const int id = tid + n * 256, key = id / (DP / 8), dim = (id % (DP / 8)) * 8, kp = key0 + key;
      pk[n] = u32x4{0u, 0u, 0u, 0u};
      if (key < KT && dim < D && kp <= p_last && kp >= lo) pk[n] = *reinterpret_cast<const u32x4*>(a.pool + row_of(kp) * D + dim);
    }
#pragma unroll
    for (int n = 0; n < (SINGLE ? 0 : NVC); ++n) {
      const int id = tid + n * 256, key = id % KT, e = (id / KT) * 8, kp = key0 + key;     // neighbouring lanes: neighbouring keys
      pv[n] = u32x4{0u, 0u, 0u, 0u};
      if (e < D && kp <= p_last && kp >= lo) pv[n] = *reinterpret_cast<const u32x4*>(a.pool + row_in(pg, kp) * D + e);
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int n = 0; n < (SINGLE ? 0 : NKC); ++n) {
      const int id = tid + n * 256, key = id / (DP / 8), dim = (id % (DP / 8)) * 8;
      if (key < KT) *reinterpret_cast<u32x4*>(&Ks[key][dim]) = pk[n];
    }
#pragma unroll
    for (int i = 0; i < (SINGLE ? KSW : 0); ++i) {       // SINGLE: the transposed rows from the key fragments
      const int e = (wave + 4 * i) * 32 + g * 8;
      if (e >= DVP) continue;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const int col = (c >> 2) * 8 + (c & 3) + 4 * mt;
        const uint32_t w[4] = {kfr[i][mt][0], kfr[i][mt][1], kfr[i][mt][2], kfr[i][mt][3]};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          Vt[e + 2 * j][col].bits = (uint16_t)(w[j] & 0xffffu);
          Vt[e + 2 * j + 1][col].bits = (uint16_t)(w[j] >> 16);
        }
      }
    }
#pragma unroll
    for (int n = 0; n < (SINGLE ? 0 : NVC); ++n) {
      const int id = tid + n * 256, key = id % KT, e = (id / KT) * 8;
      const int col = ((key & 15) >> 2) * 8 + (key & 3) + 4 * (key >> 4);       // the order of the score tiles' rows
      const uint32_t w[4] = {pv[n][0], pv[n][1], pv[n][2], pv[n][3]};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        Vt[e + 2 * i][col].bits = (uint16_t)(w[i] & 0xffffu);
        Vt[e + 2 * i + 1][col].bits = (uint16_t)(w[i] >> 16);
      }
    }
  };

  f32x4 oT[ETW];                                         // SINGLE: the tiles wave, wave + 4, ...
  float m_run = -INFINITY, l_run = 0.f;
#pragma unroll
  for (int et = 0; et < ETW; ++et) oT[et] = f32x4{0.f, 0.f, 0.f, 0.f};

  int pg_next = -1;
  if (n_steps > 0) {
    const int pg = page_of(0);
    if (n_steps > 1) pg_next = page_of(1);
    fetch(0, pg);
    if (SINGLE) fetch_keys(0, pg);
    stage();
  }
  __syncthreads();
  for (int step = 0; step < n_steps; ++step) {
    const int key0 = (t_lo + z + step * a.splits) * KT;
    const bool more = step + 1 < n_steps;
    const int pg = pg_next;                              // the next step's page, asked for a step ago
    if (more) fetch(step + 1, pg);
    if (step + 2 < n_steps) pg_next = page_of(step + 2);
    if (wave_on) {
      f32x4 sT[2];
      sT[0] = sT[1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < KSW; ++i) {
        const int ks = SINGLE ? wave + 4 * i : i;
        if (ks >= KS) continue;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const u32x4 kf = SINGLE ? kfr[SINGLE ? i : 0][mt] : *reinterpret_cast<const u32x4*>(&Ks[mt * 16 + c][ks * 32 + g * 8]);
          sT[mt] = mfma32(kf, qf[i], sT[mt]);
        }
      }
      if (SINGLE) {                                      // the four waves' partial tiles, summed in one order by all
        if (more) fetch_keys(step + 1, pg);              // the next step's keys travel during the rest of this one
        Sp[(wave * 2 + 0) * 64 + lane] = sT[0];
        Sp[(wave * 2 + 1) * 64 + lane] = sT[1];
        __syncthreads();
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const f32x4 s0 = Sp[(0 * 2 + mt) * 64 + lane], s1 = Sp[(1 * 2 + mt) * 64 + lane];
          const f32x4 s2 = Sp[(2 * 2 + mt) * 64 + lane], s3 = Sp[(3 * 2 + mt) * 64 + lane];
#pragma unroll
          for (int j = 0; j < 4; ++j) sT[mt][j] = (s0[j] + s1[j]) + (s2[j] + s3[j]);
        }
      }
      bool vis[8];
      bool any = false;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int kp = key0 + (j >> 2) * 16 + g * 4 + (j & 3);
        vis[j] = valid && kp <= qpos && kp >= lo_q;
        any = any || vis[j];
      }
      if (__ballot(any) != 0ull) {                       // else none of the wave's rows sees a key of this block
        float sc[8], m_t = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          sc[j] = vis[j] ? sT[j >> 2][j & 3] * a.scale : -INFINITY;
          m_t = fmaxf(m_t, sc[j]);
        }
        m_t = fmaxf(m_t, __shfl_xor(m_t, 16, 64));
        m_t = fmaxf(m_t, __shfl_xor(m_t, 32, 64));
        const float m_new = fmaxf(m_run, m_t);
        float sum = 0.f, corr = 1.f;
        uint32_t pw[4] = {0u, 0u, 0u, 0u};
        if (m_new > -INFINITY) {
          corr = __expf(m_run - m_new);                  // m_run = -inf gives 0
          float p[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            p[j] = __expf(sc[j] - m_new);
            sum += p[j];
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) pw[j] = pack_bf16x2(p[2 * j], p[2 * j + 1]);
          m_run = m_new;
        }
        l_run = fmaf(l_run, corr, sum);
        const u32x4 pf = u32x4{pw[0], pw[1], pw[2], pw[3]};
#pragma unroll
        for (int n = 0; n < ETW; ++n) {
          const int et = SINGLE ? wave + 4 * n : n;
          if (et >= ET) continue;
          const u32x4 vf = *reinterpret_cast<const u32x4*>(&Vt[et * 16 + c][g * 8]);
#pragma unroll
          for (int i = 0; i < 4; ++i) oT[n][i] *= corr;
          oT[n] = mfma32(vf, pf, oT[n]);
        }
      }
    }
    __syncthreads();                                     // everybody has read the buffer before it is filled again
    if (more) stage();
    __syncthreads();
  }

  if (!valid) return;
  float l_tot = l_run;
  l_tot += __shfl_xor(l_tot, 16, 64);
  l_tot += __shfl_xor(l_tot, 32, 64);
  if (a.splits > 1) {
    float* prow = a.part + ((size_t)z * a.rows_total + grow) * (R + 2);
#pragma unroll
    for (int n = 0; n < ETW; ++n) {
      const int et = SINGLE ? wave + 4 * n : n, e = et * 16 + g * 4;
      if (et >= ET || e >= R) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) prow[e + i] = oT[n][i];
    }
    if (g == 0 && (!SINGLE || wave == 0)) {
      prow[R] = m_run;
      prow[R + 1] = l_tot;
    }
    return;
  }
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
  for (int n = 0; n < ETW; ++n) {
    const int et = SINGLE ? wave + 4 * n : n, e = et * 16 + g * 4;
    if (et >= ET || e >= R) continue;
    uint2 pkd = {pack_bf16x2(oT[n][0] * inv, oT[n][1] * inv), pack_bf16x2(oT[n][2] * inv, oT[n][3] * inv)};
    *reinterpret_cast<uint2*>(a.out + grow * R + e) = pkd;
  }
}

// One row a block: out = sum_z exp(m_z - M) o_z / sum_z exp(m_z - M) l_z, M the largest of the m_z.  The splits'
// maxima and sums are read once into LDS, a split's weight is computed once, and the row's elements are added up with
// several loads in flight.
__global__ __launch_bounds__(128) void latent_merge_kernel(const float* __restrict__ part, bf16_t* __restrict__ out,
                                                           int splits, long rows_total, int R) {
  const size_t row = blockIdx.x;
  const int t = threadIdx.x;
  __shared__ float mz[32], lz[32], wz[32];
  if (t < 32) {
    float m = -INFINITY, l = 0.f;
    if (t < splits) {
      const float* p = part + ((size_t)t * rows_total + row) * (R + 2);
      m = p[R];
      l = p[R + 1];
    }
    mz[t] = m;
    lz[t] = l;
  }
  __syncthreads();
  if (t < 32) {
    float M = -INFINITY, l = 0.f;
    for (int z = 0; z < splits; ++z) M = fmaxf(M, mz[z]);
    for (int z = 0; z < splits; ++z)
      if (mz[z] > -INFINITY) l = fmaf(__expf(mz[z] - M), lz[z], l);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    wz[t] = mz[t] > -INFINITY ? __expf(mz[t] - M) * inv : 0.f;       // 0 for a split that saw no key
  }
  __syncthreads();
  const size_t stride = (size_t)rows_total * (R + 2);
  for (int e = t; e < R; e += blockDim.x) {
    const float* p = part + row * (size_t)(R + 2) + e;
    float o = 0.f;
    int z = 0;
    for (; z + 4 <= splits; z += 4) {                    // four loads in flight
      const float a0 = p[(size_t)z * stride], a1 = p[(size_t)(z + 1) * stride], a2 = p[(size_t)(z + 2) * stride],
                  a3 = p[(size_t)(z + 3) * stride];
      o = fmaf(wz[z], a0, o);
      o = fmaf(wz[z + 1], a1, o);
      o = fmaf(wz[z + 2], a2, o);
      o = fmaf(wz[z + 3], a3, o);
    }
    for (; z < splits; ++z) o = fmaf(wz[z], p[(size_t)z * stride], o);
    out[row * R + e] = f32_to_bf16(o);
  }
}

// ------------------------------------------------------------------------------------- a matrix a head, matrix cores
// y[t, h, 0:n] = W_h x[t, h, 0:k], W given as stored, [H, n, k] (k contiguous), as the transposed product
// Y^T = W X^T: the matrix's rows are the first operand's rows, the tokens the columns, so a lane ends with four
// consecutive outputs of one token.  Both operands come straight from memory in fragment order (16 bytes a lane: eight
// consecutive k of one row), no LDS and no barrier.  A wave takes MT tiles of 16 tokens and four tiles of 16 outputs;
// a block's four waves take different tokens (WIDE = false) or different outputs of the same 16 MT tokens (single
// tokens, a tile of 16 outputs a wave: the matrices are all there is to read, so the more blocks read them the better).  The r numbers behind a head's k inputs are turned in pairs (2i, 2i + 1) by the token's position and put
// behind its n outputs.
constexpr int HN = 4;         // output tiles a wave where the waves take different tokens

__device__ __forceinline__ void turn_pair(float u, float v, float cs, float sn, float& a, float& b) {
  a = fmaf(u, cs, -__fmul_rn(v, sn));
  b = fmaf(v, cs, __fmul_rn(u, sn));
}

template <int MT, bool WIDE, int HT>
__global__ __launch_bounds__(256) void heads_linear_mfma_kernel(
    const bf16_t* __restrict__ x, long x_row, int x_head, const bf16_t* __restrict__ w, bf16_t* __restrict__ y, long y_row,
    int y_head, int T, int n, int k, int r, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, g = lane >> 4;
  const int h = blockIdx.y;
  const int block_tokens = 16 * MT * (WIDE ? 1 : 4);
  const int t0 = blockIdx.x * block_tokens + (WIDE ? 0 : wave * 16 * MT);
  const int n0 = (blockIdx.z * (WIDE ? 4 : 1) + (WIDE ? wave : 0)) * (16 * HT);

  if (r > 0 && blockIdx.z == 0) {                     // the rotated tail of the block's tokens
    const int half = r >> 1, tb = blockIdx.x * block_tokens, nt = min(block_tokens, T - tb);
    for (int i = tid; i < nt * half; i += 256) {
      const int t = tb + i / half, p = i % half;
      const bf16_t* src = x + (size_t)t * x_row + (size_t)h * x_head + k;
      const int pos = positions[t];
      float y0, y1;
      turn_pair(bf16_to_f32(src[2 * p]), bf16_to_f32(src[2 * p + 1]), cos_t[(size_t)pos * half + p], sin_t[(size_t)pos * half + p], y0, y1);
      *reinterpret_cast<uint32_t*>(y + (size_t)t * y_row + (size_t)h * y_head + n + 2 * p) = pack_bf16x2(y0, y1);
    }
  }
  if (t0 >= T || n0 >= n) return;

  f32x4 acc[HT][MT];
#pragma unroll
  for (int i = 0; i < HT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16_t* wrow[HT];
  bool w_on[HT];
#pragma unroll
  for (int i = 0; i < HT; ++i) {
    const int row = n0 + i * 16 + c;
    w_on[i] = row < n;
    wrow[i] = w + ((size_t)h * n + (w_on[i] ? row : 0)) * k;
  }
  const bf16_t* xrow[MT];
  bool x_on[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int t = t0 + j * 16 + c;
    x_on[j] = t < T;
    xrow[j] = x + (size_t)(x_on[j] ? t : 0) * x_row + (size_t)h * x_head;
  }
  for (int k0 = 0; k0 < k; k0 += 32) {
    const int dim = k0 + g * 8;
    const bool in = dim < k;
    u32x4 wf[HT], xf[MT];
#pragma unroll
    for (int i = 0; i < HT; ++i) {
      wf[i] = u32x4{0u, 0u, 0u, 0u};
      if (in && w_on[i]) wf[i] = *reinterpret_cast<const u32x4*>(wrow[i] + dim);
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      xf[j] = u32x4{0u, 0u, 0u, 0u};
      if (in && x_on[j]) xf[j] = *reinterpret_cast<const u32x4*>(xrow[j] + dim);
    }
#pragma unroll
    for (int i = 0; i < HT; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j) acc[i][j] = mfma32(wf[i], xf[j], acc[i][j]);
  }
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    if (!x_on[j]) continue;
    bf16_t* dst = y + (size_t)(t0 + j * 16 + c) * y_row + (size_t)h * y_head;
#pragma unroll
    for (int i = 0; i < HT; ++i) {
      const int e = n0 + i * 16 + g * 4;
      if (e >= n) continue;
      uint2 pkd = {pack_bf16x2(acc[i][j][0], acc[i][j][1]), pack_bf16x2(acc[i][j][2], acc[i][j][3])};
      *reinterpret_cast<uint2*>(dst + e) = pkd;
    }
  }
}

int padded(int n) {
  const int sizes[] = {64, 128, 192, 256, 384, 512, 576, 640};
  for (int s : sizes)
    if (n <= s) return s;
  return 0;
}

template <int DP, int DVP, bool SINGLE>
int launch_as(const LatentArgs& a, dim3 grid, hipStream_t stream) {
  constexpr size_t lds = SINGLE ? (size_t)DVP * VPAD * sizeof(bf16_t) + 4 * 2 * 64 * sizeof(f32x4)
                                : ((size_t)KT * (DP + 8) + (size_t)DVP * VPAD) * sizeof(bf16_t);
  static bool raised = false;                            // once a process and instance: more LDS than the static limit
  if (lds > 48 * 1024 && !raised) {
    ALICE_CHECK(hipFuncSetAttribute((const void*)latent_tiled_kernel<DP, DVP, SINGLE>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds) == hipSuccess, "latent attention: %zu bytes of LDS were refused", lds);
    raised = true;
  }
  latent_tiled_kernel<DP, DVP, SINGLE><<<grid, 256, lds, stream>>>(a);
  return 0;
}

// Single tokens of at most 16 heads (every sequence of the step brings one token): a block a sequence and split.
template <int DP, int DVP>
int launch(const LatentArgs& a, dim3 grid, bool single, hipStream_t stream) {
  if (single) return launch_as<DP, DVP, true>(a, dim3(a.n_seqs, grid.y), stream);
  return launch_as<DP, DVP, false>(a, grid, stream);
}

}  // namespace

extern "C" int alice_latent_tiled_supported(int kv_rank, int rot_dim) {
  const int d = kv_rank + rot_dim;
  return kv_rank >= 8 && kv_rank % 8 == 0 && rot_dim % 8 == 0 && padded(d) != 0;
}

// The largest number of splits that alice_latent_tiled takes; `part` holds splits * T * nH * (kv_rank + 2) floats.
extern "C" int alice_latent_tiled_max_splits() { return 32; }

// q: bfloat16 [T, nH (kv_rank + rot_dim)]; pool: bfloat16 [pages, 1, page, kv_rank + rot_dim]; out: bfloat16
// [T, nH kv_rank].  The step's tokens are those of n_seqs sequences in order (cu_seqlens), each at consecutive
// positions.  splits > 1 needs `part`.  single_tokens: the caller's word that every sequence brings one token.
extern "C" int alice_latent_tiled(const void* q, const void* pool, void* out, float* part, const int* positions,
                                  const int* cu_seqlens, const int* block_table, int bt_stride, int T, int n_seqs, int nH,
                                  int kv_rank, int rot_dim, int page_size, float scale, int window, int splits,
                                  int single_tokens, hipStream_t stream) {
  ALICE_CHECK(alice_latent_tiled_supported(kv_rank, rot_dim), "latent attention: sizes %d and %d are outside the matrix-core kernel's range (multiples of 8, together at most 640)", kv_rank, rot_dim);
  ALICE_CHECK(q && pool && out && positions && cu_seqlens && block_table, "latent attention: a pointer is missing");
  ALICE_CHECK(T >= 0 && n_seqs >= 1 && nH >= 1, "latent attention: bad sizes T=%d n_seqs=%d nH=%d", T, n_seqs, nH);
  ALICE_CHECK(page_size > 0 && bt_stride > 0 && window >= 0, "latent attention: bad page geometry or window");
  ALICE_CHECK(splits >= 1 && splits <= alice_latent_tiled_max_splits() && (splits == 1 || part), "latent attention: %d splits, or no room for them", splits);
  ALICE_CHECK(((uintptr_t)q & 15) == 0 && ((uintptr_t)pool & 15) == 0 && ((uintptr_t)out & 7) == 0, "latent attention: operands are not aligned");
  if (T == 0) return 0;
  int page_shift = -1;
  for (int b = 0; b < 31; ++b)
    if (page_size == (1 << b)) page_shift = b;
  const long rows_total = (long)T * nH;
  LatentArgs a{(const bf16_t*)q, (const bf16_t*)pool, (bf16_t*)out, part, positions, cu_seqlens, block_table, bt_stride, n_seqs,
               nH, kv_rank, rot_dim, page_size, page_shift, scale, window, splits, rows_total};
  const int dp = padded(kv_rank + rot_dim);
  // the second product runs over the row's first DVP dimensions: one size class below the row's where the latent fits
  dim3 grid(ceil_div(rows_total, ROWS) + n_seqs, splits);
  ALICE_CHECK(!single_tokens || T == n_seqs, "latent attention: a step of single tokens has %d tokens for %d sequences", T, n_seqs);
  const bool single = single_tokens && nH <= 16;
  int rc = 0;
#define GO(DP, DVLOW)                                                \
  case DP:                                                           \
    rc = (DVLOW < DP && kv_rank <= DVLOW) ? launch<DP, DVLOW>(a, grid, single, stream) : launch<DP, DP>(a, grid, single, stream); \
    break
  switch (dp) {
    GO(64, 64);
    GO(128, 64);
    GO(192, 128);
    GO(256, 192);
    GO(384, 256);
    GO(512, 384);
    GO(576, 512);
    GO(640, 576);
    default:
      ALICE_CHECK(false, "latent attention: no kernel for rows of %d", kv_rank + rot_dim);
  }
#undef GO
  if (rc) return rc;
  ALICE_LAUNCH_CHECK();
  if (splits > 1) {
    latent_merge_kernel<<<(unsigned)rows_total, 128, 0, stream>>>(part, (bf16_t*)out, splits, rows_total, kv_rank);
    ALICE_LAUNCH_CHECK();
  }
  return 0;
}

extern "C" int alice_heads_linear_mfma_supported(int n, int k, int rot_dim) {
  return n >= 4 && n % 4 == 0 && k >= 8 && k % 8 == 0 && rot_dim >= 0 && rot_dim % 8 == 0;
}

// x: bfloat16 rows of x_row elements, head h at h * x_head: [k inputs | rot_dim to be turned]; w: bfloat16 [H, n, k];
// y: bfloat16 rows of y_row elements, head h at h * y_head: [n outputs | rot_dim turned].
extern "C" int alice_heads_linear_mfma(const void* x, long x_row, int x_head, const void* w, void* y, long y_row, int y_head,
                                       int T, int H, int n, int k, int rot_dim, const float* cos_t, const float* sin_t,
                                       const int* positions, hipStream_t stream) {
  ALICE_CHECK(alice_heads_linear_mfma_supported(n, k, rot_dim), "heads_linear: sizes n=%d k=%d rot_dim=%d are outside the matrix-core kernel's range", n, k, rot_dim);
  ALICE_CHECK(x && w && y && T >= 0 && H >= 1 && H <= 65535, "heads_linear: bad sizes T=%d H=%d", T, H);
  ALICE_CHECK(rot_dim == 0 || (cos_t && sin_t && positions), "heads_linear: a rotated tail needs both tables and the positions");
  ALICE_CHECK(x_head >= k + rot_dim && y_head >= n + rot_dim && x_row >= (long)(H - 1) * x_head + k + rot_dim &&
              y_row >= (long)(H - 1) * y_head + n + rot_dim, "heads_linear: the heads do not fit the rows");
  ALICE_CHECK(x_head % 8 == 0 && x_row % 8 == 0 && y_head % 4 == 0 && y_row % 4 == 0 && ((uintptr_t)x & 15) == 0 &&
              ((uintptr_t)w & 15) == 0 && ((uintptr_t)y & 7) == 0, "heads_linear: rows or heads are not aligned");
  if (T == 0) return 0;
  if (T <= 64) {                                        // few tokens: the waves share them and split the outputs
    if (T <= 16) {
      const dim3 grid(1, H, ceil_div(n, 4 * 16));
      heads_linear_mfma_kernel<1, true, 1><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)y, y_row, y_head, T, n, k, rot_dim, cos_t, sin_t, positions);
    } else {
      const dim3 grid(ceil_div(T, 32), H, ceil_div(n, 4 * 16));
      heads_linear_mfma_kernel<2, true, 1><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)y, y_row, y_head, T, n, k, rot_dim, cos_t, sin_t, positions);
    }
  } else {
    const dim3 grid(ceil_div(T, 256), H, ceil_div(n, 16 * HN));
    heads_linear_mfma_kernel<4, false, HN><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)y, y_row, y_head, T, n, k, rot_dim, cos_t, sin_t, positions);
  }
  ALICE_LAUNCH_CHECK();
  return 0;
}
