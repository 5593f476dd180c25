// Recurrent mixers whose state per head is a matrix S [d, dv] that is carried from token to token, and the short
// causal convolutions that stand before them.  Two recurrences share one kernel:
//
//   state space (plain):  S_t = diag(a_t) S_(t-1) + k_t (b_t v_t)^T,             o_t = S_t^T q_t + skip_h v_t
//   delta rule:           S' = diag(a_t) S_(t-1);  u = b_t (v_t - S'^T k_t);  S_t = S' + k_t u^T,  o_t = S_t^T q_t
//
// a_t is a decay per key channel (or one number a head, spread over the channels), b_t one number a head (the step
// size, or the write strength), q and k may be shared by groups of heads.  o is taken after the token's write.
//
// Everything here is 32-bit on both paths: the operands arrive as float32 rows of the projections and of the
// convolutions, the decays, step sizes and unit vectors are made with the full-precision functions, the state lives
// in float32 rows of the cache, one per slot, and the read-out is left in float32 for the norm that follows.
//
// recurrence_kernel: one wave per (sequence, head, CB value columns), four of them a block, walks through the sequence's tokens of the
// step with its part of the state in registers: lane (rg, col) holds RPT neighbouring rows of one column, reads
// them once and writes them once; a single token is the same walk of one step.  The tokens go through LDS TC at a
// time, the next TC tokens' operands already on their way from memory; sums over the rows of a column meet by lane
// exchanges inside a row of 16 lanes (the 64 / CB row groups of a column are neighbouring lanes), so the delta rule's
// sum a token needs no barrier and no trip through LDS; the read-outs' sums are taken once per TC tokens.  CB is 16 where that fills the chip's SIMDs, else 8 or 4 (more waves, fewer rows a lane).  Which rows belong to the sequence and which state row is
// its own are read on the device (cu_seqlens, slots), so a launch depends on sizes only.
//
// short_conv: y[t, c] = act(bias_c + sum_j w[c, j] x[t - (taps - 1) + j, c]) over the tokens of the token's own
// sequence; before the step's first token come the last taps - 1 inputs of the sequence's earlier steps, kept in
// a state row per slot (zeros at the start); a second kernel moves the step's last inputs into that row.
#include "common.h"
#include "alice_hip.h"

namespace {

__device__ __forceinline__ float silu_full(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float sigmoid_full(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_full(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// ------------------------------------------------------------------------------------------ short convolution

__global__ __launch_bounds__(256) void short_conv_kernel(const float* __restrict__ rows, int row_w, int col0, int C, int taps,
                                                         const float* __restrict__ w, const float* __restrict__ bias,
                                                         const float* __restrict__ state, float* __restrict__ out, int act,
                                                         const int* __restrict__ cu_seqlens, const int* __restrict__ seq_of_token,
                                                         const int* __restrict__ slots) {
  const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int s = seq_of_token[t];
  const int i = t - cu_seqlens[s];                     // the token's place among its sequence's tokens of this step
  const int K = taps - 1;
  const float* st = state ? state + ((size_t)slots[s] * C + c) * K : nullptr;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = K - j;                            // how many tokens before this one
    float x;
    if (back <= i) x = rows[(size_t)(t - back) * row_w + col0 + c];
    else x = st[K + i - back];                         // the input `back - i` places before the step's first token
    acc = fmaf(w[(size_t)c * taps + j], x, acc);
  }
  out[(size_t)t * C + c] = act ? silu_full(acc) : acc;
}

constexpr int MAX_TAPS = 16;

__global__ __launch_bounds__(256) void short_conv_state_kernel(const float* __restrict__ rows, int row_w, int col0, int C, int taps,
                                                               float* __restrict__ state, const int* __restrict__ cu_seqlens,
                                                               const int* __restrict__ slots) {
  const int s = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int t0 = cu_seqlens[s], n = cu_seqlens[s + 1] - t0, K = taps - 1;
  if (n <= 0) return;
  float* st = state + ((size_t)slots[s] * C + c) * K;
  float keep[MAX_TAPS];
#pragma unroll
  for (int m = 0; m < MAX_TAPS; ++m) {
    if (m < K) {
      const int off = n - K + m;                       // the step's token that lands at place m (negative: an older input)
      keep[m] = off >= 0 ? rows[(size_t)(t0 + off) * row_w + col0 + c] : st[n + m];
    }
  }
#pragma unroll
  for (int m = 0; m < MAX_TAPS; ++m)
    if (m < K) st[m] = keep[m];
}

// ------------------------------------------------------------------------------------------ what enters the recurrences

// State space: step[t, h] = softplus(rows[t, dt_col + h] + dt_bias[h]); decay[t, h] = exp(-exp(a_log[h]) step[t, h]).
__global__ void ssm_prepare_kernel(const float* __restrict__ rows, int row_w, int dt_col, const float* __restrict__ dt_bias,
                                   const float* __restrict__ a_log, float* __restrict__ step, float* __restrict__ decay, long n, int H) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int h = (int)(i % H);
  const long t = i / H;
  const float dt = softplus_full(rows[(size_t)t * row_w + dt_col + h] + dt_bias[h]);
  step[i] = dt;
  decay[i] = expf(-expf(a_log[h]) * dt);
}

// Delta rule: blocks y < 2 G make the q (y < G) and k heads of `qk` [T, q | k] unit vectors in place,
// x / sqrt(sum x^2 + unit_eps), q also times q_scale; blocks beyond turn z [T, H d] into the decays
// exp(-exp(a_log[h]) softplus(z + dt_bias)) in place and write beta[t, h] = sigmoid(rows[t, b_col + h]).
__global__ __launch_bounds__(64) void delta_prepare_kernel(float* __restrict__ qk, int qk_w, int k_col, int G, int d, float unit_eps,
                                                           float q_scale, float* __restrict__ z, const float* __restrict__ dt_bias,
                                                           const float* __restrict__ a_log, const float* __restrict__ rows, int row_w,
                                                           int b_col, float* __restrict__ beta, int H) {
  const int t = blockIdx.x, y = blockIdx.y, lane = threadIdx.x;
  if (y < 2 * G) {
    float* x = qk + (size_t)t * qk_w + (y < G ? y * d : k_col + (y - G) * d);
    float ss = 0.f;
    for (int e = lane; e < d; e += 64) ss = fmaf(x[e], x[e], ss);
    ss = wave_sum(ss);
    const float f = (y < G ? q_scale : 1.f) / sqrtf(ss + unit_eps);
    for (int e = lane; e < d; e += 64) x[e] *= f;
  } else {
    const int h = y - 2 * G;
    const float rate = expf(a_log[h]);
    float* zz = z + ((size_t)t * H + h) * d;
    for (int e = lane; e < d; e += 64) zz[e] = expf(-rate * softplus_full(zz[e] + dt_bias[h * d + e]));
    if (lane == 0) beta[(size_t)t * H + h] = sigmoid_full(rows[(size_t)t * row_w + b_col + h]);
  }
}

// ------------------------------------------------------------------------------------------ the recurrence

struct RecurrenceArgs {
  const float* q; int q_w, q_col;          // q[t, q_col + (h / per) * d + r]
  const float* k; int k_w, k_col;          // k likewise (q and k share the grouping)
  const float* v; int v_w, v_col;          // v[t, v_col + h * dv + c]
  const float* decay; int decay_per_row;   // [T, H d] or [T, H]
  const float* b;                          // [T, H]
  const float* skip;                       // [H] or null
  float* out;                              // [T, H dv]
  const int* cu_seqlens; const int* slots;
  float* S;                                // [slots, H, d, dv]
  int H, per, d, dv;
};

// x plus the x of the lane that a DPP control names (lanes a fixed distance apart inside a row of 16)
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  return x + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}
// The sum over the RG neighbouring lanes that hold one column's row groups (RG 4, 8 or 16, aligned): every one of them
// gets it.  Lanes 1 and 2 apart inside a quad, then the other quad of the half row, then the other half of the row.
template <int RG>
__device__ __forceinline__ float sum_row_groups(float x) {
  x = dpp_add<0xB1>(x);                    // quad_perm [1, 0, 3, 2]
  x = dpp_add<0x4E>(x);                    // quad_perm [2, 3, 0, 1]
  if (RG >= 8) x = dpp_add<0x141>(x);      // row_half_mirror
  if (RG >= 16) x = dpp_add<0x140>(x);     // row_mirror
  return x;
}

template <int CB, int RPT, int TC, int WPB, bool DELTA>
__global__ __launch_bounds__(64 * WPB) void recurrence_kernel(RecurrenceArgs a) {
  constexpr int RG = 64 / CB, DP = RG * RPT, NT = 64 * WPB, CBB = CB * WPB;
  constexpr int NL = TC * DP / NT;
  constexpr int NV = (TC * CBB + NT - 1) / NT;
  static_assert(RPT % 4 == 0 && (TC * DP) % NT == 0 && TC <= 64 && (RG == 4 || RG == 8 || RG == 16), "rows are read four at a time");
  __shared__ __align__(16) float sq[TC][DP];
  __shared__ __align__(16) float sk[TC][DP];
  __shared__ __align__(16) float sa[TC][DP];
  __shared__ float sv[TC][CBB];
  __shared__ float sb[TC];
  // the row groups of a column are neighbouring lanes, so that their sums meet without a trip through LDS; the waves of
  // a block take neighbouring columns and share the tokens' q, k and decays
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int col = wave * CB + lane / RG, rg = lane % RG;
  const int j = blockIdx.z * CBB + col;
  const bool col_ok = j < a.dv;
  const int t0 = a.cu_seqlens[s], t1 = a.cu_seqlens[s + 1];
  if (t1 <= t0) return;
  const int H = a.H, d = a.d, dv = a.dv;
  float* Sh = a.S + ((size_t)a.slots[s] * H + h) * d * dv;
  float st[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg * RPT + i;
    st[i] = (r < d && col_ok) ? Sh[(size_t)r * dv + j] : 0.f;
  }
  const int qk_head = h / a.per;
  const float skip = a.skip ? a.skip[h] : 0.f;
  // what this thread fetches for TC tokens: element (t, r) = (idx / DP, idx % DP) of q, k and the decay; (t, c) of v; b of token `tid`
  float pq[NL], pk[NL], pa[NL], pv[NV], pb = 0.f;
  auto fetch = [&](int tc) {
#pragma unroll
    for (int n = 0; n < NL; ++n) {
      const int idx = tid + n * NT, t = tc + idx / DP, r = idx % DP;
      pq[n] = pk[n] = pa[n] = 0.f;
      if (t < t1 && r < d) {
        pq[n] = a.q[(size_t)t * a.q_w + a.q_col + qk_head * d + r];
        pk[n] = a.k[(size_t)t * a.k_w + a.k_col + qk_head * d + r];
        pa[n] = a.decay_per_row ? a.decay[((size_t)t * H + h) * d + r] : a.decay[(size_t)t * H + h];
      }
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int idx = tid + n * NT, t = tc + idx / CBB, c = blockIdx.z * CBB + idx % CBB;
      pv[n] = (idx < TC * CBB && t < t1 && c < dv) ? a.v[(size_t)t * a.v_w + a.v_col + h * dv + c] : 0.f;
    }
    pb = (tid < TC && tc + tid < t1) ? a.b[(size_t)(tc + tid) * H + h] : 0.f;
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += TC) {
    const int n_tok = min(TC, t1 - tc);
    __syncthreads();                                   // the last tokens' operands have been read
#pragma unroll
    for (int n = 0; n < NL; ++n) {
      const int idx = tid + n * NT;
      sq[idx / DP][idx % DP] = pq[n];
      sk[idx / DP][idx % DP] = pk[n];
      sa[idx / DP][idx % DP] = pa[n];                  // (rows beyond d hold zeros and stay zero)
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int idx = tid + n * NT;
      if (idx < TC * CBB) sv[idx / CBB][idx % CBB] = pv[n];
    }
    if (tid < TC) sb[tid] = pb;
    __syncthreads();
    if (tc + TC < t1) fetch(tc + TC);                  // the next tokens' operands are on their way during the walk
    float part[TC], vs[TC];                            // the lanes' shares of the read-outs meet once per TC tokens
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      part[tt] = 0.f;
      vs[tt] = 0.f;
      if (tt < n_tok) {
        const float vj = sv[tt][col], bt = sb[tt];
        vs[tt] = vj;
        float u = bt * vj;
        float4 kk[RPT / 4];
#pragma unroll
        for (int i = 0; i < RPT; i += 4) kk[i / 4] = *reinterpret_cast<const float4*>(&sk[tt][rg * RPT + i]);
        if (DELTA) {
          float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;   // four sums side by side: no chain of dependent additions
#pragma unroll
          for (int i = 0; i < RPT; i += 4) {
            const float4 aa = *reinterpret_cast<const float4*>(&sa[tt][rg * RPT + i]);
            st[i] *= aa.x;      p0 = fmaf(st[i], kk[i / 4].x, p0);
            st[i + 1] *= aa.y;  p1 = fmaf(st[i + 1], kk[i / 4].y, p1);
            st[i + 2] *= aa.z;  p2 = fmaf(st[i + 2], kk[i / 4].z, p2);
            st[i + 3] *= aa.w;  p3 = fmaf(st[i + 3], kk[i / 4].w, p3);
          }
          u = bt * (vj - sum_row_groups<RG>((p0 + p1) + (p2 + p3)));
        }
        float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
        for (int i = 0; i < RPT; i += 4) {
          const float4 qq = *reinterpret_cast<const float4*>(&sq[tt][rg * RPT + i]);
          if (DELTA) {
            st[i] = fmaf(kk[i / 4].x, u, st[i]);
            st[i + 1] = fmaf(kk[i / 4].y, u, st[i + 1]);
            st[i + 2] = fmaf(kk[i / 4].z, u, st[i + 2]);
            st[i + 3] = fmaf(kk[i / 4].w, u, st[i + 3]);
          } else {
            const float4 aa = *reinterpret_cast<const float4*>(&sa[tt][rg * RPT + i]);
            st[i] = fmaf(aa.x, st[i], kk[i / 4].x * u);
            st[i + 1] = fmaf(aa.y, st[i + 1], kk[i / 4].y * u);
            st[i + 2] = fmaf(aa.z, st[i + 2], kk[i / 4].z * u);
            st[i + 3] = fmaf(aa.w, st[i + 3], kk[i / 4].w * u);
          }
          o0 = fmaf(st[i], qq.x, o0);
          o1 = fmaf(st[i + 1], qq.y, o1);
          o2 = fmaf(st[i + 2], qq.z, o2);
          o3 = fmaf(st[i + 3], qq.w, o3);
        }
        part[tt] = (o0 + o1) + (o2 + o3);
      }
    }
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      const float o = sum_row_groups<RG>(part[tt]);
      if (tt < n_tok && rg == 0 && col_ok) a.out[(size_t)(tc + tt) * H * dv + h * dv + j] = fmaf(skip, vs[tt], o);
    }
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg * RPT + i;
    if (r < d && col_ok) Sh[(size_t)r * dv + j] = st[i];
  }
}

// ------------------------------------------------------------------------------------------ norm and gate behind a read-out

// A block per (token, part): the row's part of n elements is RMS-normed (eps inside the root) and multiplied by a
// weight (of the part's length, shared by the parts, or of the row's length).  gate_act 1: silu of the gate row,
// applied before the norm; 2: sigmoid of the gate row, applied after it; 0: no gate.
template <typename TO>
__global__ __launch_bounds__(256) void norm_gate_kernel(const float* __restrict__ x, int width, int parts, const float* __restrict__ gate,
                                                        int gate_w, int gate_col, int gate_act, const float* __restrict__ w,
                                                        int w_shared, float eps, TO* __restrict__ out) {
  __shared__ float red[17];
  const int t = blockIdx.x, g = blockIdx.y, n = width / parts;
  const float* xr = x + (size_t)t * width + (size_t)g * n;
  const float* gr = gate ? gate + (size_t)t * gate_w + gate_col + (size_t)g * n : nullptr;
  float ss = 0.f;
  for (int e = threadIdx.x; e < n; e += blockDim.x) {
    float y = xr[e];
    if (gate_act == 1) y *= silu_full(gr[e]);
    ss = fmaf(y, y, ss);
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)n + eps);
  for (int e = threadIdx.x; e < n; e += blockDim.x) {
    float y = xr[e];
    if (gate_act == 1) y *= silu_full(gr[e]);
    y = y * inv * w[w_shared ? e : g * n + e];
    if (gate_act == 2) y *= sigmoid_full(gr[e]);
    store_f32(out + (size_t)t * width + (size_t)g * n, e, y);
  }
}

}  // namespace

extern "C" int alice_short_conv(const float* rows, int row_w, int col0, int channels, int taps, const float* w, const float* bias,
                                float* state, float* out, int act, const int* cu_seqlens, const int* seq_of_token,
                                const int* slots, int T, int n_seqs, hipStream_t stream) {
  ALICE_CHECK(rows && w && out && cu_seqlens && seq_of_token && slots, "short_conv: a pointer is missing");
  ALICE_CHECK(T >= 0 && n_seqs >= 0 && channels >= 1 && taps >= 1 && taps <= MAX_TAPS, "short_conv: bad sizes (taps 1..%d)", MAX_TAPS);
  ALICE_CHECK(col0 >= 0 && col0 + channels <= row_w, "short_conv: rows of %d elements are too short for the channels", row_w);
  ALICE_CHECK(taps == 1 || state != nullptr, "short_conv: more than one tap needs the state rows");
  ALICE_CHECK(ceil_div(channels, 256) <= 65535, "short_conv: too many channels for one launch");
  if (T == 0 || n_seqs == 0) return 0;
  dim3 grid(T, ceil_div(channels, 256));
  short_conv_kernel<<<grid, 256, 0, stream>>>(rows, row_w, col0, channels, taps, w, bias, taps > 1 ? state : nullptr, out, act,
                                              cu_seqlens, seq_of_token, slots);
  ALICE_LAUNCH_CHECK();
  if (taps > 1) {
    dim3 g2(n_seqs, ceil_div(channels, 256));
    short_conv_state_kernel<<<g2, 256, 0, stream>>>(rows, row_w, col0, channels, taps, state, cu_seqlens, slots);
    ALICE_LAUNCH_CHECK();
  }
  return 0;
}

extern "C" int alice_ssm_prepare(const float* rows, int row_w, int dt_col, const float* dt_bias, const float* a_log, float* step,
                                 float* decay, int T, int H, hipStream_t stream) {
  ALICE_CHECK(rows && dt_bias && a_log && step && decay, "ssm_prepare: a pointer is missing");
  ALICE_CHECK(T >= 0 && H >= 1 && dt_col >= 0 && dt_col + H <= row_w, "ssm_prepare: bad sizes");
  const long n = (long)T * H;
  if (n == 0) return 0;
  ssm_prepare_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(rows, row_w, dt_col, dt_bias, a_log, step, decay, n, H);
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_delta_prepare(float* qk, int qk_w, int k_col, int G, int d, float unit_eps, float q_scale, float* z,
                                   const float* dt_bias, const float* a_log, const float* rows, int row_w, int b_col, float* beta,
                                   int T, int H, hipStream_t stream) {
  ALICE_CHECK(qk && z && dt_bias && a_log && rows && beta, "delta_prepare: a pointer is missing");
  ALICE_CHECK(T >= 0 && H >= 1 && G >= 1 && d >= 1 && unit_eps >= 0.f, "delta_prepare: bad sizes");
  ALICE_CHECK(G * d <= k_col && k_col + G * d <= qk_w && b_col >= 0 && b_col + H <= row_w, "delta_prepare: the rows are too short for the heads");
  ALICE_CHECK(2 * G + H <= 65535, "delta_prepare: too many heads for one launch");
  if (T == 0) return 0;
  dim3 grid(T, 2 * G + H);
  delta_prepare_kernel<<<grid, 64, 0, stream>>>(qk, qk_w, k_col, G, d, unit_eps, q_scale, z, dt_bias, a_log, rows, row_w, b_col, beta, H);
  ALICE_LAUNCH_CHECK();
  return 0;
}

// Value columns a wave: 16 where (sequences x heads x columns) fill the chip's SIMDs, else 8 or 4: more waves, each with
// fewer rows a lane (the rows of a column are then spread over 8 or 16 lanes).
extern "C" int alice_matrix_recurrence_columns(int n_seqs, int H, int d, int dv) {
  const long waves16 = (long)n_seqs * H * ceil_div(dv, 16);
  return (waves16 >= 1024 || d <= 32) ? 16 : ((waves16 >= 512 || d <= 64) ? 8 : 4);
}

extern "C" int alice_matrix_recurrence(const float* q, int q_w, int q_col, const float* k, int k_w, int k_col, const float* v, int v_w,
                                       int v_col, const float* decay, int decay_per_row, const float* b, const float* skip, float* out,
                                       const int* cu_seqlens, const int* slots, float* S, int n_seqs, int n_slots, int H, int qk_heads,
                                       int d, int dv, int delta, int columns, hipStream_t stream) {
  ALICE_CHECK(q && k && v && decay && b && out && cu_seqlens && slots && S, "matrix_recurrence: a pointer is missing");
  ALICE_CHECK(n_seqs >= 0 && n_slots >= 1 && H >= 1 && qk_heads >= 1 && H % qk_heads == 0 && d >= 1 && dv >= 1, "matrix_recurrence: bad sizes");
  ALICE_CHECK(d <= 256, "matrix_recurrence: key size %d is beyond 256, the range of this kernel", d);
  ALICE_CHECK(q_col >= 0 && k_col >= 0 && v_col >= 0 && q_col + qk_heads * d <= q_w && k_col + qk_heads * d <= k_w && v_col + H * dv <= v_w,
              "matrix_recurrence: the rows are too short for the heads");
  ALICE_CHECK(H <= 65535 && ceil_div(dv, 16) <= 65535, "matrix_recurrence: too many heads or value columns for one launch");
  if (n_seqs == 0) return 0;
  RecurrenceArgs a{q, q_w, q_col, k, k_w, k_col, v, v_w, v_col, decay, decay_per_row, b, skip, out, cu_seqlens, slots, S, H, H / qk_heads, d, dv};
  int cb = columns ? columns : alice_matrix_recurrence_columns(n_seqs, H, d, dv);
  ALICE_CHECK(cb == 16 || cb == 8 || cb == 4, "matrix_recurrence: %d value columns a wave are not built (4, 8, 16; 0: by the step's size)", columns);
  if (d <= 32 || (cb == 4 && d <= 64)) cb = d <= 32 ? 16 : 8;      // (fewer than four rows a lane are not built)
  constexpr int WPB = 4;                       // waves a block: they share the staged q, k and decays of a head's tokens
  dim3 grid(n_seqs, H, ceil_div(dv, cb * WPB));
#define GO(CB, RPT, TC)                                                                     \
  do {                                                                                      \
    if (delta) recurrence_kernel<CB, RPT, TC, WPB, true><<<grid, 64 * WPB, 0, stream>>>(a); \
    else recurrence_kernel<CB, RPT, TC, WPB, false><<<grid, 64 * WPB, 0, stream>>>(a);      \
  } while (0)
  if (cb == 16) {
    if (d <= 16) GO(16, 4, 16);
    else if (d <= 32) GO(16, 8, 16);
    else if (d <= 64) GO(16, 16, 16);
    else if (d <= 128) GO(16, 32, 8);
    else GO(16, 64, 8);
  } else if (cb == 8) {
    if (d <= 64) GO(8, 8, 16);
    else if (d <= 128) GO(8, 16, 8);
    else GO(8, 32, 8);
  } else {
    if (d <= 128) GO(4, 8, 8);
    else GO(4, 16, 8);
  }
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_norm_gate(const float* x, int width, int parts, const float* gate, int gate_w, int gate_col, int gate_act,
                               const float* w, int w_shared, float eps, void* out, int out_dtype, int T, hipStream_t stream) {
  ALICE_CHECK(x && w && out && dtype_ok(out_dtype), "norm_gate: a pointer is missing or the dtype is unknown");
  ALICE_CHECK(T >= 0 && width >= 1 && parts >= 1 && width % parts == 0 && parts <= 65535, "norm_gate: %d parts must divide the width %d", parts, width);
  ALICE_CHECK(gate_act >= 0 && gate_act <= 2 && (gate_act == 0 || (gate && gate_col >= 0 && gate_col + width <= gate_w)),
              "norm_gate: the gate rows are missing or too short");
  ALICE_CHECK(eps > 0.f, "norm_gate: eps must be positive");
  if (T == 0) return 0;
  dim3 grid(T, parts);
  const int threads = width / parts > 128 ? 256 : 64;
  if (out_dtype == DT_F32) norm_gate_kernel<float><<<grid, threads, 0, stream>>>(x, width, parts, gate, gate_w, gate_col, gate_act, w, w_shared, eps, (float*)out);
  else norm_gate_kernel<bf16_t><<<grid, threads, 0, stream>>>(x, width, parts, gate, gate_w, gate_col, gate_act, w, w_shared, eps, (bf16_t*)out);
  ALICE_LAUNCH_CHECK();
  return 0;
}
