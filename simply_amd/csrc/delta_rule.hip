// A recurrent mixer with a matrix state per head (the gated delta rule) over a ragged batch of requests:
//
//   short causal convolution per channel, then silu          short_conv_silu_kernel (+ conv_tail_update_kernel)
//   q, k to unit length, q / sqrt(size); beta and decay      delta_prepare_kernel
//   S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q   delta_rule_kernel
//
// A request's tokens of this step are rows first .. first + count - 1 of the step (seq_meta [S, 4]: state slot,
// first row, count, position of the first); what earlier steps left is the slot's state: the matrix S per head and
// the last taps - 1 inputs of the convolution.  Everything is 32-bit; sums run in a fixed order that depends on
// nothing but the sizes, so a token's result is the same however the tokens are cut into steps and whatever else
// is in the batch.
#include "api.h"
#include "common.h"

namespace sa {

constexpr int kMaxTaps = 8;
constexpr int kConvTokens = 16;  // tokens that one thread of the convolution walks through

// y[t, c] = silu(sum_j taps[c, j] * x[t - (n - 1 - j), c]) with x before the step's first token taken from the
// request's tail [n - 1][C] (oldest first).  A thread takes one channel and kConvTokens consecutive tokens.
__global__ __launch_bounds__(kWave) void short_conv_silu_kernel(
    const void* __restrict__ x, int x_dtype, int64_t x_stride, const void* __restrict__ taps, int taps_dtype, int n,
    const float* __restrict__ tails, int64_t tail_stride, const int* __restrict__ seq_meta, float* __restrict__ y,
    int C) {
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int j0 = blockIdx.x * kConvTokens;
  const int c = blockIdx.z * kWave + threadIdx.x;
  if (j0 >= count || c >= C) return;
  float w[kMaxTaps], win[kMaxTaps];   // win[i]: input at token j - (n - 1 - i)
#pragma unroll
  for (int i = 0; i < kMaxTaps; ++i) w[i] = i < n ? load_f(taps, taps_dtype, static_cast<size_t>(c) * n + i) : 0.f;
  const float* tail = tails + static_cast<size_t>(slot) * tail_stride;
  auto input = [&](int j) -> float {   // j: token of the request in this step; negative: before the step
    if (j >= 0) return load_f(x, x_dtype, static_cast<size_t>(first + j) * x_stride + c);
    return tail[static_cast<size_t>(n - 1 + j) * C + c];
  };
#pragma unroll
  for (int i = 0; i < kMaxTaps; ++i) win[i] = (i >= 1 && i < n) ? input(j0 - (n - i)) : 0.f;   // win[1..n-1]: the n - 1 before j0
  const int jn = count - j0 < kConvTokens ? count - j0 : kConvTokens;
  for (int j = 0; j < jn; ++j) {
#pragma unroll
    for (int i = 0; i + 1 < kMaxTaps; ++i) win[i] = win[i + 1];
    // (the newest sits at win[n - 1]: entries from n on are never read)
    const float cur = input(j0 + j);
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i)
      if (i == n - 1) win[i] = cur;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i)
      if (i < n) acc = fmaf(w[i], win[i], acc);
    y[static_cast<size_t>(first + j0 + j) * C + c] = acc / (1.f + expf(-acc));
  }
}

// The tails after the step: the last n - 1 inputs of every request, from this step's rows and, where the step brought
// fewer than n - 1 tokens, from the old tail.  A thread takes one channel of one request; it reads old entries only
// at places that it has not written yet.
__global__ __launch_bounds__(kWave) void conv_tail_update_kernel(const void* __restrict__ x, int x_dtype,
                                                                 int64_t x_stride, int n, float* __restrict__ tails,
                                                                 int64_t tail_stride, const int* __restrict__ seq_meta,
                                                                 int C) {
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int c = blockIdx.x * kWave + threadIdx.x;
  if (c >= C || count <= 0) return;
  float* tail = tails + static_cast<size_t>(slot) * tail_stride;
  for (int i = 0; i < n - 1; ++i) {
    const int j = count - (n - 1) + i;   // token of this step that becomes entry i; negative: an old entry
    tail[static_cast<size_t>(i) * C + c] = j >= 0 ? load_f(x, x_dtype, static_cast<size_t>(first + j) * x_stride + c)
                                                  : tail[static_cast<size_t>(n - 1 + j) * C + c];
  }
}

// Per (token, unit): units 0 .. 2 G - 1 are the q and k heads of qkv [T, C] (q heads first), each made a unit vector
// x / sqrt(sum(x^2) + 1e-6), the queries also times size^(-1/2); unit 2 G computes, for every value head h,
// beta = sigmoid(b), g = exp(-exp(A_log) * softplus(a + dt_bias)) and ln g into gates [T, 3 H] (in this order).
__global__ __launch_bounds__(kWave) void delta_prepare_kernel(float* __restrict__ qkv, int C, int G, int dk,
                                                              const void* __restrict__ ab, int ab_dtype,
                                                              int64_t ab_stride, const void* __restrict__ a_log,
                                                              const void* __restrict__ dt_bias, int vec_dtype, int H,
                                                              float* __restrict__ gates) {
  const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  if (unit < 2 * G) {
    float* head = qkv + static_cast<size_t>(t) * C + static_cast<size_t>(unit) * dk;
    float ss = 0.f;
    for (int i = lane; i < dk; i += kWave) ss = fmaf(head[i], head[i], ss);
    ss = wave_sum(ss);
    float r = 1.f / sqrtf(ss + 1e-6f);
    if (unit < G) r *= 1.f / sqrtf(static_cast<float>(dk));
    for (int i = lane; i < dk; i += kWave) head[i] *= r;
    return;
  }
  for (int h = lane; h < H; h += kWave) {
    const float a = load_f(ab, ab_dtype, static_cast<size_t>(t) * ab_stride + h);
    const float b = load_f(ab, ab_dtype, static_cast<size_t>(t) * ab_stride + H + h);
    const float z = a + load_f(dt_bias, vec_dtype, h);
    const float sp = z > 30.f ? z : log1pf(expf(z));
    const float lg = -expf(load_f(a_log, vec_dtype, h)) * sp;
    gates[static_cast<size_t>(t) * 3 * H + h] = 1.f / (1.f + expf(-b));
    gates[static_cast<size_t>(t) * 3 * H + H + h] = expf(lg);
    gates[static_cast<size_t>(t) * 3 * H + 2 * H + h] = lg;
  }
}

// The recurrence.  A workgroup of 256 threads takes 256 / LPC columns of one head's state for one request: LPC lanes
// (4 or 16, neighbours in a row of 16 lanes) share a column, lane `part` of them holding rows part, part + LPC, ...
// of it in registers (DK / LPC of them).  The step's q, k and v of kRuleTokens tokens at a time go through LDS.
// Columns are independent of each other; a column's sums run within a lane over its rows in increasing order, in
// four partial sums that are added in a fixed order, then across the lanes by data-parallel primitives in a fixed
// order: nothing depends on how the tokens are cut into steps or on the batch.  The chain of dependent operations
// per token, and the instructions that one wave issues for it, are what bound a prompt's time (tokens follow one
// another, and a head's columns are all the waves there are): 16 or 32 lanes per column keep both short where a
// column has 64 rows or more.
template <int LPC>
__device__ __forceinline__ float lanes_sum(float v) {
  v += lane_exchange<0xB1>(v);   // quad_perm [1, 0, 3, 2]
  v += lane_exchange<0x4E>(v);   // quad_perm [2, 3, 0, 1]
  if (LPC >= 16) {
    v += lane_exchange<0x141>(v);  // row_half_mirror
    v += lane_exchange<0x140>(v);  // row_mirror
  }
  if (LPC >= 32) {   // two rows of 16 lanes: gfx950's row swap brings the neighbouring row's sum
    const unsigned u = __float_as_uint(v);
    const auto rows = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    v = __uint_as_float(rows[0]) + __uint_as_float(rows[1]);
  }
  if (LPC == 64) {   // and the other half of the wave
    const unsigned u = __float_as_uint(v);
    const auto halves = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    v = __uint_as_float(halves[0]) + __uint_as_float(halves[1]);
  }
  return v;
}

template <int DK, int LPC, int kRuleTokens>
__global__ __launch_bounds__(256) void delta_rule_kernel(const float* __restrict__ qkv, int C, int G, int dk, int dv,
                                                         const float* __restrict__ gates, int H,
                                                         float* __restrict__ state, int64_t state_stride,
                                                         const int* __restrict__ seq_meta, float* __restrict__ out,
                                                         int max_count) {
  constexpr int R = DK / LPC, COLS = 256 / LPC;
  static_assert(R % 4 == 0 || R < 4, "rows per lane come in fours");
  constexpr int NACC = R < 4 ? 1 : 4;
  __shared__ float qs[kRuleTokens][DK], ks[kRuleTokens][DK], vs[kRuleTokens][COLS], bg[kRuleTokens][2];
  const int* meta = seq_meta + 4 * blockIdx.x;
  const int slot = meta[0], first = meta[1], count = meta[2];
  if (count >= max_count) return;   // (the chunked kernels take the requests with many tokens)
  const int h = blockIdx.y, tid = threadIdx.x;
  const int col = blockIdx.z * COLS + tid / LPC, part = tid % LPC;
  const bool live = col < dv;
  const int qk_head = h / (H / G);
  // a head's state is kept column by column, [dv][dk]: the lanes that share a column read neighbouring words
  float* S = state + static_cast<size_t>(slot) * state_stride + static_cast<size_t>(h) * dk * dv;
  float s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = r * LPC + part;
    s[r] = (live && i < dk) ? S[static_cast<size_t>(col) * dk + i] : 0.f;
  }
  const int v_at = 2 * G * dk + h * dv;
  // A tile's q, k, v and gates are asked for a tile ahead, into registers, and put into LDS when the tile's turn
  // comes: the loads are under way while the tile before is worked through.
  constexpr int PQ = kRuleTokens * DK / 256, PV = (kRuleTokens * COLS + 255) / 256;
  float pq[PQ], pk[PQ], pv[PV], pg = 0.f;
  auto fetch = [&](int t0) __attribute__((always_inline)) {
    const int tn = count - t0 < kRuleTokens ? count - t0 : kRuleTokens;
#pragma unroll
    for (int i = 0; i < PQ; ++i) {
      const int idx = tid + i * 256, j = idx / DK, d = idx % DK;
      const bool ok = j < tn && d < dk;
      const float* row = qkv + static_cast<size_t>(first + t0 + (ok ? j : 0)) * C;
      pq[i] = ok ? row[qk_head * dk + d] : 0.f;
      pk[i] = ok ? row[(G + qk_head) * dk + d] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < PV; ++i) {
      const int idx = tid + i * 256, j = idx / COLS, c = blockIdx.z * COLS + idx % COLS;
      const bool ok = idx < kRuleTokens * COLS && j < tn && c < dv;
      pv[i] = ok ? qkv[static_cast<size_t>(first + t0 + j) * C + v_at + c] : 0.f;
    }
    pg = tid < 2 * tn ? gates[static_cast<size_t>(first + t0 + tid / 2) * 3 * H + (tid % 2) * H + h] : 0.f;
  };
  if (count > 0) fetch(0);
  for (int t0 = 0; t0 < count; t0 += kRuleTokens) {
    const int tn = count - t0 < kRuleTokens ? count - t0 : kRuleTokens;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PQ; ++i) {
      const int idx = tid + i * 256;
      qs[idx / DK][idx % DK] = pq[i];
      ks[idx / DK][idx % DK] = pk[i];
    }
#pragma unroll
    for (int i = 0; i < PV; ++i) {
      const int idx = tid + i * 256;
      if (idx < kRuleTokens * COLS) vs[idx / COLS][idx % COLS] = pv[i];
    }
    if (tid < 2 * kRuleTokens) bg[tid / 2][tid % 2] = pg;
    __syncthreads();
    if (t0 + kRuleTokens < count) fetch(t0 + kRuleTokens);
    // the token's operands are read from LDS a token ahead, into one of two sets of registers in turn
    struct Operands {
      float k[R], q[R], v, beta, g;
    };
    auto read = [&](Operands& x, int j) __attribute__((always_inline)) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        x.k[r] = ks[j][r * LPC + part];
        x.q[r] = qs[j][r * LPC + part];
      }
      x.v = vs[j][tid / LPC];
      x.beta = bg[j][0];
      x.g = bg[j][1];
    };
    auto token = [&](const Operands& x, int j) __attribute__((always_inline)) {
      float d[NACC];
#pragma unroll
      for (int a = 0; a < NACC; ++a) d[a] = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        s[r] *= x.g;
        d[r % NACC] = fmaf(s[r], x.k[r], d[r % NACC]);
      }
      float dot = d[0];
      if (NACC == 4) dot = (d[0] + d[NACC > 1 ? 1 : 0]) + (d[NACC > 2 ? 2 : 0] + d[NACC > 3 ? 3 : 0]);
      dot = lanes_sum<LPC>(dot);
      const float u = x.beta * (x.v - dot);
#pragma unroll
      for (int a = 0; a < NACC; ++a) d[a] = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        s[r] = fmaf(x.k[r], u, s[r]);
        d[r % NACC] = fmaf(s[r], x.q[r], d[r % NACC]);
      }
      float o = d[0];
      if (NACC == 4) o = (d[0] + d[NACC > 1 ? 1 : 0]) + (d[NACC > 2 ? 2 : 0] + d[NACC > 3 ? 3 : 0]);
      o = lanes_sum<LPC>(o);
      if (live && part == 0)
        out[static_cast<size_t>(first + t0 + j) * (static_cast<size_t>(H) * dv) + static_cast<size_t>(h) * dv + col] = o;
    };
    Operands A, B;
    read(A, 0);
    for (int j = 0; j < tn; j += 2) {
      if (j + 1 < tn) read(B, j + 1);
      token(A, j);
      if (j + 1 < tn) {
        if (j + 2 < tn) read(A, j + 2);
        token(B, j + 1);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = r * LPC + part;
    if (live && i < dk) S[static_cast<size_t>(col) * dk + i] = s[r];
  }
}


// ------------------------------------------------------------------ the same rule, a chunk of 32 tokens at a time
// For requests that bring many tokens.  Within a chunk, with L_t = ln g_1 + ... + ln g_t counted from the chunk's
// start, S0 the state before the chunk and e(t, i) = exp(L_t - L_i):
//
//   u_t = beta_t (v_t - exp(L_t) S0^T k_t - sum_{i<t} e(t, i) (k_t . k_i) u_i)
//   o_t = exp(L_t) S0^T q_t + sum_{i<=t} e(t, i) (q_t . k_i) u_i
//   S   = exp(L_C) S0 + sum_t e(C, t) k_t u_t^T
//
// so with A[t][i] = beta_t e(t, i) (k_t . k_i) below the diagonal, U = (I + A)^-1 B for B_t = beta_t (v_t -
// exp(L_t) S0^T k_t).  The first kernel computes, for every chunk and head at once, T = (I + A)^-1 and
// P[t][i] = e(t, i) (q_t . k_i) (neither depends on the state); the second walks a request's chunks in order with a
// block of the state's columns in LDS and does, per chunk, the products with S0, U = T B, the outputs and the new
// state: sums of 32 or of the key size per element, no sum across lanes, all 32-bit.  The order of the sums differs
// from the token-by-token kernel's (rounding only).  A chunk's factors lie in `scratch` as [T 32x32][P 32x32]
// [exp(L_t) 32][e(C, t) 32][beta 32] per (request, chunk, head); tokens beyond a request's last count as beta = 0,
// g = 1, k = q = 0.
constexpr int kChunk = 32;
constexpr int kChunkWords = 2 * kChunk * kChunk + 3 * kChunk;

template <int DK>
__global__ __launch_bounds__(256) void delta_chunk_factors_kernel(const float* __restrict__ qkv, int C, int G, int dk,
                                                                  const float* __restrict__ gates, int H,
                                                                  const int* __restrict__ seq_meta, int min_count,
                                                                  float* __restrict__ scratch, int max_chunks) {
  constexpr int LD = DK + 1;
  __shared__ float ks[kChunk][LD], qs[kChunk][LD];
  __shared__ float Am[kChunk][kChunk + 1], Tm[kChunk][kChunk + 1], Lc[kChunk], bt[kChunk];
  const int n = blockIdx.x, s = blockIdx.y, h = blockIdx.z, tid = threadIdx.x;
  const int* meta = seq_meta + 4 * s;
  const int first = meta[1], count = meta[2];
  const int t0 = n * kChunk;
  if (count < min_count || t0 >= count) return;
  const int tn = count - t0 < kChunk ? count - t0 : kChunk;
  const int qk_head = h / (H / G);
  for (int idx = tid; idx < kChunk * DK; idx += 256) {
    const int j = idx / DK, d = idx % DK;
    const bool ok = j < tn && d < dk;
    const float* row = qkv + static_cast<size_t>(first + t0 + (ok ? j : 0)) * C;
    ks[j][d] = ok ? row[(G + qk_head) * dk + d] : 0.f;
    qs[j][d] = ok ? row[qk_head * dk + d] : 0.f;
  }
  if (tid < kChunk) {
    const size_t g_at = static_cast<size_t>(first + t0 + tid) * 3 * H + h;
    bt[tid] = tid < tn ? gates[g_at] : 0.f;
    Lc[tid] = tid < tn ? gates[g_at + 2 * H] : 0.f;
  }
  __syncthreads();
  if (tid == 0)
    for (int t = 1; t < kChunk; ++t) Lc[t] += Lc[t - 1];
  __syncthreads();
  float* out = scratch + ((static_cast<size_t>(s) * max_chunks + n) * H + h) * kChunkWords;
  for (int idx = tid; idx < kChunk * kChunk; idx += 256) {
    const int t = idx / kChunk, i = idx % kChunk;
    float a = 0.f, p = 0.f;
    if (i <= t) {
      float dk_[4] = {0.f, 0.f, 0.f, 0.f}, dq_[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
      for (int d = 0; d < DK; ++d) {
        dk_[d % 4] = fmaf(ks[t][d], ks[i][d], dk_[d % 4]);
        dq_[d % 4] = fmaf(qs[t][d], ks[i][d], dq_[d % 4]);
      }
      const float e = expf(Lc[t] - Lc[i]);
      p = e * ((dq_[0] + dq_[1]) + (dq_[2] + dq_[3]));
      if (i < t) a = bt[t] * e * ((dk_[0] + dk_[1]) + (dk_[2] + dk_[3]));
    }
    Am[t][i] = a;
    out[kChunk * kChunk + idx] = p;
  }
  __syncthreads();
  if (tid < kChunk) {   // column tid of (I + A)^-1, from the diagonal down
    const int j = tid;
    for (int t = 0; t < kChunk; ++t) {
      float v = t == j ? 1.f : 0.f;
      for (int i = j; i < t; ++i) v = fmaf(-Am[t][i], Tm[i][j], v);
      Tm[t][j] = v;
    }
    out[2 * kChunk * kChunk + tid] = expf(Lc[tid]);
    out[2 * kChunk * kChunk + kChunk + tid] = expf(Lc[kChunk - 1] - Lc[tid]);
    out[2 * kChunk * kChunk + 2 * kChunk + tid] = bt[tid];
  }
  __syncthreads();
  for (int idx = tid; idx < kChunk * kChunk; idx += 256) out[idx] = Tm[idx / kChunk][idx % kChunk];
}

template <int DK>
__global__ __launch_bounds__(256) void delta_chunk_scan_kernel(const float* __restrict__ qkv, int C, int G, int dk, int dv,
                                                               int H, float* __restrict__ state, int64_t state_stride,
                                                               const int* __restrict__ seq_meta, int min_count,
                                                               const float* __restrict__ scratch, int max_chunks,
                                                               float* __restrict__ out) {
  constexpr int NC = 8, LD = DK + 4;   // columns of the state per workgroup; rows of 16-byte pieces
  __shared__ __attribute__((aligned(16))) float ks[kChunk][LD];
  __shared__ __attribute__((aligned(16))) float qs[kChunk][LD];
  __shared__ __attribute__((aligned(16))) float Ss[NC][LD];   // the columns, each with its rows side by side
  __shared__ float Tm[kChunk][kChunk + 1], Pm[kChunk][kChunk + 1];
  __shared__ float vs[kChunk][NC], Bm[kChunk][NC], Um[kChunk][NC], gam[kChunk], wl[kChunk], bt[kChunk];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int* meta = seq_meta + 4 * s;
  const int slot = meta[0], first = meta[1], count = meta[2];
  if (count < min_count) return;
  const int col0 = blockIdx.z * NC;
  const int qk_head = h / (H / G);
  const int v_at = 2 * G * dk + h * dv;
  float* S = state + static_cast<size_t>(slot) * state_stride + static_cast<size_t>(h) * dk * dv;   // [dv][dk]
  for (int idx = tid; idx < NC * DK; idx += 256) {
    const int c = idx / DK, d = idx % DK;
    Ss[c][d] = (col0 + c < dv && d < dk) ? S[static_cast<size_t>(col0 + c) * dk + d] : 0.f;
  }
  const int t = tid / NC, c = tid % NC;        // the element of [32 tokens][NC columns] that this thread computes
  const int chunks = (count + kChunk - 1) / kChunk;
  for (int n = 0; n < chunks; ++n) {
    const int t0 = n * kChunk;
    const int tn = count - t0 < kChunk ? count - t0 : kChunk;
    const float* f = scratch + ((static_cast<size_t>(s) * max_chunks + n) * H + h) * kChunkWords;
    __syncthreads();   // the chunk before has been read to its end
    for (int idx = tid; idx < kChunk * DK; idx += 256) {
      const int j = idx / DK, d = idx % DK;
      const bool ok = j < tn && d < dk;
      const float* row = qkv + static_cast<size_t>(first + t0 + (ok ? j : 0)) * C;
      ks[j][d] = ok ? row[(G + qk_head) * dk + d] : 0.f;
      qs[j][d] = ok ? row[qk_head * dk + d] : 0.f;
    }
    for (int idx = tid; idx < kChunk * kChunk; idx += 256) {
      Tm[idx / kChunk][idx % kChunk] = f[idx];
      Pm[idx / kChunk][idx % kChunk] = f[kChunk * kChunk + idx];
    }
    vs[t][c] = (t < tn && col0 + c < dv) ? qkv[static_cast<size_t>(first + t0 + t) * C + v_at + col0 + c] : 0.f;
    if (tid < kChunk) {
      gam[tid] = f[2 * kChunk * kChunk + tid];
      wl[tid] = f[2 * kChunk * kChunk + kChunk + tid];
      bt[tid] = f[2 * kChunk * kChunk + 2 * kChunk + tid];
    }
    __syncthreads();
    // S0^T k_t and S0^T q_t for this thread's (t, c)
    float4 ka = {0.f, 0.f, 0.f, 0.f}, qa = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int d = 0; d < DK; d += 4) {
      const float4 k4 = *reinterpret_cast<const float4*>(&ks[t][d]);
      const float4 q4 = *reinterpret_cast<const float4*>(&qs[t][d]);
      const float4 s4 = *reinterpret_cast<const float4*>(&Ss[c][d]);
      ka.x = fmaf(k4.x, s4.x, ka.x); ka.y = fmaf(k4.y, s4.y, ka.y); ka.z = fmaf(k4.z, s4.z, ka.z); ka.w = fmaf(k4.w, s4.w, ka.w);
      qa.x = fmaf(q4.x, s4.x, qa.x); qa.y = fmaf(q4.y, s4.y, qa.y); qa.z = fmaf(q4.z, s4.z, qa.z); qa.w = fmaf(q4.w, s4.w, qa.w);
    }
    const float KS = (ka.x + ka.y) + (ka.z + ka.w), QS = (qa.x + qa.y) + (qa.z + qa.w);
    Bm[t][c] = bt[t] * (vs[t][c] - gam[t] * KS);
    __syncthreads();
    float u = 0.f;
#pragma unroll 8
    for (int i = 0; i < kChunk; ++i) u = fmaf(Tm[t][i], Bm[i][c], u);   // (T is 0 above its diagonal)
    Um[t][c] = u;
    __syncthreads();
    float o = gam[t] * QS;
#pragma unroll 8
    for (int i = 0; i < kChunk; ++i) o = fmaf(Pm[t][i], Um[i][c], o);   // (P is 0 above its diagonal)
    if (t < tn && col0 + c < dv)
      out[static_cast<size_t>(first + t0 + t) * (static_cast<size_t>(H) * dv) + static_cast<size_t>(h) * dv + col0 + c] = o;
    // the state after the chunk: four neighbouring rows of one column per thread and turn
    const float g_all = gam[kChunk - 1];
    for (int piece = tid / NC; piece * 4 < DK; piece += 256 / NC) {
      const int d = piece * 4;
      float4 a = *reinterpret_cast<const float4*>(&Ss[c][d]);
      a.x *= g_all; a.y *= g_all; a.z *= g_all; a.w *= g_all;
#pragma unroll 8
      for (int j = 0; j < kChunk; ++j) {
        const float w = wl[j] * Um[j][c];
        const float4 k4 = *reinterpret_cast<const float4*>(&ks[j][d]);
        a.x = fmaf(k4.x, w, a.x); a.y = fmaf(k4.y, w, a.y); a.z = fmaf(k4.z, w, a.z); a.w = fmaf(k4.w, w, a.w);
      }
      // (every read of Ss by the products above lies before the last two barriers; this thread alone reads and
      // writes these four words now)
      *reinterpret_cast<float4*>(&Ss[c][d]) = a;
    }
  }
  __syncthreads();
  for (int idx = tid; idx < NC * DK; idx += 256) {
    const int cc = idx / DK, d = idx % DK;
    if (col0 + cc < dv && d < dk) S[static_cast<size_t>(col0 + cc) * dk + d] = Ss[cc][d];
  }
}

}  // namespace sa

using namespace sa;

extern "C" int sa_short_conv_silu(const void* x, int x_dtype, int64_t x_stride, const void* taps, int taps_dtype,
                                  int num_taps, float* tails, int64_t tail_stride, const int* seq_meta, int num_seqs,
                                  int max_q_len, float* y, int C, int update_tails, hipStream_t stream) {
  if (num_seqs == 0 || max_q_len == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && max_q_len > 0 && C > 0 && x != nullptr && taps != nullptr &&
                 (tails != nullptr || num_taps == 1) && seq_meta != nullptr && y != nullptr,
             "short_conv_silu: bad sizes S=%d q=%d C=%d", num_seqs, max_q_len, C);
  SA_REQUIRE(num_taps >= 1 && num_taps <= kMaxTaps, "short_conv_silu: 1 to %d taps, got %d", kMaxTaps, num_taps);
  SA_REQUIRE(x_stride >= C && tail_stride >= static_cast<int64_t>(num_taps - 1) * C,
             "short_conv_silu: a stride is below what the %d channels need", C);
  SA_REQUIRE(num_seqs <= 65535 && (C + kWave - 1) / kWave <= 65535, "short_conv_silu: too many requests or channels");
  const dim3 grid((max_q_len + kConvTokens - 1) / kConvTokens, num_seqs, (C + kWave - 1) / kWave);
  short_conv_silu_kernel<<<grid, kWave, 0, stream>>>(x, x_dtype, x_stride, taps, taps_dtype, num_taps, tails,
                                                     tail_stride, seq_meta, y, C);
  if (update_tails && num_taps > 1)
    conv_tail_update_kernel<<<dim3((C + kWave - 1) / kWave, num_seqs), kWave, 0, stream>>>(
        x, x_dtype, x_stride, num_taps, tails, tail_stride, seq_meta, C);
  return check_launch("short_conv_silu");
}

extern "C" int sa_delta_prepare(float* qkv, int T, int C, int G, int dk, const void* ab, int ab_dtype, int64_t ab_stride,
                                const void* a_log, const void* dt_bias, int vec_dtype, int H, float* gates,
                                hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && G > 0 && dk > 0 && H > 0 && C >= 2 * G * dk && H % G == 0 && ab_stride >= 2 * H,
             "delta_prepare: bad sizes T=%d C=%d G=%d dk=%d H=%d", T, C, G, dk, H);
  SA_REQUIRE(qkv != nullptr && ab != nullptr && a_log != nullptr && dt_bias != nullptr && gates != nullptr,
             "delta_prepare: a null pointer");
  SA_REQUIRE(2 * G + 1 <= 65535, "delta_prepare: too many heads");
  delta_prepare_kernel<<<dim3(T, 2 * G + 1), kWave, 0, stream>>>(qkv, C, G, dk, ab, ab_dtype, ab_stride, a_log, dt_bias,
                                                                 vec_dtype, H, gates);
  return check_launch("delta_prepare");
}

// How many tokens a request must bring for the chunked kernels to take it (0: they do not take this key size), and
// the floats of scratch memory that they need for num_seqs requests of at most max_q_len tokens.
extern "C" int sa_delta_rule_chunk_threshold(int dk) { return (dk <= 128 && dk % 4 == 0) ? 2 * kChunk : 0; }
extern "C" int64_t sa_delta_rule_scratch_words(int num_seqs, int max_q_len, int H) {
  return static_cast<int64_t>(num_seqs) * ((max_q_len + kChunk - 1) / kChunk) * H * kChunkWords;
}

extern "C" int sa_delta_rule(const float* qkv, int C, int G, int dk, int dv, const float* gates, int H, float* state,
                             int64_t state_stride, const int* seq_meta, int num_seqs, int min_q_len, int max_q_len,
                             float* scratch, int64_t scratch_words, float* out, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && G > 0 && H > 0 && H % G == 0 && dk > 0 && dv > 0 && C >= 2 * G * dk + H * dv,
             "delta_rule: bad sizes S=%d C=%d G=%d H=%d dk=%d dv=%d", num_seqs, C, G, H, dk, dv);
  SA_REQUIRE(dk <= 256, "delta_rule: key size %d is above 256", dk);
  SA_REQUIRE(state_stride >= static_cast<int64_t>(H) * dk * dv, "delta_rule: the state rows are too short");
  SA_REQUIRE(qkv != nullptr && gates != nullptr && state != nullptr && seq_meta != nullptr && out != nullptr,
             "delta_rule: a null pointer");
  SA_REQUIRE(H <= 65535 && dv <= 65535 * 8 && num_seqs <= 65535, "delta_rule: too many heads, columns or requests");
  SA_REQUIRE(max_q_len >= 1 && min_q_len >= 0 && min_q_len <= max_q_len, "delta_rule: bad token counts");
  // requests with many tokens go chunk by chunk (if there is scratch memory for their chunks' factors), the others
  // token by token
  int threshold = sa_delta_rule_chunk_threshold(dk);
  if (threshold == 0 || max_q_len < threshold || scratch == nullptr ||
      scratch_words < sa_delta_rule_scratch_words(num_seqs, max_q_len, H))
    threshold = 0x7fffffff;
  if (max_q_len >= threshold) {
    const int max_chunks = (max_q_len + kChunk - 1) / kChunk;
    const dim3 grid1(max_chunks, num_seqs, H), grid2(num_seqs, H, (dv + 7) / 8);
#define SA_DELTA_CHUNKED(DK)                                                                                          \
  do {                                                                                                                \
    delta_chunk_factors_kernel<DK><<<grid1, 256, 0, stream>>>(qkv, C, G, dk, gates, H, seq_meta, threshold, scratch,  \
                                                              max_chunks);                                           \
    delta_chunk_scan_kernel<DK><<<grid2, 256, 0, stream>>>(qkv, C, G, dk, dv, H, state, state_stride, seq_meta,        \
                                                           threshold, scratch, max_chunks, out);                      \
  } while (0)
    if (dk <= 32) SA_DELTA_CHUNKED(32);
    else if (dk <= 64) SA_DELTA_CHUNKED(64);
    else SA_DELTA_CHUNKED(128);
#undef SA_DELTA_CHUNKED
    if (check_launch("delta_rule (chunked)")) return 1;
    if (min_q_len >= threshold) return 0;   // nobody is left for the token-by-token kernel
  }
#define SA_DELTA_RULE(DK, LPC, TT)                                                                                  \
  delta_rule_kernel<DK, LPC, TT><<<dim3(num_seqs, H, (dv + 256 / LPC - 1) / (256 / LPC)), 256, 0, stream>>>(         \
      qkv, C, G, dk, dv, gates, H, state, state_stride, seq_meta, out, threshold)
  // (16 tokens per tile: 32 gave the same time per token of a prompt and cost the decode step a third more)
  if (dk <= 16) SA_DELTA_RULE(16, 4, 16);
  else if (dk <= 32) SA_DELTA_RULE(32, 4, 16);
  else if (dk <= 64) SA_DELTA_RULE(64, 16, 16);
  else if (dk <= 128) SA_DELTA_RULE(128, 64, 16);
  else SA_DELTA_RULE(256, 64, 16);
#undef SA_DELTA_RULE
  return check_launch("delta_rule");
}
