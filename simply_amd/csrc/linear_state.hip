// Recurrent mixers whose state is a matrix per head that decays and takes one outer product per token:
//
//   S_t = diag(a_t) S_(t-1) + c_t k_t v_t^T,   o_t = S_t^T q_t
//
// with a decay per key channel and c = 1 (gated linear attention), or with one decay and one input factor per head
// (the matrix memory with exponential gates, whose decay and factor come from a running maximum of the logarithms
// of its gates; its normalizer n_t = a_t n_(t-1) + c_t k_t is one more column of S whose value is always 1).
//
//   exp_gates_kernel          i, f from their projections, the running maximum m, a = exp(f + m' - m), c = exp(i - m)
//   linear_state_kernel       the recurrence, prefill and decode; a decay per channel may come as z with
//                             a = sigmoid(z + b)^(1/tau), computed as the tile is staged
//   normalized_readout_kernel o / (max(|n.q|, exp(-m)) + 1e-6), each head to unit RMS, times a weight and sigmoid(gate)
//
// A request's tokens of this step are rows first .. first + count - 1 (seq_meta [S, 4]: state slot, first row, count,
// position of the first); what earlier steps left is the slot's state.  Gates, decays, sums and the state are 32-bit;
// q, k and v are read from the projection in its own element type.  Sums run in an order that depends on the sizes
// alone, so a token's result does not depend on how the tokens are cut into steps or on the batch.
#include <type_traits>

#include "api.h"
#include "common.h"

namespace sa {

__device__ inline float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// The gates of the matrix memory.  raw [T, 2 H]: the projections of the input and forget gates (input gates first),
// bias [2 H] alike (null: none).  i = cap tanh((x_i + b_i) / cap), f = log_sigmoid(cap tanh((x_f + b_f) / cap));
// m_t = max(f + m_(t-1), i) from the slot's m (which starts at 0);
// gates [T, 3 H]: exp(f + m_(t-1) - m_t), exp(i - m_t), exp(-m_t).  A wave per (request, head) takes 64 tokens at a
// time: their gates in parallel, the maximum one token after the other through lane reads.
__global__ __launch_bounds__(kWave) void exp_gates_kernel(const float* __restrict__ raw, int64_t raw_stride,
                                                          const void* __restrict__ bias, int bias_dtype, float cap, int H,
                                                          float* __restrict__ m_state, int64_t state_stride,
                                                          const int* __restrict__ seq_meta, float* __restrict__ gates) {
  const int* meta = seq_meta + 4 * blockIdx.x;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int h = blockIdx.y, lane = threadIdx.x;
  if (count <= 0) return;
  float* mp = m_state + static_cast<size_t>(slot) * state_stride + h;
  float m = *mp;
  const float bi = bias != nullptr ? load_f(bias, bias_dtype, h) : 0.f;
  const float bf = bias != nullptr ? load_f(bias, bias_dtype, H + h) : 0.f;
  for (int t0 = 0; t0 < count; t0 += kWave) {
    const int tn = count - t0 < kWave ? count - t0 : kWave;
    const bool ok = lane < tn;
    const size_t row = static_cast<size_t>(first + t0 + (ok ? lane : 0));
    const float xi = raw[row * raw_stride + h] + bi, xf = raw[row * raw_stride + H + h] + bf;
    const float ig = cap * tanhf(xi / cap);
    const float fg = log_sigmoid(cap * tanhf(xf / cap));
    float before = 0.f, after = 0.f;
#pragma unroll
    for (int j = 0; j < kWave; ++j) {
      const float fj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fg), j));
      const float ij = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ig), j));
      const float next = fmaxf(fj + m, ij);
      if (lane == j) {
        before = m;
        after = next;
      }
      m = j < tn ? next : m;
    }
    if (ok) {
      float* g = gates + row * 3 * H;
      g[h] = expf(fg + before - after);
      g[H + h] = expf(ig - after);
      g[2 * H + h] = expf(-after);
    }
  }
  if (lane == 0) *mp = m;
}

// The recurrence.  A workgroup of 256 threads takes 256 / LPC columns of one head's state for one request: LPC lanes
// share a column, lane `part` of them holding rows part, part + LPC, ... of it in registers.  The step's q, k, v and
// decays of kStateTokens tokens at a time go through LDS, asked for a tile ahead.  SCALAR: one decay and one input
// factor per head and token (gates [T, >= 2 H]: decays, then factors); else a decay per key channel (gates
// [T, H * dk]) and no factor.  `ones`: 1 if the state has one more column whose value is always 1 (column dv).
// The state of a head is kept column by column, [dv + ones][dk].
constexpr int kStateTokens = 16;
template <int DK, int LPC, bool SCALAR, typename XT>
__global__ __launch_bounds__(256) void linear_state_kernel(
    const XT* __restrict__ proj, int64_t proj_stride, int q_at, int k_at, int v_at, float q_mult,
    const float* __restrict__ gates, int64_t gates_stride, const void* __restrict__ gate_bias, int bias_dtype,
    float inv_tau, int H, int dk, int dv, int ones, float* __restrict__ state, int64_t state_stride,
    const int* __restrict__ seq_meta, float* __restrict__ out) {
  constexpr int R = DK / LPC, COLS = 256 / LPC;
  constexpr int AD = SCALAR ? 1 : DK;
  __shared__ float qs[kStateTokens][DK], ks[kStateTokens][DK], vs[kStateTokens][COLS], as[kStateTokens][AD],
      cs[kStateTokens][2];
  const int* meta = seq_meta + 4 * blockIdx.x;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int h = blockIdx.y, tid = threadIdx.x;
  const int CT = dv + ones;
  const int col = blockIdx.z * COLS + tid / LPC, part = tid % LPC;
  const bool live = col < CT;
  float* S = state + static_cast<size_t>(slot) * state_stride + static_cast<size_t>(h) * dk * CT;
  float s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = r * LPC + part;
    s[r] = (live && i < dk) ? S[static_cast<size_t>(col) * dk + i] : 0.f;
  }
  constexpr int PQ = kStateTokens * DK / 256, PV = (kStateTokens * COLS + 255) / 256;
  float pq[PQ], pk[PQ], pa[SCALAR ? 1 : PQ], pb[SCALAR ? 1 : PQ], pv[PV], pc = 0.f;
  bool pok[SCALAR ? 1 : PQ];
  auto fetch = [&](int t0) __attribute__((always_inline)) {
    const int tn = count - t0 < kStateTokens ? count - t0 : kStateTokens;
#pragma unroll
    for (int i = 0; i < PQ; ++i) {
      const int idx = tid + i * 256, j = idx / DK, d = idx % DK;
      const bool ok = j < tn && d < dk;
      const size_t t = static_cast<size_t>(first + t0 + (ok ? j : 0));
      const XT* row = proj + t * proj_stride;
      pq[i] = ok ? to_float(row[q_at + h * dk + d]) * q_mult : 0.f;
      pk[i] = ok ? to_float(row[k_at + h * dk + d]) : 0.f;
      if constexpr (!SCALAR) {
        // (with inv_tau > 0 the gates are z and the bias rides along: the decay is computed when the tile is put into
        // LDS, a tile later, so that nothing waits for these loads here)
        pa[i] = ok ? gates[t * gates_stride + h * dk + d] : 0.f;
        if (inv_tau > 0.f) pb[i] = (ok && gate_bias != nullptr) ? load_f(gate_bias, bias_dtype, h * dk + d) : 0.f;
        pok[i] = ok;
      }
    }
#pragma unroll
    for (int i = 0; i < PV; ++i) {
      const int idx = tid + i * 256, j = idx / COLS, c = blockIdx.z * COLS + idx % COLS;
      const bool ok = idx < kStateTokens * COLS && j < tn && c < CT;
      pv[i] = !ok ? 0.f : c < dv ? to_float(proj[static_cast<size_t>(first + t0 + j) * proj_stride + v_at + h * dv + c]) : 1.f;
    }
    if constexpr (SCALAR) pc = tid < 2 * tn ? gates[static_cast<size_t>(first + t0 + tid / 2) * gates_stride + (tid % 2) * H + h] : 0.f;
  };
  if (count > 0) fetch(0);
  for (int t0 = 0; t0 < count; t0 += kStateTokens) {
    const int tn = count - t0 < kStateTokens ? count - t0 : kStateTokens;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PQ; ++i) {
      const int idx = tid + i * 256;
      qs[idx / DK][idx % DK] = pq[i];
      ks[idx / DK][idx % DK] = pk[i];
      if constexpr (!SCALAR) {
        // a = sigmoid(z + bias)^(1 / tau): a bfloat16 run takes the hardware's exponential and logarithm, a 32-bit
        // run the library's
        float a = pa[i];
        if (inv_tau > 0.f && pok[i]) {
          a += pb[i];
          if constexpr (sizeof(XT) == 2) a = __expf((fminf(a, 0.f) - __logf(1.f + __expf(-fabsf(a)))) * inv_tau);
          else a = expf(log_sigmoid(a) * inv_tau);
        }
        as[idx / DK][idx % AD] = a;
      }
    }
#pragma unroll
    for (int i = 0; i < PV; ++i) {
      const int idx = tid + i * 256;
      if (idx < kStateTokens * COLS) vs[idx / COLS][idx % COLS] = pv[i];
    }
    if constexpr (SCALAR) if (tid < 2 * kStateTokens) cs[tid / 2][tid % 2] = pc;
    __syncthreads();
    if (t0 + kStateTokens < count) fetch(t0 + kStateTokens);
    // four tokens at a time: their updates follow one another, their sums across the lanes run side by side (a wave
    // issues in order, and one such sum alone is a chain of dependent steps that nothing else covers).  A whole tile
    // runs without a test per token, so that the reads of its operands can be asked for ahead of their use.
    auto group = [&](int j0, auto whole) __attribute__((always_inline)) {
      constexpr bool WHOLE = decltype(whole)::value;
      float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = j0 + i;
        if (WHOLE || j < tn) {   // (uniform)
          float u = vs[j][tid / LPC], a0 = 1.f;
          if constexpr (SCALAR) {
            a0 = cs[j][0];
            u *= cs[j][1];
          }
          float d[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int r = 0; r < R; ++r) {
            float a = a0;
            if constexpr (!SCALAR) a = as[j][(r * LPC + part) % AD];
            s[r] = fmaf(ks[j][r * LPC + part], u, s[r] * a);
            d[r % 4] = fmaf(s[r], qs[j][r * LPC + part], d[r % 4]);
          }
          o[i] = (d[0] + d[1]) + (d[2] + d[3]);
        }
      }
      lanes_sum4<LPC>(o);
      if (live && part == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (WHOLE || j0 + i < tn)
            out[static_cast<size_t>(first + t0 + j0 + i) * (static_cast<size_t>(H) * CT) + static_cast<size_t>(h) * CT + col] = o[i];
      }
    };
    if (tn == kStateTokens) {
#pragma unroll
      for (int j0 = 0; j0 < kStateTokens; j0 += 4) group(j0, std::true_type{});
    } else {
      for (int j0 = 0; j0 < tn; j0 += 4) group(j0, std::false_type{});
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = r * LPC + part;
    if (live && i < dk) S[static_cast<size_t>(col) * dk + i] = s[r];
  }
}

// out[t, h, :] = unit_rms(x[t, h, 0:size] / (max(|x[t, h, size]|, floor[t, h]) + 1e-6)) * w[h, :] * sigmoid(g[t, h, :]):
// x has size + 1 entries per head, the last one being the normalizer's product with the query; floor is exp(-m).
// A wave per (token, head).
__global__ __launch_bounds__(kWave) void normalized_readout_kernel(
    const float* __restrict__ x, const float* __restrict__ floor, int64_t floor_stride, const void* __restrict__ g,
    int g_dtype, int64_t g_stride, const void* __restrict__ w, int w_dtype, float eps, void* __restrict__ out,
    int out_dtype, int64_t out_stride, int H, int size) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* head = x + (static_cast<size_t>(t) * H + h) * (size + 1);
  const float denom = fmaxf(fabsf(head[size]), floor[static_cast<size_t>(t) * floor_stride + h]) + 1e-6f;
  float ss = 0.f;
  for (int d = threadIdx.x; d < size; d += kWave) {
    const float v = head[d] / denom;
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float r = 1.f / sqrtf(ss / static_cast<float>(size) + eps);
  for (int d = threadIdx.x; d < size; d += kWave) {
    const float v = head[d] / denom * r * load_f(w, w_dtype, static_cast<size_t>(h) * size + d);
    const float gate = load_f(g, g_dtype, static_cast<size_t>(t) * g_stride + static_cast<size_t>(h) * size + d);
    store_f(out, out_dtype, static_cast<size_t>(t) * out_stride + static_cast<size_t>(h) * size + d,
            v / (1.f + expf(-gate)));
  }
}

}  // namespace sa

using namespace sa;

extern "C" int sa_exp_gates(const float* raw, int64_t raw_stride, const void* bias, int bias_dtype, float cap, int H,
                            float* m_state, int64_t state_stride, const int* seq_meta, int num_seqs, float* gates,
                            hipStream_t stream) {
  if (num_seqs == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && num_seqs <= 65535 && H > 0 && H <= 65535 && raw_stride >= 2 * H && cap > 0.f,
             "exp_gates: bad sizes S=%d H=%d", num_seqs, H);
  SA_REQUIRE(raw != nullptr && m_state != nullptr && seq_meta != nullptr && gates != nullptr && state_stride >= H,
             "exp_gates: a null pointer or state rows too short");
  exp_gates_kernel<<<dim3(num_seqs, H), kWave, 0, stream>>>(raw, raw_stride, bias, bias_dtype, cap, H, m_state,
                                                            state_stride, seq_meta, gates);
  return check_launch("exp_gates");
}

extern "C" int sa_linear_state(const void* proj, int dtype, int64_t proj_stride, int q_at, int k_at, int v_at,
                               float q_mult, const float* gates, int64_t gates_stride, const void* gate_bias,
                               int bias_dtype, float tau, int scalar, int H, int dk, int dv, int ones, float* state,
                               int64_t state_stride, const int* seq_meta, int num_seqs, float* out, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && num_seqs <= 65535 && H > 0 && H <= 65535 && dk > 0 && dv > 0 && (ones == 0 || ones == 1),
             "linear_state: bad sizes S=%d H=%d dk=%d dv=%d", num_seqs, H, dk, dv);
  SA_REQUIRE(dk <= 256, "linear_state: key size %d is above 256", dk);
  const int CT = dv + ones;
  SA_REQUIRE(state_stride >= static_cast<int64_t>(H) * dk * CT, "linear_state: the state rows are too short");
  SA_REQUIRE(q_at >= 0 && k_at >= 0 && v_at >= 0 && proj_stride >= q_at + static_cast<int64_t>(H) * dk &&
                 proj_stride >= k_at + static_cast<int64_t>(H) * dk && proj_stride >= v_at + static_cast<int64_t>(H) * dv,
             "linear_state: the projection rows are too short");
  SA_REQUIRE(gates_stride >= (scalar ? 2 * H : H * dk), "linear_state: the gate rows are too short");
  SA_REQUIRE(proj != nullptr && gates != nullptr && state != nullptr && seq_meta != nullptr && out != nullptr,
             "linear_state: a null pointer");
  SA_REQUIRE(dtype == kF32 || dtype == kBF16, "linear_state: unknown dtype %d", dtype);
  SA_REQUIRE(CT <= 65535 * 4, "linear_state: too many columns");
  SA_REQUIRE(tau >= 0.f && (scalar == 0 || tau == 0.f), "linear_state: tau belongs to decays per channel and is not negative");
  const float inv_tau = tau > 0.f ? 1.f / tau : 0.f;
#define SA_STATE_LAUNCH(DK, LPC, SC, XT)                                                                             \
  linear_state_kernel<DK, LPC, SC, XT><<<dim3(num_seqs, H, (CT + 256 / LPC - 1) / (256 / LPC)), 256, 0, stream>>>(   \
      static_cast<const XT*>(proj), proj_stride, q_at, k_at, v_at, q_mult, gates, gates_stride, gate_bias, bias_dtype, \
      inv_tau, H, dk, dv, ones, state, state_stride, seq_meta, out)
#define SA_STATE_SIZES(SC, XT)                       \
  do {                                               \
    if (dk <= 16) SA_STATE_LAUNCH(16, 4, SC, XT);    \
    else if (dk <= 32) SA_STATE_LAUNCH(32, 4, SC, XT);    \
    else if (dk <= 64) SA_STATE_LAUNCH(64, 16, SC, XT);   \
    else if (dk <= 128) SA_STATE_LAUNCH(128, 32, SC, XT); \
    else SA_STATE_LAUNCH(256, 64, SC, XT);           \
  } while (0)
  if (dtype == kBF16) {
    if (scalar) SA_STATE_SIZES(true, bf16);
    else SA_STATE_SIZES(false, bf16);
  } else {
    if (scalar) SA_STATE_SIZES(true, float);
    else SA_STATE_SIZES(false, float);
  }
#undef SA_STATE_SIZES
#undef SA_STATE_LAUNCH
  return check_launch("linear_state");
}

extern "C" int sa_normalized_readout(const float* x, const float* floor, int64_t floor_stride, const void* g, int g_dtype,
                                     int64_t g_stride, const void* w, int w_dtype, float eps, void* out, int out_dtype,
                                     int64_t out_stride, int T, int H, int size, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && H > 0 && H <= 65535 && size > 0, "normalized_readout: bad sizes T=%d H=%d size=%d", T, H, size);
  SA_REQUIRE(x != nullptr && floor != nullptr && g != nullptr && w != nullptr && out != nullptr,
             "normalized_readout: a null pointer");
  const int64_t width = static_cast<int64_t>(H) * size;
  SA_REQUIRE(floor_stride >= H && g_stride >= width && out_stride >= width, "normalized_readout: a row stride is too small");
  normalized_readout_kernel<<<dim3(T, H), kWave, 0, stream>>>(x, floor, floor_stride, g, g_dtype, g_stride, w, w_dtype, eps,
                                                              out, out_dtype, out_stride, H, size);
  return check_launch("normalized_readout");
}
