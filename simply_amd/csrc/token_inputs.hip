// Kernels that read tables by token: an embedding that adds a hashed pair-of-tokens row and a learned position row
// to the token's row, and a gate that is multiplied by a token's row of a side table.  Also two small row kernels
// that mixers with biases and mixers that run side by side need: a bias added in place, and a weighted sum of two
// results.
#include "api.h"
#include "common.h"

namespace sa {

// out[t, :] = table[token] + pair[row] + pos[position]  (32-bit sums in this order; pair or pos null: left out).
// row = (previous * mul_prev + token * mul_cur) mod buckets, or `buckets` (the table's last row) for a request's
// first token.  The token before a step's first one is the slot's entry of `last` (int32 per slot), which the
// workgroup of a request's first token of the step reads and then sets to the step's last token of the request: it
// alone touches the entry.  Grid (most tokens of a request, requests).
__global__ void embed_sum_kernel(const int* __restrict__ tokens, const int* __restrict__ positions,
                                 const int* __restrict__ seq_meta, const void* __restrict__ table, int table_dtype,
                                 const void* __restrict__ pair, int pair_dtype, long long buckets, long long mul_prev,
                                 long long mul_cur, int* __restrict__ last, int64_t last_stride,
                                 const void* __restrict__ pos, int pos_dtype, int max_positions, float* __restrict__ out,
                                 int D) {
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int j = blockIdx.x;
  if (j >= count) return;
  const int t = first + j;
  const int token = tokens[t], p = positions[t];
  long long row = buckets;
  if (pair != nullptr) {
    int* mine = last + static_cast<size_t>(slot) * last_stride;
    const int before = j > 0 ? tokens[t - 1] : *mine;
    if (p > 0) row = (static_cast<long long>(before) * mul_prev + static_cast<long long>(token) * mul_cur) % buckets;
    __syncthreads();   // every thread has read the entry
    if (j == 0 && threadIdx.x == 0) *mine = tokens[first + count - 1];
  }
  const int pp = p < max_positions ? p : max_positions - 1;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float v = load_f(table, table_dtype, static_cast<size_t>(token) * D + d);
    if (pair != nullptr) v += load_f(pair, pair_dtype, static_cast<size_t>(row) * D + d);
    if (pos != nullptr) v += load_f(pos, pos_dtype, static_cast<size_t>(pp) * D + d);
    out[static_cast<size_t>(t) * D + d] = v;
  }
}

// z[t, j] = act(z[t, j]) * table[tokens[t], col0 + j] in place (the activation in 32-bit, exact).
__global__ void token_gate_kernel(void* __restrict__ z, int dtype, int64_t stride, const int* __restrict__ tokens,
                                  const void* __restrict__ table, int table_dtype, int64_t table_stride, int col0, int N,
                                  int act) {
  const int t = blockIdx.y, n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const size_t at = static_cast<size_t>(t) * stride + n;
  const float e = load_f(table, table_dtype, static_cast<size_t>(tokens[t]) * table_stride + col0 + n);
  store_f(z, dtype, at, gated_activation_exact(act, load_f(z, dtype, at)) * e);
}

// x[t, n] += b[n] in place.
__global__ void bias_add_kernel(void* __restrict__ x, int dtype, int64_t stride, const void* __restrict__ b, int b_dtype,
                                int N) {
  const int t = blockIdx.y, n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const size_t at = static_cast<size_t>(t) * stride + n;
  store_f(x, dtype, at, load_f(x, dtype, at) + load_f(b, b_dtype, n));
}

// out[t, n] = a * x[t, n] + b * y[t, n]
__global__ void weighted_sum_kernel(const void* __restrict__ x, int64_t x_stride, float a, const void* __restrict__ y,
                                    int64_t y_stride, float b, int dtype, void* __restrict__ out, int64_t out_stride,
                                    int N) {
  const int t = blockIdx.y, n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  store_f(out, dtype, static_cast<size_t>(t) * out_stride + n,
          fmaf(a, load_f(x, dtype, static_cast<size_t>(t) * x_stride + n),
               b * load_f(y, dtype, static_cast<size_t>(t) * y_stride + n)));
}

}  // namespace sa

using namespace sa;

extern "C" int sa_embed_sum(const int* tokens, const int* positions, const int* seq_meta, int num_seqs, int max_q_len,
                            const void* table, int table_dtype, int V, const void* pair, int pair_dtype, int64_t buckets,
                            int64_t mul_prev, int64_t mul_cur, int* last, int64_t last_stride, const void* pos,
                            int pos_dtype, int max_positions, float* out, int D, hipStream_t stream) {
  if (num_seqs == 0 || max_q_len == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && num_seqs <= 65535 && max_q_len > 0 && D > 0 && V > 0, "embed_sum: bad sizes S=%d q=%d D=%d",
             num_seqs, max_q_len, D);
  SA_REQUIRE(tokens != nullptr && positions != nullptr && seq_meta != nullptr && table != nullptr && out != nullptr,
             "embed_sum: a null pointer");
  SA_REQUIRE(pair == nullptr || (buckets > 0 && last != nullptr && last_stride >= 1 && mul_prev >= 0 && mul_cur >= 0),
             "embed_sum: a table of pairs needs its buckets and the slots' last tokens");
  SA_REQUIRE(pos == nullptr || max_positions > 0, "embed_sum: a table of positions needs its length");
  const int threads = D >= 1024 ? 256 : D >= 256 ? 128 : 64;
  embed_sum_kernel<<<dim3(max_q_len, num_seqs), threads, 0, stream>>>(tokens, positions, seq_meta, table, table_dtype, pair,
                                                                      pair_dtype, buckets, mul_prev, mul_cur, last,
                                                                      last_stride, pos, pos_dtype, max_positions, out, D);
  return check_launch("embed_sum");
}

extern "C" int sa_token_gate(void* z, int dtype, int64_t stride, const int* tokens, const void* table, int table_dtype,
                             int64_t table_stride, int col0, int T, int N, int act, hipStream_t stream) {
  if (T == 0 || N == 0) return 0;
  SA_REQUIRE(T > 0 && T <= 65535 && N > 0 && stride >= N && col0 >= 0 && table_stride >= col0 + N,
             "token_gate: bad sizes T=%d N=%d", T, N);
  SA_REQUIRE(act >= 0 && act < kNumActivations, "token_gate: unknown activation %d", act);
  SA_REQUIRE(z != nullptr && tokens != nullptr && table != nullptr, "token_gate: a null pointer");
  token_gate_kernel<<<dim3((N + 255) / 256, T), 256, 0, stream>>>(z, dtype, stride, tokens, table, table_dtype,
                                                                  table_stride, col0, N, act);
  return check_launch("token_gate");
}

extern "C" int sa_bias_add(void* x, int dtype, int64_t stride, const void* b, int b_dtype, int T, int N,
                           hipStream_t stream) {
  if (T == 0 || N == 0) return 0;
  SA_REQUIRE(T > 0 && T <= 65535 && N > 0 && stride >= N && x != nullptr && b != nullptr, "bias_add: bad sizes T=%d N=%d", T,
             N);
  bias_add_kernel<<<dim3((N + 255) / 256, T), 256, 0, stream>>>(x, dtype, stride, b, b_dtype, N);
  return check_launch("bias_add");
}

extern "C" int sa_weighted_sum(const void* x, int64_t x_stride, float a, const void* y, int64_t y_stride, float b,
                               int dtype, void* out, int64_t out_stride, int T, int N, hipStream_t stream) {
  if (T == 0 || N == 0) return 0;
  SA_REQUIRE(T > 0 && T <= 65535 && N > 0 && x_stride >= N && y_stride >= N && out_stride >= N,
             "weighted_sum: bad sizes T=%d N=%d", T, N);
  SA_REQUIRE(x != nullptr && y != nullptr && out != nullptr, "weighted_sum: a null pointer");
  weighted_sum_kernel<<<dim3((N + 255) / 256, T), 256, 0, stream>>>(x, x_stride, a, y, y_stride, b, dtype, out, out_stride,
                                                                    N);
  return check_launch("weighted_sum");
}
