// Gated linear recurrence with a short causal convolution in front (the recurrent block of Griffin-style designs), over
// the engine's per-sequence state slots.
//
//   conv_state   out[t, c] = b[c] + sum_k taps[c, k] * in[t - (K - 1) + k, c]; inputs before the step's first row come
//                from the slot's tail (the last K - 1 inputs of the sequence), an empty (zero) history at position 0.  The
//                tail is rewritten with the step's last K - 1 inputs (shifted in place when the step is shorter).  An
//                optional SiLU on the output, or the row's own input added to it (in + conv(in)).
//   lru_scan     r = sigmoid(gate_r), i = sigmoid(gate_i), log a = -c r softplus(lam), S = a S + sqrt(1 - a^2) i u,
//                out = S * y.  The state S is fp32 and lives in the sequence's slot; a sequence's first step starts from
//                S = 0 (position 0 is not special-cased beyond that: the recurrence's own formula applies to it).
//
// The convolution and the recurrence's coefficients (every sigmoid, softplus, exponential and root) are computed for
// all rows in parallel; only S = a S + b and the product with the gelu branch walk a sequence's rows in order, one
// thread per (sequence, channel) -- a decode step is one iteration.  The biases of the two input projections and the
// gelu of the branch are applied here, so those projections are plain GEMMs with fp32 output.  Everything here is fp32
// whatever the element type of the projections around it.
#include "api_layers.h"

namespace dsse {
namespace {

DEV float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }
DEV float softplusf(float x) { return x > 20.0f ? x : log1pf(expf(x)); }
DEV float gelu_tanh_f(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

constexpr int kConvRows = 8;   // rows per workgroup of the convolution (its rows are independent of each other)

template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(ConvStateParams p) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ql = p.q_len[seq];
  const int t0 = blockIdx.z * kConvRows;
  if (c >= p.C || t0 >= ql) return;
  // single: one launch block per sequence walks all of its rows (one, in a decode step) and then moves the tail itself
  const int t1 = p.single ? ql : (t0 + kConvRows < ql ? t0 + kConvRows : ql);
  const int K = p.K, Kt = K - 1;
  const int row0 = p.q_start[seq];
  const bool fresh = p.ctx_len[seq] - ql == 0;  // the sequence starts in this step: nothing before it
  float* tail = p.tail + (int64_t)p.state_slot[seq] * Kt * p.C + c;  // tail[j * C]: input at offset j - Kt
  const T* taps = reinterpret_cast<const T*>(p.taps) + (int64_t)c * K;
  const float bias = p.bias ? (float)reinterpret_cast<const T*>(p.bias)[c] : 0.0f;
  const float ib = p.in_bias ? (float)reinterpret_cast<const T*>(p.in_bias)[c] : 0.0f;  // the input projection's bias
  const float* in = p.in + (int64_t)row0 * p.ld_in + c;
  for (int t = t0; t < t1; ++t) {
    float v = bias;
    for (int k = 0; k < K; ++k) {
      const int i = t - Kt + k;
      const float x = i >= 0 ? in[(int64_t)i * p.ld_in] + ib : (fresh ? 0.0f : tail[(int64_t)(Kt + i) * p.C]);
      v += (float)taps[k] * x;
    }
    if (p.act == 1) v = v / (1.0f + expf(-v));
    else if (p.act == 2) v += in[(int64_t)t * p.ld_in] + ib;
    if (p.out) p.out[(int64_t)(row0 + t) * p.C + c] = v;
    if (p.out_b) reinterpret_cast<T*>(p.out_b)[(int64_t)(row0 + t) * p.C + c] = (T)v;
  }
  if (p.single)  // this thread alone reads and writes its (slot, channel): ascending, as in conv_tail_kernel
    for (int j = 0; j < Kt; ++j) {
      const int i = ql - Kt + j;
      tail[(int64_t)j * p.C] = i >= 0 ? in[(int64_t)i * p.ld_in] + ib : (fresh ? 0.0f : tail[(int64_t)(Kt + i) * p.C]);
    }
}

// After every row of the step has read the old tail: the slot's new tail = the step's last K - 1 inputs.  Ascending:
// entry j takes the input at offset ql - Kt + j, which for a short step is the old entry j + ql (> j, not yet
// overwritten).
template <typename T>
__global__ __launch_bounds__(256) void conv_tail_kernel(ConvStateParams p) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ql = p.q_len[seq];
  if (c >= p.C || ql <= 0) return;
  const int Kt = p.K - 1;
  const bool fresh = p.ctx_len[seq] - ql == 0;
  float* tail = p.tail + (int64_t)p.state_slot[seq] * Kt * p.C + c;
  const float ib = p.in_bias ? (float)reinterpret_cast<const T*>(p.in_bias)[c] : 0.0f;
  const float* in = p.in + (int64_t)p.q_start[seq] * p.ld_in + c;
  for (int j = 0; j < Kt; ++j) {
    const int i = ql - Kt + j;
    tail[(int64_t)j * p.C] = i >= 0 ? in[(int64_t)i * p.ld_in] + ib : (fresh ? 0.0f : tail[(int64_t)(Kt + i) * p.C]);
  }
}

// Everything of the recurrence that does not depend on the state, for every row at once: the gates' pre-activations
// [recurrence gate | input gate] of each block are overwritten with (a, b) of S = a S + b:
// a = exp(-c sigmoid(g_r) softplus(lam)), b = sqrt(1 - a^2) sigmoid(g_i) u.
template <typename T>
__global__ __launch_bounds__(256) void lru_coeff_kernel(LruScanParams p, int rows) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int64_t row = blockIdx.x;
  if (c >= p.C) return;
  const float sp = softplusf((float)reinterpret_cast<const T*>(p.lam)[c]);
  const int b = c / p.bw, o = c % p.bw;
  float* g = const_cast<float*>(p.gates) + row * 2 * p.C + (int64_t)b * 2 * p.bw;
  const float r = sigmoidf(g[o]), gi = sigmoidf(g[p.bw + o]);
  const float log_a = -p.c * r * sp;
  g[o] = expf(log_a);
  g[p.bw + o] = sqrtf(-expm1f(2.0f * log_a)) * gi * p.u[row * p.C + c];  // sqrt(1 - a^2) without cancellation near a = 1
}

template <typename T>
__global__ __launch_bounds__(256) void lru_scan_kernel(LruScanParams p) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ql = p.q_len[seq];
  if (c >= p.C || ql <= 0) return;
  const int row0 = p.q_start[seq];
  float* st = p.state + (int64_t)p.state_slot[seq] * p.C + c;
  float S = p.ctx_len[seq] - ql == 0 ? 0.0f : *st;
  const int b = c / p.bw, o = c % p.bw;
  const float yb = p.y_bias ? (float)reinterpret_cast<const T*>(p.y_bias)[c] : 0.0f;
  const float* ab = p.gates + (int64_t)row0 * 2 * p.C + (int64_t)b * 2 * p.bw + o;
  const float* y = p.y + (int64_t)row0 * p.C + c;
  T* out = reinterpret_cast<T*>(p.out) + (int64_t)row0 * p.C + c;
  int t = 0;
  for (; t + 4 <= ql; t += 4) {  // the loads of four steps are in flight before the four dependent updates
    float a[4], bb[4], yy[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = ab[(int64_t)(t + i) * 2 * p.C];
      bb[i] = ab[(int64_t)(t + i) * 2 * p.C + p.bw];
      yy[i] = y[(int64_t)(t + i) * p.C];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      S = a[i] * S + bb[i];
      out[(int64_t)(t + i) * p.C] = (T)(S * gelu_tanh_f(yy[i] + yb));
    }
  }
  for (; t < ql; ++t) {
    S = ab[(int64_t)t * 2 * p.C] * S + ab[(int64_t)t * 2 * p.C + p.bw];
    out[(int64_t)t * p.C] = (T)(S * gelu_tanh_f(y[(int64_t)t * p.C] + yb));
  }
  *st = S;
}

// Prompt portions: the walk in three phases so that no thread takes more than ~3 x 32 dependent steps.  A chunk is
// kScanRows rows of one sequence; its scratch slot is (first row) / kScanRows + (sequence index), which is unique because
// sequences are packed in row order.
//   1. per chunk, in parallel: A = prod a_t and B = the chunk's walk from S = 0          (S_end = A S_in + B)
//   2. per sequence: the chunks in order -- each chunk's incoming state replaces its B, the last one is the slot's state
//   3. per chunk, in parallel: the walk from the incoming state, times gelu(branch + bias)
constexpr int kScanRows = 32;
constexpr int kChunkedFrom = 128;  // rows of a step from which the walk is chunked (below: one thread per sequence)

DEV int scan_slot(int row0, int t0, int seq) { return (row0 + t0) / kScanRows + seq; }

__global__ __launch_bounds__(256) void lru_chunk_reduce_kernel(LruScanParams p) {
  const int seq = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ql = p.q_len[seq], t0 = blockIdx.z * kScanRows;
  if (c >= p.C || t0 >= ql) return;
  const int t1 = t0 + kScanRows < ql ? t0 + kScanRows : ql;
  const int row0 = p.q_start[seq];
  const int b = c / p.bw, o = c % p.bw;
  const float* ab = p.gates + (int64_t)row0 * 2 * p.C + (int64_t)b * 2 * p.bw + o;
  float A = 1.0f, B = 0.0f;
  for (int t = t0; t < t1; ++t) {
    const float a = ab[(int64_t)t * 2 * p.C];
    B = a * B + ab[(int64_t)t * 2 * p.C + p.bw];
    A *= a;
  }
  const int64_t s = (int64_t)scan_slot(row0, t0, seq) * p.C + c;
  p.chunk_a[s] = A;
  p.chunk_b[s] = B;
}

__global__ __launch_bounds__(256) void lru_chunk_carry_kernel(LruScanParams p) {
  const int seq = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ql = p.q_len[seq];
  if (c >= p.C || ql <= 0) return;
  const int row0 = p.q_start[seq];
  float* st = p.state + (int64_t)p.state_slot[seq] * p.C + c;
  float S = p.ctx_len[seq] - ql == 0 ? 0.0f : *st;
  for (int t0 = 0; t0 < ql; t0 += kScanRows) {
    const int64_t s = (int64_t)scan_slot(row0, t0, seq) * p.C + c;
    const float next = p.chunk_a[s] * S + p.chunk_b[s];
    p.chunk_b[s] = S;  // the chunk's incoming state
    S = next;
  }
  *st = S;
}

template <typename T>
__global__ __launch_bounds__(256) void lru_chunk_apply_kernel(LruScanParams p) {
  const int seq = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ql = p.q_len[seq], t0 = blockIdx.z * kScanRows;
  if (c >= p.C || t0 >= ql) return;
  const int t1 = t0 + kScanRows < ql ? t0 + kScanRows : ql;
  const int row0 = p.q_start[seq];
  const int b = c / p.bw, o = c % p.bw;
  const float yb = p.y_bias ? (float)reinterpret_cast<const T*>(p.y_bias)[c] : 0.0f;
  const float* ab = p.gates + (int64_t)row0 * 2 * p.C + (int64_t)b * 2 * p.bw + o;
  const float* y = p.y + (int64_t)row0 * p.C + c;
  T* out = reinterpret_cast<T*>(p.out) + (int64_t)row0 * p.C + c;
  float S = p.chunk_b[(int64_t)scan_slot(row0, t0, seq) * p.C + c];
  for (int t = t0; t < t1; ++t) {
    S = ab[(int64_t)t * 2 * p.C] * S + ab[(int64_t)t * 2 * p.C + p.bw];
    out[(int64_t)t * p.C] = (T)(S * gelu_tanh_f(y[(int64_t)t * p.C] + yb));
  }
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_conv_state(const dsse::ConvStateParams* p, hipStream_t st) {
  if (p->nseq <= 0 || p->rows <= 0) return hipSuccess;
  dim3 grid((p->C + 255) / 256, p->nseq, p->single ? 1 : (p->rows + dsse::kConvRows - 1) / dsse::kConvRows);
  dim3 tgrid((p->C + 255) / 256, p->nseq);
  const bool tails = p->K > 1 && !p->single;
  if (p->f32) {
    hipLaunchKernelGGL(dsse::conv_state_kernel<float>, grid, dim3(256), 0, st, *p);
    if (tails) hipLaunchKernelGGL(dsse::conv_tail_kernel<float>, tgrid, dim3(256), 0, st, *p);
  } else {
    hipLaunchKernelGGL(dsse::conv_state_kernel<bf16>, grid, dim3(256), 0, st, *p);
    if (tails) hipLaunchKernelGGL(dsse::conv_tail_kernel<bf16>, tgrid, dim3(256), 0, st, *p);
  }
  return hipGetLastError();
}

extern "C" hipError_t dsse_lru_scan(const dsse::LruScanParams* p, hipStream_t st) {
  if (p->nseq <= 0 || p->rows <= 0) return hipSuccess;
  dim3 cgrid(p->rows, (p->C + 255) / 256);
  dim3 grid((p->C + 255) / 256, p->nseq);
  if (p->coeff) {
    if (p->f32) hipLaunchKernelGGL(dsse::lru_coeff_kernel<float>, cgrid, dim3(256), 0, st, *p, p->rows);
    else hipLaunchKernelGGL(dsse::lru_coeff_kernel<bf16>, cgrid, dim3(256), 0, st, *p, p->rows);
  }
  if (p->chunk_a && p->chunk_b && p->rows >= dsse::kChunkedFrom) {  // prompt portions: the three-phase walk
    dim3 zgrid((p->C + 255) / 256, p->nseq, (p->rows + dsse::kScanRows - 1) / dsse::kScanRows);
    hipLaunchKernelGGL(dsse::lru_chunk_reduce_kernel, zgrid, dim3(256), 0, st, *p);
    hipLaunchKernelGGL(dsse::lru_chunk_carry_kernel, grid, dim3(256), 0, st, *p);
    if (p->f32) hipLaunchKernelGGL(dsse::lru_chunk_apply_kernel<float>, zgrid, dim3(256), 0, st, *p);
    else hipLaunchKernelGGL(dsse::lru_chunk_apply_kernel<bf16>, zgrid, dim3(256), 0, st, *p);
    return hipGetLastError();
  }
  if (p->f32) hipLaunchKernelGGL(dsse::lru_scan_kernel<float>, grid, dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::lru_scan_kernel<bf16>, grid, dim3(256), 0, st, *p);
  return hipGetLastError();
}
