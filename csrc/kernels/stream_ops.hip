// Row-wise fp32 pieces of pre-norm designs with matrix-state mixers:
//
//   stream_step      resid += mult * y + embed[id] + vec, then xb = tanh(alpha * resid) * w + b (the element-wise norm
//                    that needs no row statistic, so the add and the norm are one pass over the row)
//   gated_act        h = act(gate) * up from the fused gate | up projection's fp32 output (SiLU or tanh-form gelu)
//   norm_rope_rows   a row of heads: RMS norm over the whole row with a gain, a unit vector per head, an RMS norm per
//                    head with one gain vector for all heads (or without a gain), or nothing;
//                    rotate-half rotation of each head's leading coordinates; a scale; written to a chosen output row
//                    (a cache row: keys and values go straight into their pages) in fp32 or bf16
//   gate_math        decays and gates in place: exp(-exp(A) softplus(x + dt)), sigmoid(x), sigmoid(x)^(1/tau)
//   gated_head_norm  out = o / rms(o) * w * silu(gate) per (row, head), or * sigmoid(gate)
//   rms_mix          out = c * (rms-norm(ya) * wa + rms-norm(yb) * wb)
//   logit_cap        logits * scale, then cap * tanh(. / cap)
//
// Everything is computed in fp32; only xb / h / out of the element type and bf16 cache rows are rounded.
#include "api_mixers.h"

namespace dsse {
namespace {

DEV float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
DEV float silu_f(float x) { return x / (1.0f + expf(-x)); }
DEV float softplus_f(float x) { return x > 20.0f ? x : log1pf(expf(x)); }
DEV float gelu_tanh_f(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

DEV float block_sum256(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < nw; ++i) s += red[i];
  return s;
}

template <typename T>
__global__ __launch_bounds__(256) void stream_step_kernel(StreamStepParams p) {
  const int row = blockIdx.x;
  float* resid = p.resid + (int64_t)row * p.W;
  const float* y = p.y ? p.y + (int64_t)row * p.W : nullptr;
  const T* e = nullptr;
  if (p.embed) {
    int id = p.ids[row];
    id = (unsigned)id < (unsigned)p.vocab ? id : 0;  // padded / inactive rows carry any id
    e = reinterpret_cast<const T*>(p.embed) + (int64_t)id * p.W;
  }
  T* xb = p.w ? reinterpret_cast<T*>(p.xb) + (int64_t)row * p.W : nullptr;
  const float alpha = p.w ? p.alpha[0] : 0.0f;
  const bool adds = y || e || p.vec;
  for (int d = threadIdx.x; d < p.W; d += blockDim.x) {
    float v = resid[d];
    if (y) v += p.mult * y[d];
    if (e) v += (float)e[d];
    if (p.vec) v += p.vec[d];
    if (adds) resid[d] = v;
    if (xb) xb[d] = (T)(tanhf(alpha * v) * p.w[d] + p.b[d]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_act_kernel(const float* gu, int ldg, T* h, int M, int F, int kind) {
  const int64_t n = (int64_t)M * F;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / F;
    const int c = (int)(i - r * F);
    const float g = gu[r * ldg + c], u = gu[r * ldg + F + c];
    h[i] = (T)((kind == 0 ? silu_f(g) : gelu_tanh_f(g)) * u);
  }
}

// One workgroup per row, one wave per head (four heads at a time).  A head's normed values pass through the wave's LDS strip so
// that a coordinate and its rotation partner are both at hand whatever lane loaded them, and so that the kernel works
// in place (out == x): a head is read completely before any of it is written.
constexpr int kMaxHeadDim = 512;

template <typename OutT>
__global__ __launch_bounds__(256) void norm_rope_rows_kernel(NormRopeParams p) {
  __shared__ float red[4];
  __shared__ float strip[4][kMaxHeadDim];
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float* x = p.x + (int64_t)row * p.ldx;
  const int N = p.nh * p.D;
  float inv_row = 1.0f;
  if (p.kind == 1) {
    float ss = 0.f;
    for (int d = threadIdx.x; d < N; d += blockDim.x) ss += x[d] * x[d];
    ss = block_sum256(ss, red);
    inv_row = 1.0f / sqrtf(ss / (float)N + p.eps);
  }
  int orow = p.out_rows ? p.out_rows[row] : row;
  if (orow < 0 || orow >= p.num_out_rows) return;  // uniform for the workgroup; after the only block-wide barrier
  OutT* out = reinterpret_cast<OutT*>(p.out) + (int64_t)orow * p.ldo;
  int pos = p.rope ? p.positions[row] : 0;
  pos = pos < 0 ? 0 : (pos >= p.rope_len ? p.rope_len - 1 : pos);
  const float2* cs = p.rope ? p.rope + (int64_t)pos * p.half : nullptr;
  const int dims = p.rope ? 2 * p.half : 0;
  float* s = strip[wave];
  for (int h0 = 0; h0 < p.nh; h0 += 4) {  // uniform trip count: the barriers below are reached by every wave
    const int h = h0 + wave;
    const bool on = h < p.nh;
    const float* xh = x + (on ? h : 0) * p.D;
    float inv = inv_row;
    if (p.kind >= 2) {
      float ss = 0.f;
      for (int i = lane; i < p.D; i += 64) ss += xh[i] * xh[i];
      ss = wave_sum(ss);
      inv = 1.0f / sqrtf((p.kind == 3 ? ss / (float)p.D : ss) + p.eps);
    }
    if (on)
      for (int i = lane; i < p.D; i += 64)
        s[i] = xh[i] * inv * (p.kind == 1 ? p.norm_w[h * p.D + i] : (p.kind == 3 && p.norm_w ? p.norm_w[i] : 1.0f));
    __syncthreads();  // the strip is written before it is read
    if (on)
      for (int i = lane; i < p.D; i += 64) {
        float v = s[i];
        if (i < dims) {
          const bool lo = i < p.half;
          const float2 c = cs[lo ? i : i - p.half];
          const float o = s[lo ? i + p.half : i - p.half];
          v = lo ? v * c.x - o * c.y : v * c.x + o * c.y;
        }
        out[h * p.D + i] = (OutT)(v * p.scale);
        if (p.out_t) {  // the same number once more where the MFMA attention's value operand wants it
          const int page = orow / kBS, off = orow % kBS;
          const int at = ((off & 15) >> 2) * 8 + ((off >> 4) & 1) * 4 + (off & 3);
          reinterpret_cast<OutT*>(p.out_t)[(((int64_t)page * p.nh + h) * p.D + i) * kBS + at] = (OutT)(v * p.scale);
        }
      }
    __syncthreads();  // the strip is read before the next head overwrites it
  }
}

__global__ __launch_bounds__(256) void gate_math_kernel(float* x, int ld, int M, int N, int kind, const float* p1,
                                                        int rep1, const float* p2, int rep2, float c) {
  const int64_t n = (int64_t)M * N;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / N;
    const int col = (int)(i - r * N);
    float* px = x + r * ld + col;
    const float v = *px;
    float o;
    if (kind == 0) {
      o = expf(-expf(p1[col / rep1]) * softplus_f(v + p2[col / rep2]));
    } else if (kind == 1) {
      o = sigmoid_f(v);
    } else {
      const float ls = fminf(v, 0.0f) - log1pf(expf(-fabsf(v)));  // log sigmoid(v)
      o = expf(ls / c);
    }
    *px = o;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* o, const float* w, const float* gate, int ldg,
                                                              T* out, int M, int H, int V, float eps, int gate_kind) {
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (row, head)
  if (item >= (int64_t)M * H) return;
  const int64_t row = item / H;
  const int h = (int)(item - row * H);
  const float* oh = o + item * V;
  const float* g = gate + row * ldg + (int64_t)h * V;
  T* dst = out + item * V;
  float ss = 0.f;
  for (int i = lane; i < V; i += 64) ss += oh[i] * oh[i];
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)V + eps);
  for (int i = lane; i < V; i += 64) dst[i] = (T)(oh[i] * inv * (w ? w[i] : 1.0f) * (gate_kind == 1 ? sigmoid_f(g[i]) : silu_f(g[i])));
}

__global__ __launch_bounds__(256) void rms_mix_kernel(const float* ya, const float* wa, const float* yb, const float* wb,
                                                      float* out, int W, float eps, float coef) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const float* a = ya + row * W;
  const float* b = yb + row * W;
  float sa = 0.f, sb = 0.f;
  for (int d = threadIdx.x; d < W; d += blockDim.x) {
    sa += a[d] * a[d];
    sb += b[d] * b[d];
  }
  sa = block_sum256(sa, red);
  sb = block_sum256(sb, red);
  const float ia = 1.0f / sqrtf(sa / (float)W + eps), ib = 1.0f / sqrtf(sb / (float)W + eps);
  for (int d = threadIdx.x; d < W; d += blockDim.x) out[row * W + d] = coef * (a[d] * ia * wa[d] + b[d] * ib * wb[d]);
}

__global__ __launch_bounds__(256) void logit_cap_kernel(float* x, int64_t n, float scale, float cap) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const float v = x[i] * scale;
    x[i] = cap > 0.0f ? cap * tanhf(v / cap) : v;
  }
}

inline int flat_blocks(int64_t n) {
  const int64_t b = (n + 255) / 256;
  return (int)(b < 1 ? 1 : (b > 4096 ? 4096 : b));
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_stream_step(const dsse::StreamStepParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  if (p->f32) hipLaunchKernelGGL(dsse::stream_step_kernel<float>, dim3(p->M), dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::stream_step_kernel<bf16>, dim3(p->M), dim3(256), 0, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_gated_act(const float* gu, int ldg, void* h, int M, int F, int kind, int f32, hipStream_t st) {
  if (M <= 0 || F <= 0) return hipSuccess;
  const int blocks = dsse::flat_blocks((int64_t)M * F);
  if (f32)
    hipLaunchKernelGGL(dsse::gated_act_kernel<float>, dim3(blocks), dim3(256), 0, st, gu, ldg, reinterpret_cast<float*>(h),
                       M, F, kind);
  else
    hipLaunchKernelGGL(dsse::gated_act_kernel<bf16>, dim3(blocks), dim3(256), 0, st, gu, ldg, reinterpret_cast<bf16*>(h),
                       M, F, kind);
  return hipGetLastError();
}

extern "C" hipError_t dsse_norm_rope_rows(const dsse::NormRopeParams* p, hipStream_t st) {
  if (p->T <= 0 || p->nh <= 0) return hipSuccess;
  if (p->D > dsse::kMaxHeadDim) return hipErrorInvalidValue;
  if (p->out_f32) hipLaunchKernelGGL(dsse::norm_rope_rows_kernel<float>, dim3(p->T), dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::norm_rope_rows_kernel<bf16>, dim3(p->T), dim3(256), 0, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_gate_math(float* x, int ld, int M, int N, int kind, const float* p1, int rep1, const float* p2,
                                     int rep2, float c, hipStream_t st) {
  if (M <= 0 || N <= 0) return hipSuccess;
  if (rep1 < 1 || rep2 < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(dsse::gate_math_kernel, dim3(dsse::flat_blocks((int64_t)M * N)), dim3(256), 0, st, x, ld, M, N, kind,
                     p1, rep1, p2, rep2, c);
  return hipGetLastError();
}

extern "C" hipError_t dsse_gated_head_norm(const float* o, const float* w, const float* gate, int ldg, void* out, int M,
                                           int H, int V, float eps, int gate_kind, int f32, hipStream_t st) {
  if (M <= 0 || H <= 0) return hipSuccess;
  const int blocks = (int)(((int64_t)M * H + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(dsse::gated_head_norm_kernel<float>, dim3(blocks), dim3(256), 0, st, o, w, gate, ldg,
                       reinterpret_cast<float*>(out), M, H, V, eps, gate_kind);
  else
    hipLaunchKernelGGL(dsse::gated_head_norm_kernel<bf16>, dim3(blocks), dim3(256), 0, st, o, w, gate, ldg,
                       reinterpret_cast<bf16*>(out), M, H, V, eps, gate_kind);
  return hipGetLastError();
}

extern "C" hipError_t dsse_rms_mix(const float* ya, const float* wa, const float* yb, const float* wb, float* out, int M,
                                   int W, float eps, float coef, hipStream_t st) {
  if (M <= 0) return hipSuccess;
  hipLaunchKernelGGL(dsse::rms_mix_kernel, dim3(M), dim3(256), 0, st, ya, wa, yb, wb, out, W, eps, coef);
  return hipGetLastError();
}

extern "C" hipError_t dsse_logit_cap(float* logits, long long n, float scale, float cap, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(dsse::logit_cap_kernel, dim3(dsse::flat_blocks(n)), dim3(256), 0, st, logits, (int64_t)n, scale, cap);
  return hipGetLastError();
}
