// Row-wise fp32 pieces of pre-norm designs that carry several residual streams and route squared-ReLU experts:
//
//   stream_mix   one pass over the S residual copies of a row between two sublayers: (first step) every stream =
//                embed[id] * scale; (a sublayer is finished) x_t = sum_s mix[s][t] x_s + mult * out[t] * y for all
//                streams at once from the old ones, y summed over its nsum parts first (the routed experts' slots);
//                (a sublayer follows) u = sum_s in[s] x_s, h = u / rms(u) * gain; (a trace or the head follows) the sum
//                of the streams.  The write-back of one sublayer, the read of the next and its norm are ONE kernel, and
//                a row's streams leave and enter memory once.
//   act_rows     out = act(x) * sigmoid(gate): identity, xIELU (a_p z^2 + z/2 | a_n (e^z - 1 - z) + z/2) or relu^2,
//                with an optional sigmoid gate from a column range of another fp32 buffer
//   moe_route    sigmoid scores + per-expert correction -> group-limited top-k (groups ranked by the sum of their two
//                best choice scores) -> weights = chosen scores / their sum * scale
//
// Everything is computed in fp32; only h / out of the element type are rounded.
#include "api_mixers.h"

namespace dsse {
namespace {

constexpr int kMaxStreams = 8;

DEV float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < nw; ++i) s += red[i];
  return s;
}

// One workgroup per row.  The mixed streams go back to memory in the first sweep; the norm's second sweep re-forms u
// from them (the row's S * W floats are still in the nearest cache), so no width limit comes from LDS or registers.
template <typename T, typename HT>
__global__ __launch_bounds__(256) void stream_mix_kernel(StreamMixParams p) {
  __shared__ float red[4];
  __shared__ float s_mix[kMaxStreams * kMaxStreams], s_in[kMaxStreams], s_out[kMaxStreams];
  const int row = blockIdx.x, S = p.S, W = p.W;
  for (int i = threadIdx.x; i < S * S; i += blockDim.x) s_mix[i] = p.mix ? p.mix[i] : (i / S == i % S ? 1.0f : 0.0f);
  for (int i = threadIdx.x; i < S; i += blockDim.x) {
    s_in[i] = p.in_w ? p.in_w[i] : 0.0f;
    s_out[i] = p.y ? p.mult * (p.out_w ? p.out_w[i] : 1.0f) : 0.0f;
  }
  __syncthreads();
  float* x = p.streams + (int64_t)row * p.ld;
  const T* e = nullptr;
  if (p.embed) {
    int id = p.ids[row];
    id = (unsigned)id < (unsigned)p.vocab ? id : 0;  // padded / inactive rows carry any id
    e = reinterpret_cast<const T*>(p.embed) + (int64_t)id * W;
  }
  const float* y = p.y ? p.y + (int64_t)row * p.nsum * W : nullptr;
  float* tot = p.total ? p.total + (int64_t)row * W : nullptr;
  const bool rewrite = e || y;
  float ss = 0.f;
  for (int d = threadIdx.x; d < W; d += blockDim.x) {
    float xs[kMaxStreams], xn[kMaxStreams];
    if (e) {
      const float v = (float)e[d] * p.embed_scale;
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s) xs[s] = v;
    } else {
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s) xs[s] = s < S ? x[(int64_t)s * W + d] : 0.0f;
    }
    if (y) {
      float yv = 0.f;
      for (int k = 0; k < p.nsum; ++k) yv += y[(int64_t)k * W + d];
#pragma unroll
      for (int t = 0; t < kMaxStreams; ++t) {
        if (t >= S) break;
        float v = s_out[t] * yv;
#pragma unroll
        for (int s = 0; s < kMaxStreams; ++s)
          if (s < S) v += s_mix[s * S + t] * xs[s];
        xn[t] = v;
      }
    } else {
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s) xn[s] = xs[s];
    }
    float u = 0.f, sum = 0.f;
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s) {
      if (s >= S) break;
      if (rewrite) x[(int64_t)s * W + d] = xn[s];
      u += s_in[s] * xn[s];
      sum += xn[s];
    }
    ss += u * u;
    if (tot) tot[d] = sum;
  }
  if (!p.h) return;  // uniform
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + p.eps);
  HT* h = reinterpret_cast<HT*>(p.h) + (int64_t)row * W;
  for (int d = threadIdx.x; d < W; d += blockDim.x) {  // the same thread wrote these addresses in the first sweep
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s)
      if (s < S) u += s_in[s] * x[(int64_t)s * W + d];
    h[d] = (HT)(u * inv * p.norm_w[d]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void act_rows_kernel(const float* x, int ldx, T* out, int M, int F, int kind,
                                                       const float* params, const float* gate, int ldg) {
  const int64_t n = (int64_t)M * F;
  const float ap = kind == 1 ? params[0] : 0.0f, an = kind == 1 ? params[1] : 0.0f;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / F;
    const int c = (int)(i - r * F);
    float z = x[r * ldx + c];
    if (kind == 1) {
      z = z > 0.0f ? ap * z * z + 0.5f * z : an * (expm1f(z) - z) + 0.5f * z;
    } else if (kind == 2) {
      z = z > 0.0f ? z * z : 0.0f;
    }
    if (gate) z *= 1.0f / (1.0f + expf(-gate[r * ldg + c]));
    out[i] = (T)z;
  }
}

// One thread per row; E <= kMaxRouteExperts choice scores live in the thread's scratch.  Ties go to the lower index.
constexpr int kMaxRouteExperts = 256;

__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ z, const float* __restrict__ corr, int M,
                                                       int E, int top, int groups, int keep, float scale, int* topk_idx,
                                                       float* topk_w) {
  const int row = blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= M) return;
  const float* zr = z + (int64_t)row * E;
  int* idx = topk_idx + (int64_t)row * top;
  float* wt = topk_w + (int64_t)row * top;
  float choice[kMaxRouteExperts];
  const float ninf = -__builtin_inff();
  for (int e = 0; e < E; ++e) {
    float v = zr[e];
    v = v == v ? v : 0.0f;
    choice[e] = 1.0f / (1.0f + expf(-v)) + corr[e];
  }
  if (groups > 1) {
    const int per = E / groups;
    float gs[kMaxRouteExperts];  // a group's score: the sum of its two largest choice scores
    for (int o = 0; o < groups; ++o) {
      float a = ninf, b = ninf;
      for (int j = 0; j < per; ++j) {
        const float c = choice[o * per + j];
        if (c > a) b = a, a = c;
        else if (c > b) b = c;
      }
      gs[o] = per > 1 ? a + b : a;
    }
    // rank of a group = groups with a larger score (or the same score and a lower index); eligible when rank < keep
    for (int g = 0; g < groups; ++g) {
      int rank = 0;
      for (int o = 0; o < groups; ++o) rank += o != g && (gs[o] > gs[g] || (gs[o] == gs[g] && o < g));
      if (rank >= keep)
        for (int j = 0; j < per; ++j) choice[g * per + j] = ninf;
    }
  }
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bv = ninf;
    for (int e = 0; e < E; ++e) {
      bool used = false;
      for (int j = 0; j < k; ++j) used |= idx[j] == e;
      if (used) continue;
      if (best < 0 || choice[e] > bv) best = e, bv = choice[e];
    }
    best = best < 0 ? 0 : best;
    idx[k] = best;
    float v = zr[best];
    v = v == v ? v : 0.0f;
    const float s = 1.0f / (1.0f + expf(-v));
    wt[k] = s;
    sum += s;
  }
  const float inv = scale / (sum + 1e-20f);
  for (int k = 0; k < top; ++k) wt[k] *= inv;
}

inline int flat_blocks(int64_t n) {
  const int64_t b = (n + 255) / 256;
  return (int)(b < 1 ? 1 : (b > 4096 ? 4096 : b));
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_stream_mix(const dsse::StreamMixParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  if (p->S < 1 || p->S > dsse::kMaxStreams || p->nsum < 1) return hipErrorInvalidValue;
  const dim3 g(p->M), b(256);
  if (p->f32) {
    hipLaunchKernelGGL((dsse::stream_mix_kernel<float, float>), g, b, 0, st, *p);
  } else if (p->h_f32) {
    hipLaunchKernelGGL((dsse::stream_mix_kernel<bf16, float>), g, b, 0, st, *p);
  } else {
    hipLaunchKernelGGL((dsse::stream_mix_kernel<bf16, bf16>), g, b, 0, st, *p);
  }
  return hipGetLastError();
}

extern "C" hipError_t dsse_act_rows(const float* x, int ldx, void* out, int M, int F, int kind, const float* params,
                                    const float* gate, int ldg, int f32, hipStream_t st) {
  if (M <= 0 || F <= 0) return hipSuccess;
  if (kind == 1 && !params) return hipErrorInvalidValue;
  const int blocks = dsse::flat_blocks((int64_t)M * F);
  if (f32)
    hipLaunchKernelGGL(dsse::act_rows_kernel<float>, dim3(blocks), dim3(256), 0, st, x, ldx, reinterpret_cast<float*>(out),
                       M, F, kind, params, gate, ldg);
  else
    hipLaunchKernelGGL(dsse::act_rows_kernel<bf16>, dim3(blocks), dim3(256), 0, st, x, ldx, reinterpret_cast<bf16*>(out),
                       M, F, kind, params, gate, ldg);
  return hipGetLastError();
}

extern "C" hipError_t dsse_moe_route(const float* z, const float* corr, int M, int E, int top, int groups, int keep,
                                     float scale, int* topk_idx, float* topk_w, hipStream_t st) {
  if (M <= 0) return hipSuccess;
  if (E > dsse::kMaxRouteExperts || groups < 1 || E % groups || top > E) return hipErrorInvalidValue;
  hipLaunchKernelGGL(dsse::moe_route_kernel, dim3((M + 63) / 64), dim3(64), 0, st, z, corr, M, E, top, groups, keep, scale,
                     topk_idx, topk_w);
  return hipGetLastError();
}
