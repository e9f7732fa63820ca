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

// One workgroup per row, the stream count a template parameter (every per-stream array is indexed statically and lives
// in registers).  A thread owns groups of VEC consecutive channels (VEC = 4 when the width allows 16-byte accesses):
// it reads the S old values of each, mixes, writes the S new ones, and keeps u = sum_s in[s] x_s of up to kKeep groups
// in registers for the norm's second sweep; wider rows re-form the rest from the streams it has just written (the same
// thread wrote those addresses).
constexpr int kKeep = 4;

template <int VEC>
struct Pack { float v[VEC]; };

template <int VEC>
DEV Pack<VEC> ld_pack(const float* p) {
  Pack<VEC> r;
  if (VEC == 4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p);
    r.v[0] = t[0], r.v[1] = t[1], r.v[2] = t[2], r.v[3] = t[3];
  } else {
    r.v[0] = p[0];
  }
  return r;
}
template <int VEC>
DEV void st_pack(float* p, const Pack<VEC>& r) {
  if (VEC == 4) *reinterpret_cast<f32x4*>(p) = f32x4{r.v[0], r.v[1], r.v[2], r.v[3]};
  else p[0] = r.v[0];
}
template <int VEC, typename T>
DEV void st_elem(T* p, const Pack<VEC>& r) {
#pragma unroll
  for (int j = 0; j < VEC; ++j) p[j] = (T)r.v[j];
}

template <typename T, typename HT, int S, int VEC>
__global__ __launch_bounds__(256) void stream_mix_kernel(StreamMixParams p) {
  __shared__ float red[4];
  const int row = blockIdx.x, W = p.W;
  float m_mix[S][S], m_in[S], m_out[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    m_in[s] = p.in_w ? p.in_w[s] : 0.0f;
    m_out[s] = p.y ? p.mult * (p.out_w ? p.out_w[s] : 1.0f) : 0.0f;
#pragma unroll
    for (int t = 0; t < S; ++t) m_mix[s][t] = p.mix ? p.mix[s * S + t] : (s == t ? 1.0f : 0.0f);
  }
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
  Pack<VEC> keep[kKeep];
  float ss = 0.f;
  int it = 0;
  for (int d = threadIdx.x * VEC; d < W; d += 256 * VEC, ++it) {
    Pack<VEC> xs[S], xn[S];
    if (e) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float v = (float)e[d + j] * p.embed_scale;
#pragma unroll
        for (int s = 0; s < S; ++s) xs[s].v[j] = v;
      }
    } else {
#pragma unroll
      for (int s = 0; s < S; ++s) xs[s] = ld_pack<VEC>(x + (int64_t)s * W + d);
    }
    if (y) {
      Pack<VEC> yv = ld_pack<VEC>(y + d);
      for (int k = 1; k < p.nsum; ++k) {
        const Pack<VEC> t = ld_pack<VEC>(y + (int64_t)k * W + d);
#pragma unroll
        for (int j = 0; j < VEC; ++j) yv.v[j] += t.v[j];
      }
#pragma unroll
      for (int t = 0; t < S; ++t)
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          float v = m_out[t] * yv.v[j];
#pragma unroll
          for (int s = 0; s < S; ++s) v += m_mix[s][t] * xs[s].v[j];
          xn[t].v[j] = v;
        }
    } else {
#pragma unroll
      for (int s = 0; s < S; ++s) xn[s] = xs[s];
    }
    Pack<VEC> u, sum;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float uu = 0.f, sm = 0.f;
#pragma unroll
      for (int s = 0; s < S; ++s) uu += m_in[s] * xn[s].v[j], sm += xn[s].v[j];
      u.v[j] = uu, sum.v[j] = sm;
      ss += uu * uu;
    }
    if (rewrite)
#pragma unroll
      for (int s = 0; s < S; ++s) st_pack<VEC>(x + (int64_t)s * W + d, xn[s]);
    if (tot) st_pack<VEC>(tot + d, sum);
#pragma unroll
    for (int k = 0; k < kKeep; ++k)
      if (k == it) keep[k] = u;
  }
  if (!p.h) return;  // uniform
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + p.eps);
  HT* h = reinterpret_cast<HT*>(p.h) + (int64_t)row * W;
  it = 0;
  for (int d = threadIdx.x * VEC; d < W; d += 256 * VEC, ++it) {
    Pack<VEC> u;
    if (it < kKeep) {
#pragma unroll
      for (int k = 0; k < kKeep; ++k)
        if (k == it) u = keep[k];
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) u.v[j] = 0.f;
#pragma unroll
      for (int s = 0; s < S; ++s) {
        const Pack<VEC> t = ld_pack<VEC>(x + (int64_t)s * W + d);
#pragma unroll
        for (int j = 0; j < VEC; ++j) u.v[j] += m_in[s] * t.v[j];
      }
    }
    const Pack<VEC> g = ld_pack<VEC>(p.norm_w + d);
#pragma unroll
    for (int j = 0; j < VEC; ++j) u.v[j] *= inv * g.v[j];
    st_elem<VEC, HT>(h + d, u);
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

// One wave per row, E <= kMaxRouteExperts.  Choice scores sit in LDS; lanes own groups for the group scores and
// ranks, and every pick is a wave-wide argmax (ties go to the lower index, as in the reference).
constexpr int kMaxRouteExperts = 256;

__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ z, const float* __restrict__ corr, int M,
                                                       int E, int top, int groups, int keep, float scale, int kind,
                                                       int* topk_idx, float* topk_w) {
  __shared__ float choice[kMaxRouteExperts], score[kMaxRouteExperts], gs[kMaxRouteExperts];
  const int row = blockIdx.x, lane = threadIdx.x;
  const float* zr = z + (int64_t)row * E;
  const float ninf = -__builtin_inff();
  float zmax = ninf, zsum = 0.f;
  if (kind == 1) {  // softmax over all experts: the row's maximum and the sum of exponentials, wave-wide
    for (int e = lane; e < E; e += 64) {
      const float v = zr[e];
      zmax = fmaxf(zmax, v == v ? v : 0.0f);
    }
    zmax = wave_max(zmax);
    for (int e = lane; e < E; e += 64) {
      const float v = zr[e];
      zsum += expf((v == v ? v : 0.0f) - zmax);
    }
    zsum = wave_sum(zsum);
  }
  for (int e = lane; e < E; e += 64) {
    float v = zr[e];
    v = v == v ? v : 0.0f;
    const float sg = kind == 1 ? expf(v - zmax) / zsum : 1.0f / (1.0f + expf(-v));
    score[e] = sg;
    choice[e] = corr ? sg + corr[e] : sg;
  }
  __syncthreads();
  if (groups > 1) {
    const int per = E / groups;
    for (int o = lane; o < groups; o += 64) {  // a group's score: the sum of its two largest choice scores (kind 1: the largest)
      float a = ninf, b = ninf;
      for (int j = 0; j < per; ++j) {
        const float c = choice[o * per + j];
        if (c > a) b = a, a = c;
        else if (c > b) b = c;
      }
      gs[o] = per > 1 && kind == 0 ? a + b : a;
    }
    __syncthreads();
    // rank of a group = groups with a larger score (or the same score and a lower index); eligible when rank < keep
    for (int g = lane; g < groups; g += 64) {
      int rank = 0;
      for (int o = 0; o < groups; ++o) rank += o != g && (gs[o] > gs[g] || (gs[o] == gs[g] && o < g));
      if (rank >= keep)
        for (int j = 0; j < per; ++j) choice[g * per + j] = ninf;
    }
    __syncthreads();
  }
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = ninf;
    int best = E;  // "none yet": any real index wins a tie against it
    for (int e = lane; e < E; e += 64) {
      const float c = choice[e];
      if (c != c) continue;  // a NaN never ranks
      if (best == E || c > bv) best = e, bv = c;  // ascending e: the lower index keeps a tie
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(bv, o);
      const int oi = __shfl_xor(best, o);
      if (oi < E && (best == E || ov > bv || (ov == bv && oi < best))) bv = ov, best = oi;
    }
    best = best < E ? best : 0;
    const float sg = score[best];
    sum += sg;
    __syncthreads();  // every lane has read choice[] for this pick
    if (lane == 0) {
      choice[best] = __builtin_nanf("");  // taken: out of every later pick
      topk_idx[(int64_t)row * top + k] = best;
      topk_w[(int64_t)row * top + k] = sg;
    }
    __syncthreads();
  }
  const float inv = kind == 1 ? scale : scale / (sum + 1e-20f);
  __syncthreads();
  for (int k = lane; k < top; k += 64) topk_w[(int64_t)row * top + k] *= inv;
}

inline int flat_blocks(int64_t n) {
  const int64_t b = (n + 255) / 256;
  return (int)(b < 1 ? 1 : (b > 4096 ? 4096 : b));
}

}  // namespace
}  // namespace dsse

namespace dsse {
namespace {
template <typename T, typename HT, int VEC>
void launch_stream_mix(const StreamMixParams& p, hipStream_t st) {
  const dim3 g(p.M), b(256);
  switch (p.S) {
    case 1: hipLaunchKernelGGL((stream_mix_kernel<T, HT, 1, VEC>), g, b, 0, st, p); break;
    case 2: hipLaunchKernelGGL((stream_mix_kernel<T, HT, 2, VEC>), g, b, 0, st, p); break;
    case 3: hipLaunchKernelGGL((stream_mix_kernel<T, HT, 3, VEC>), g, b, 0, st, p); break;
    case 4: hipLaunchKernelGGL((stream_mix_kernel<T, HT, 4, VEC>), g, b, 0, st, p); break;
    case 5: hipLaunchKernelGGL((stream_mix_kernel<T, HT, 5, VEC>), g, b, 0, st, p); break;
    case 6: hipLaunchKernelGGL((stream_mix_kernel<T, HT, 6, VEC>), g, b, 0, st, p); break;
    case 7: hipLaunchKernelGGL((stream_mix_kernel<T, HT, 7, VEC>), g, b, 0, st, p); break;
    default: hipLaunchKernelGGL((stream_mix_kernel<T, HT, 8, VEC>), g, b, 0, st, p); break;
  }
}
template <int VEC>
void launch_stream_mix_types(const StreamMixParams& p, hipStream_t st) {
  if (p.f32) launch_stream_mix<float, float, VEC>(p, st);
  else if (p.h_f32) launch_stream_mix<bf16, float, VEC>(p, st);
  else launch_stream_mix<bf16, bf16, VEC>(p, st);
}
}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_stream_mix(const dsse::StreamMixParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  if (p->S < 1 || p->S > dsse::kMaxStreams || p->nsum < 1) return hipErrorInvalidValue;
  // 16-byte accesses need every row of every operand on a 16-byte boundary: the width and the row stride multiples
  // of four floats and the bases aligned (torch allocations are; column slices may not be)
  auto al = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec = p->W % 4 == 0 && p->ld % 4 == 0 && al(p->streams) && al(p->y) && al(p->total) && al(p->norm_w) &&
                   (p->h_f32 || p->f32 ? al(p->h) : true);
  if (vec) dsse::launch_stream_mix_types<4>(*p, st);
  else dsse::launch_stream_mix_types<1>(*p, st);
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
                                     float scale, int kind, int* topk_idx, float* topk_w, hipStream_t st) {
  if (M <= 0) return hipSuccess;
  if (E > dsse::kMaxRouteExperts || groups < 1 || E % groups || top > E) return hipErrorInvalidValue;
  if ((kind != 0 && kind != 1) || (kind == 0 && !corr)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(dsse::moe_route_kernel, dim3(M), dim3(64), 0, st, z, corr, M, E, top, groups, keep, scale, kind,
                     topk_idx, topk_w);
  return hipGetLastError();
}
