// Row-wise fp32 pieces of designs that norm a sublayer's input AND its output, add a hashed embedding of token pairs
// and feed every layer a slice of a per-token table:
//
//   embed_pair_rows  resid = embed[id] + pair[(prev * a + id * b) mod n]  (row n at position 0); the same row once more
//                    in the element type where the projection that opens a loop pass reads it; decode slots store their
//                    token as the next token's predecessor
//   add_norm_rows    resid += y / rms(y) * g_add  (y summed over the experts' slots first), then
//                    out = resid / rms(resid) * g_out (or resid itself): the add of one sublayer and the norm of the next
//                    in one pass over the row, the row held in registers between its two statistics
//   token_gate_rows  out = gelu_tanh(x) * table[id, col0 : col0 + F]
//   token_side_rows  a whole per-layer token input for decode-sized steps in ONE launch: the pending add + norm, the
//                    gate's few dot products per row, the table slice, the back-projection, its norm and add, and the
//                    next sublayer's norm -- five launches of latency-sized kernels otherwise
//
// Everything is computed in fp32; only outputs of the element type are rounded.
#include "api_mixers.h"

namespace dsse {
namespace {

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
__global__ __launch_bounds__(256) void embed_pair_rows_kernel(EmbedPairParams p) {
  const int row = blockIdx.x;
  int id = p.ids[row];
  const int raw_id = id;
  id = (unsigned)id < (unsigned)p.vocab ? id : 0;  // padded / inactive rows carry any id
  const T* e = reinterpret_cast<const T*>(p.embed) + (int64_t)id * p.W;
  const T* b = nullptr;
  if (p.pair) {
    long long pv = p.prev[row];
    pv = pv > 0 ? pv : 0;
    const long long r = p.positions[row] <= 0 ? p.buckets : (pv * p.mul_prev + (long long)id * p.mul_cur) % p.buckets;
    b = reinterpret_cast<const T*>(p.pair) + r * p.W;
  }
  float* resid = p.resid + (int64_t)row * p.W;
  T* x0 = p.x0 ? reinterpret_cast<T*>(p.x0) + (int64_t)row * p.ldx0 : nullptr;
  for (int d = threadIdx.x; d < p.W; d += blockDim.x) {
    float v = (float)e[d];
    if (b) v += (float)b[d];
    resid[d] = v;
    if (x0) x0[d] = (T)v;
  }
  // every thread has read prev[row] (the barrier), then the row's own token replaces it (prev_out may be prev itself)
  __syncthreads();
  if (threadIdx.x == 0 && p.prev_out && row < p.n_prev_out && (!p.keep || p.keep[row] > 0)) p.prev_out[row] = raw_id;
}

constexpr int kNormRegs = 8;  // vectors of VEC floats a thread keeps of its row: rows up to 256 * 8 * VEC floats

template <int VEC>
struct FVec {
  float v[VEC];
};
template <int VEC>
DEV FVec<VEC> ld_f(const float* p) {
  FVec<VEC> r;
  if constexpr (VEC == 4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) r.v[e] = t[e];
  } else {
    r.v[0] = *p;
  }
  return r;
}
template <int VEC>
DEV void st_f(float* p, const FVec<VEC>& r) {
  if constexpr (VEC == 4) *reinterpret_cast<f32x4*>(p) = f32x4{r.v[0], r.v[1], r.v[2], r.v[3]};
  else *p = r.v[0];
}
template <int VEC>
DEV void st_f(bf16* p, const FVec<VEC>& r) {
  if constexpr (VEC == 4) *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)r.v[0], (bf16)r.v[1], (bf16)r.v[2], (bf16)r.v[3]};
  else *p = (bf16)r.v[0];
}

// REG: the row (y summed over its parts, then the new stream) stays in registers between the passes; otherwise it is
// read again from memory (any width).  VEC 4: 16-byte accesses (the width, the strides and every base allow them).
template <typename OutT, int VEC, bool REG>
__global__ __launch_bounds__(256) void add_norm_rows_kernel(AddNormParams p) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int W = p.W;
  float* resid = p.resid + row * W;
  const float* y = p.y ? p.y + row * p.nsum * W : nullptr;
  FVec<VEC> vals[REG ? kNormRegs : 1];
  auto each = [&](auto fn) {  // fn(register slot, first column) for this thread's vectors of the row
    if constexpr (REG) {
#pragma unroll
      for (int i = 0; i < kNormRegs; ++i) {
        const int d = (i * 256 + (int)threadIdx.x) * VEC;
        if (d < W) fn(i, d);
      }
    } else {
      for (int d = (int)threadIdx.x * VEC; d < W; d += 256 * VEC) fn(0, d);
    }
  };
  auto parts = [&](int d) {  // the row's parts of y summed
    FVec<VEC> v = ld_f<VEC>(y + d);
    for (int s = 1; s < p.nsum; ++s) {
      const FVec<VEC> t = ld_f<VEC>(y + (int64_t)s * W + d);
#pragma unroll
      for (int e = 0; e < VEC; ++e) v.v[e] += t.v[e];
    }
    return v;
  };
  float ss = 0.f;
  if (y) {
    float sy = 0.f;
    each([&](int i, int d) {
      const FVec<VEC> v = parts(d);
#pragma unroll
      for (int e = 0; e < VEC; ++e) sy += v.v[e] * v.v[e];
      if (REG) vals[i] = v;
    });
    sy = block_sum256(sy, red);
    const float inv = 1.0f / sqrtf(sy / (float)W + p.eps);
    each([&](int i, int d) {
      const FVec<VEC> v = REG ? vals[i] : parts(d);
      const FVec<VEC> g = ld_f<VEC>(p.g_add + d);
      FVec<VEC> r = ld_f<VEC>(resid + d);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        r.v[e] += v.v[e] * inv * g.v[e];
        ss += r.v[e] * r.v[e];
      }
      st_f<VEC>(resid + d, r);
      if (REG) vals[i] = r;
    });
  } else if (p.out || p.out32) {
    each([&](int i, int d) {
      const FVec<VEC> r = ld_f<VEC>(resid + d);
#pragma unroll
      for (int e = 0; e < VEC; ++e) ss += r.v[e] * r.v[e];
      if (REG) vals[i] = r;
    });
  }
  if (!p.out && !p.out32) return;  // uniform
  float inv = 1.0f;
  if (p.g_out) {
    ss = block_sum256(ss, red);
    inv = 1.0f / sqrtf(ss / (float)W + p.eps);
  }
  OutT* out = p.out ? reinterpret_cast<OutT*>(p.out) + row * p.ldo : nullptr;
  float* out32 = p.out32 ? p.out32 + row * W : nullptr;
  each([&](int i, int d) {
    FVec<VEC> r = REG ? vals[i] : ld_f<VEC>(resid + d);
    if (p.g_out) {
      const FVec<VEC> g = ld_f<VEC>(p.g_out + d);
#pragma unroll
      for (int e = 0; e < VEC; ++e) r.v[e] = r.v[e] * inv * g.v[e];
    }
    if (out) st_f<VEC>(out + d, r);
    if (out32) st_f<VEC>(out32 + d, r);
  });
}

template <typename T>
__global__ __launch_bounds__(256) void token_gate_rows_kernel(const float* x, int ldx, const int* ids, const T* table,
                                                              int vocab, int ldt, int col0, T* out, int M, int F) {
  const int64_t n = (int64_t)M * F;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / F;
    const int c = (int)(i - r * F);
    int id = ids[r];
    id = (unsigned)id < (unsigned)vocab ? id : 0;
    out[i] = (T)(gelu_tanh_f(x[r * ldx + c]) * (float)table[(int64_t)id * ldt + col0 + c]);
  }
}

// One workgroup of sixteen waves per row: a decode step has few rows, so a row's work is spread as wide as one
// workgroup goes.  The row lives in LDS: first the rounded stream (what the gate's projection reads), then the
// back-projection's output.  A wave owns gate columns in groups of four (one pass over the stream row feeds four
// independent sums, so four 16-byte loads are in flight per step); a thread owns every 1024th channel of the
// back-projection (its weight row is F contiguous numbers: independent 16-byte loads).
constexpr int kSideThreads = 1024;

DEV float block_sum_wide(float v, float* red) {  // red holds one number per wave
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
__global__ __launch_bounds__(kSideThreads) void token_side_rows_kernel(TokenSideParams p) {
  extern __shared__ float side_sm[];
  float* xs = side_sm;      // [W]
  float* gs = xs + p.W;     // [F]
  float* red = gs + p.F;    // [16]
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  const int64_t row = blockIdx.x;
  const int W = p.W, F = p.F;
  const int nt = blockDim.x, nw = blockDim.x >> 6;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* resid = p.resid + row * W;
  if (p.y) {
    const float* y = p.y + row * p.nsum * W;
    float sy = 0.f;
    for (int d = threadIdx.x; d < W; d += nt) {
      float v = 0.f;
      for (int s = 0; s < p.nsum; ++s) v += y[(int64_t)s * W + d];
      xs[d] = v;
      sy += v * v;
    }
    sy = block_sum_wide(sy, red);
    const float inv = 1.0f / sqrtf(sy / (float)W + p.eps);
    for (int d = threadIdx.x; d < W; d += nt) {
      const float r = resid[d] + xs[d] * inv * p.g_add[d];
      resid[d] = r;
      xs[d] = (float)(T)r;
    }
  } else {
    for (int d = threadIdx.x; d < W; d += nt) xs[d] = (float)(T)resid[d];
  }
  __syncthreads();
  int id = p.ids[row];
  id = (unsigned)id < (unsigned)p.vocab ? id : 0;
  const T* trow = reinterpret_cast<const T*>(p.table) + (int64_t)id * p.ldt + p.col0;
  const T* gate_w = reinterpret_cast<const T*>(p.gate_w);
  const bool vw = W % VEC == 0;
  for (int j0 = wave * 4; j0 < F; j0 += nw * 4) {
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    const T* gw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) gw[u] = gate_w + (int64_t)(j0 + u < F ? j0 + u : j0) * W;
    if (vw) {
      for (int d = lane * VEC; d < W; d += 64 * VEC) {
        float x[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[e] = xs[d + e];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if constexpr (VEC == 8) {
            const bf16x8 t = *reinterpret_cast<const bf16x8*>(gw[u] + d);
#pragma unroll
            for (int e = 0; e < 8; ++e) s[u] += (float)t[e] * x[e];
          } else {
            const f32x4 t = *reinterpret_cast<const f32x4*>(gw[u] + d);
#pragma unroll
            for (int e = 0; e < 4; ++e) s[u] += t[e] * x[e];
          }
        }
      }
    } else {
      for (int d = lane; d < W; d += 64) {
        const float x = xs[d];
#pragma unroll
        for (int u = 0; u < 4; ++u) s[u] += (float)gw[u][d] * x;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float t = wave_sum(s[u]);
      if (lane == 0 && j0 + u < F) gs[j0 + u] = (float)(T)(gelu_tanh_f(t) * (float)trow[j0 + u]);
    }
  }
  __syncthreads();  // the gate columns are complete, and nobody reads the rounded stream any more
  const T* proj_w = reinterpret_cast<const T*>(p.proj_w);
  const bool vf = F % VEC == 0;
  float sy = 0.f;
  for (int d = threadIdx.x; d < W; d += nt) {
    const T* pw = proj_w + (int64_t)d * F;
    float v = 0.f;
    if (vf) {
#pragma unroll 8
      for (int j = 0; j < F; j += VEC) {
        if constexpr (VEC == 8) {
          const bf16x8 t = *reinterpret_cast<const bf16x8*>(pw + j);
#pragma unroll
          for (int e = 0; e < 8; ++e) v += (float)t[e] * gs[j + e];
        } else {
          const f32x4 t = *reinterpret_cast<const f32x4*>(pw + j);
#pragma unroll
          for (int e = 0; e < 4; ++e) v += t[e] * gs[j + e];
        }
      }
    } else {
      for (int j = 0; j < F; ++j) v += (float)pw[j] * gs[j];
    }
    xs[d] = v;  // this thread's own channel: read back below by the same thread
    sy += v * v;
  }
  sy = block_sum_wide(sy, red);
  const float inv = 1.0f / sqrtf(sy / (float)W + p.eps);
  float ss = 0.f;
  for (int d = threadIdx.x; d < W; d += nt) {
    const float r = resid[d] + xs[d] * inv * p.side_norm[d];
    resid[d] = r;
    xs[d] = r;
    ss += r * r;
  }
  if (!p.out && !p.out32) return;  // uniform
  float inv2 = 1.0f;
  if (p.g_out) {
    ss = block_sum_wide(ss, red);
    inv2 = 1.0f / sqrtf(ss / (float)W + p.eps);
  }
  T* out = p.out ? reinterpret_cast<T*>(p.out) + row * p.ldo : nullptr;
  float* out32 = p.out32 ? p.out32 + row * W : nullptr;
  for (int d = threadIdx.x; d < W; d += nt) {
    float r = xs[d];
    if (p.g_out) r = r * inv2 * p.g_out[d];
    if (out) out[d] = (T)r;
    if (out32) out32[d] = r;
  }
}

template <typename OutT>
void launch_add_norm(const AddNormParams& p, hipStream_t st) {
  const dim3 g(p.M), b(256);
  auto al = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec = p.W % 4 == 0 && p.ldo % 4 == 0 && al(p.y) && al(p.resid) && al(p.g_add) && al(p.g_out) && al(p.out) &&
                   al(p.out32);
  if (vec && p.W <= 256 * kNormRegs * 4) hipLaunchKernelGGL((add_norm_rows_kernel<OutT, 4, true>), g, b, 0, st, p);
  else if (p.W <= 256 * kNormRegs) hipLaunchKernelGGL((add_norm_rows_kernel<OutT, 1, true>), g, b, 0, st, p);
  else hipLaunchKernelGGL((add_norm_rows_kernel<OutT, 1, false>), g, b, 0, st, p);
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_embed_pair_rows(const dsse::EmbedPairParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  if (p->pair && p->buckets < 1) return hipErrorInvalidValue;
  if (p->f32) hipLaunchKernelGGL(dsse::embed_pair_rows_kernel<float>, dim3(p->M), dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::embed_pair_rows_kernel<bf16>, dim3(p->M), dim3(256), 0, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_add_norm_rows(const dsse::AddNormParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  if (p->nsum < 1 || (p->y && !p->g_add)) return hipErrorInvalidValue;
  if (p->out_f32) dsse::launch_add_norm<float>(*p, st);
  else dsse::launch_add_norm<bf16>(*p, st);
  return hipGetLastError();
}

extern "C" hipError_t dsse_token_gate_rows(const float* x, int ldx, const int* ids, const void* table, int vocab, int ldt,
                                           int col0, void* out, int M, int F, int f32, hipStream_t st) {
  if (M <= 0 || F <= 0) return hipSuccess;
  const int64_t nb = ((int64_t)M * F + 255) / 256;
  const int blocks = (int)(nb > 4096 ? 4096 : nb);
  if (f32)
    hipLaunchKernelGGL(dsse::token_gate_rows_kernel<float>, dim3(blocks), dim3(256), 0, st, x, ldx, ids,
                       reinterpret_cast<const float*>(table), vocab, ldt, col0, reinterpret_cast<float*>(out), M, F);
  else
    hipLaunchKernelGGL(dsse::token_gate_rows_kernel<bf16>, dim3(blocks), dim3(256), 0, st, x, ldx, ids,
                       reinterpret_cast<const bf16*>(table), vocab, ldt, col0, reinterpret_cast<bf16*>(out), M, F);
  return hipGetLastError();
}

extern "C" hipError_t dsse_token_side_rows(const dsse::TokenSideParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  const size_t lds = (size_t)(p->W + p->F + 16) * sizeof(float);
  if (p->nsum < 1 || (p->y && !p->g_add) || p->F < 1 || lds > 64 * 1024) return hipErrorInvalidValue;
  const dim3 block(dsse::kSideThreads);
  if (p->f32) hipLaunchKernelGGL(dsse::token_side_rows_kernel<float>, dim3(p->M), block, lds, st, *p);
  else hipLaunchKernelGGL(dsse::token_side_rows_kernel<bf16>, dim3(p->M), block, lds, st, *p);
  return hipGetLastError();
}
