// General row-major GEMM on MFMA: out[M, N] = act(X[M, K] . W[N, K]^T + bias), any M, N, K, batched over blockIdx.z.
//
// The engine's tiled-layout GEMMs (gemm_skinny / gemm_stream / gemm_wide / gemm_tiled / gemm_pipe) want N % 16 == 0 and
// K % 128 == 0 and a pre-tiled weight.  Layer designs whose inner sizes come from a checkpoint's configuration (expert
// widths, latent ranks, per-head slices, block-diagonal gates) need a kernel with no shape contract: this one reads both
// operands straight from global memory as MFMA fragments (K is the contiguous axis of X and of W, so a lane's fragment is
// one 16-byte load), zero-fills past M, N and K, and strides over a batch axis (per-head or per-block weights).
//
// Two element types: bf16 (v_mfma_f32_16x16x32_bf16) and fp32 (v_mfma_f32_16x16x4_f32, true 32-bit products) -- the
// latter is the engine's exact mode.  A lane (r = lane & 15, g = lane >> 4) holds PER consecutive k of row r; which k a
// (lane group, element) pair stands for only has to agree between the A and the B fragment, so both use k0 + PER g + j.
#include "api_layers.h"
#include "frag.h"

namespace dsse {
namespace {

// TM x TN 16x16 tiles per wave, WGM x WGN waves per workgroup (4 waves).
template <typename T, int TM, int TN, int WGM, int WGN>
__global__ __launch_bounds__(256) void gemm_rm_kernel(GemmRmParams p) {
  using F = Frag<T>;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int wm = wave / WGN, wn = wave % WGN;
  const int row0 = blockIdx.y * (WGM * TM * 16) + wm * TM * 16;
  const int col0 = blockIdx.x * (WGN * TN * 16) + wn * TN * 16;
  const int z = blockIdx.z;
  const T* X = reinterpret_cast<const T*>(p.x) + (int64_t)z * p.xbs;
  const T* W = reinterpret_cast<const T*>(p.w) + (int64_t)z * p.wbs;
  const T* bias = p.bias ? reinterpret_cast<const T*>(p.bias) + (int64_t)z * p.bbs : nullptr;
  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const T* xr[TM];
  const T* wr[TN];
  bool xv[TM], wv[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = row0 + 16 * i + r;
    xv[i] = row < p.M;
    xr[i] = X + (int64_t)(xv[i] ? row : 0) * p.ldx;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = col0 + 16 * j + r;
    wv[j] = col < p.N;
    wr[j] = W + (int64_t)(wv[j] ? col : 0) * p.ldw;
  }
  const bool vx = p.vecx != 0, vw = p.vecw != 0;
  for (int k0 = 0; k0 < p.K; k0 += F::KS) {
    const int k = k0 + F::PER * g;
    typename F::V a[TM], b[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) a[i] = load_frag<T>(xr[i], k, p.K, xv[i], vx);
#pragma unroll
    for (int j = 0; j < TN; ++j) b[j] = load_frag<T>(wr[j], k, p.K, wv[j], vw);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = mma(a[i], b[j], acc[i][j]);
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = col0 + 16 * j + r;
      if (col >= p.N) continue;
      const float bv = bias ? (float)bias[col] : 0.0f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int row = row0 + 16 * i + 4 * g + e;
        if (row >= p.M) continue;
        float v = acc[i][j][e] + bv;
        if (p.act == 1) v = gelu_tanh(v);
        const int64_t o = (int64_t)z * p.obs + (int64_t)row * p.ldo + col;
        if (p.out_f32) reinterpret_cast<float*>(p.out)[o] = v;
        else reinterpret_cast<T*>(p.out)[o] = (T)v;
      }
    }
}

// Up to 16 rows (decode buckets, per-head and per-block slices), or many rows of a NARROW output (a router's logits, a
// few-column gate: up to 64 columns): a workgroup owns one 16 x 16 output tile and its four waves split the K axis
// (k-steps w, w + 4, ...), meeting in LDS.  Four times the workgroups of a 16 x 64 tile and a quarter of the dependent
// k-steps per wave: these launches are latency-bound, not bandwidth-bound -- a narrow output leaves the 64 x 64 tiles
// of the general kernel a handful of workgroups that each walk the whole K axis.
// NW waves per workgroup: four, or sixteen when the launch has few tiles and a long K axis (a router's logits for a
// decode step are ONE tile: sixteen waves walk a sixteenth of K each instead of four a quarter).
template <typename T, int NW>
__global__ __launch_bounds__(NW * 64) void gemm_rm_skinny_kernel(GemmRmParams p) {
  using F = Frag<T>;
  __shared__ float red[NW * 4 * 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int col0 = blockIdx.x * 16, row0 = blockIdx.y * 16;
  const int z = blockIdx.z;
  const T* X = reinterpret_cast<const T*>(p.x) + (int64_t)z * p.xbs;
  const T* W = reinterpret_cast<const T*>(p.w) + (int64_t)z * p.wbs;
  const T* bias = p.bias ? reinterpret_cast<const T*>(p.bias) + (int64_t)z * p.bbs : nullptr;
  const bool xv = row0 + r < p.M, wv = col0 + r < p.N;
  const T* xr = X + (int64_t)(xv ? row0 + r : 0) * p.ldx;
  const T* wr = W + (int64_t)(wv ? col0 + r : 0) * p.ldw;
  const bool vx = p.vecx != 0, vw = p.vecw != 0;
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = wave * F::KS; k0 < p.K; k0 += NW * F::KS) {
    const int k = k0 + F::PER * g;
    acc = mma(load_frag<T>(xr, k, p.K, xv, vx), load_frag<T>(wr, k, p.K, wv, vw), acc);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) red[(wave * 4 + e) * 64 + lane] = acc[e];
  __syncthreads();
  if (wave != 0) return;
  const int col = col0 + r;
  if (col >= p.N) return;
  const float bv = bias ? (float)bias[col] : 0.0f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int row = row0 + 4 * g + e;
    if (row >= p.M) continue;
    float v = bv;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += red[(4 * w + e) * 64 + lane];
    if (p.act == 1) v = gelu_tanh(v);
    const int64_t o = (int64_t)z * p.obs + (int64_t)row * p.ldo + col;
    if (p.out_f32) reinterpret_cast<float*>(p.out)[o] = v;
    else reinterpret_cast<T*>(p.out)[o] = (T)v;
  }
}

template <typename T, int TM, int TN, int WGM, int WGN>
hipError_t launch(const GemmRmParams& p, hipStream_t st) {
  dim3 grid((p.N + WGN * TN * 16 - 1) / (WGN * TN * 16), (p.M + WGM * TM * 16 - 1) / (WGM * TM * 16), p.batch);
  hipLaunchKernelGGL((gemm_rm_kernel<T, TM, TN, WGM, WGN>), grid, dim3(256), 0, st, p);
  return hipGetLastError();
}

template <typename T>
hipError_t dispatch(const GemmRmParams& p, hipStream_t st) {
  if (p.M <= 16 || (p.N <= 64 && p.K >= 256)) {
    const dim3 grid((p.N + 15) / 16, (p.M + 15) / 16, p.batch);
    if ((int64_t)grid.x * grid.y * grid.z <= 256 && p.K >= 64 * Frag<T>::KS)
      hipLaunchKernelGGL((gemm_rm_skinny_kernel<T, 16>), grid, dim3(1024), 0, st, p);
    else
      hipLaunchKernelGGL((gemm_rm_skinny_kernel<T, 4>), grid, dim3(256), 0, st, p);
    return hipGetLastError();
  }
  if (p.M >= 256 && p.N >= 256) return launch<T, 4, 4, 2, 2>(p, st);
  return launch<T, 2, 2, 2, 2>(p, st);
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_gemm_rm(const dsse::GemmRmParams* p, hipStream_t st) {
  if (p->M <= 0 || p->N <= 0 || p->batch <= 0) return hipSuccess;
  return p->f32 ? dsse::dispatch<float>(*p, st) : dsse::dispatch<bf16>(*p, st);
}
