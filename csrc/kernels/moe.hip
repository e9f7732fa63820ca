// Routed mixture of experts: router (fp32 logits, the k largest, a softmax among those k) and the token-major
// expert feed-forward (each row walks its chosen experts and the always-on shared expert).
//
//   moe_router   one wave per row: logits z[e] = w[e] . x + b[e] in fp32 (lanes split the width, wave reduction), then
//                the `top` largest (lowest index first among equals) and their softmax.
//   moe_ffn      one workgroup per row: x in LDS; per expert, a wave per hidden unit computes silu(gate . x) * (up . x)
//                into LDS, then a wave per output coordinate adds weight * (down . hidden).  The row's result leaves as
//                fp32 (the residual norm follows).  Each expert's weights are read once per row that chose it: the
//                decode-shaped path (few rows per expert), and correct for any row count.
#include "api_layers.h"
#include "frag.h"

namespace dsse {
namespace {

template <typename T>
__global__ __launch_bounds__(64) void moe_router_kernel(MoeRouterParams p) {
  extern __shared__ float z[];  // [E]
  const int row = blockIdx.x, lane = threadIdx.x;
  const T* x = reinterpret_cast<const T*>(p.x) + (int64_t)row * p.W;
  const T* w = reinterpret_cast<const T*>(p.w);
  for (int e = 0; e < p.E; ++e) {
    float s = 0.f;
    for (int d = lane; d < p.W; d += 64) s += (float)w[(int64_t)e * p.W + d] * (float)x[d];
    s = wave_sum(s);
    if (lane == 0) z[e] = s + (p.b ? (float)reinterpret_cast<const T*>(p.b)[e] : 0.0f);
  }
  __syncthreads();
  if (lane == 0) {
    int* idx = p.topk_idx + (int64_t)row * p.top;
    float* wt = p.topk_w + (int64_t)row * p.top;
    float mx = 0.f;
    for (int k = 0; k < p.top; ++k) {
      int best = -1;
      float bv = 0.f;
      for (int e = 0; e < p.E; ++e) {
        bool used = false;
        for (int j = 0; j < k; ++j) used |= idx[j] == e;
        if (used) continue;
        if (best < 0 || z[e] > bv) best = e, bv = z[e];  // a NaN logit (an inactive row's garbage) still picks e
      }
      idx[k] = best < 0 ? 0 : best;
      wt[k] = bv;
      if (k == 0) mx = bv;
    }
    float sum = 0.f;
    for (int k = 0; k < p.top; ++k) {
      wt[k] = expf(wt[k] - mx);
      sum += wt[k];
    }
    for (int k = 0; k < p.top; ++k) wt[k] /= sum;
  }
}

// The choice alone, from fp32 logits [M, E] (the router's GEMM, bias added): one thread per row.
__global__ __launch_bounds__(256) void moe_topk_kernel(const float* __restrict__ z, int M, int E, int top, int* topk_idx,
                                                       float* topk_w) {
  const int row = blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= M) return;
  const float* zr = z + (int64_t)row * E;
  int* idx = topk_idx + (int64_t)row * top;
  float* wt = topk_w + (int64_t)row * top;
  float mx = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bv = 0.f;
    for (int e = 0; e < E; ++e) {
      bool used = false;
      for (int j = 0; j < k; ++j) used |= idx[j] == e;
      if (used) continue;
      const float v = zr[e];
      if (best < 0 || v > bv) best = e, bv = v;
    }
    idx[k] = best < 0 ? 0 : best;
    wt[k] = bv;
    if (k == 0) mx = bv;
  }
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    wt[k] = expf(wt[k] - mx);
    sum += wt[k];
  }
  for (int k = 0; k < top; ++k) wt[k] /= sum;
}

template <typename T>
DEV void expert_row(const T* gate, const T* up, const T* down, int W, int F, float wgt, const float* xs, float* hs,
                    float* acc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int f = wave; f < F; f += nw) {
    float g = 0.f, u = 0.f;
    const T* gr = gate + (int64_t)f * W;
    const T* ur = up + (int64_t)f * W;
    for (int d = lane; d < W; d += 64) {
      const float xv = xs[d];
      g += (float)gr[d] * xv;
      u += (float)ur[d] * xv;
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0) hs[f] = g / (1.0f + expf(-g)) * u;
  }
  __syncthreads();
  for (int d = wave; d < W; d += nw) {
    float s = 0.f;
    const T* dr = down + (int64_t)d * F;
    for (int f = lane; f < F; f += 64) s += (float)dr[f] * hs[f];
    s = wave_sum(s);
    if (lane == 0) acc[d] += wgt * s;
  }
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(256) void moe_ffn_kernel(MoeFfnParams p) {
  extern __shared__ float smem[];
  float* xs = smem;            // [W]
  float* acc = smem + p.W;     // [W]
  float* hs = acc + p.W;       // [max(F, Fs)]
  const int row = blockIdx.x;
  const T* x = reinterpret_cast<const T*>(p.x) + (int64_t)row * p.W;
  for (int d = threadIdx.x; d < p.W; d += blockDim.x) {
    xs[d] = (float)x[d];
    acc[d] = 0.f;
  }
  __syncthreads();
  for (int k = 0; k < p.top; ++k) {
    int e = p.topk_idx[(int64_t)row * p.top + k];
    e = (unsigned)e < (unsigned)p.E ? e : 0;
    const float wgt = p.topk_w[(int64_t)row * p.top + k];
    expert_row<T>(reinterpret_cast<const T*>(p.gate) + (int64_t)e * p.F * p.W,
                  reinterpret_cast<const T*>(p.up) + (int64_t)e * p.F * p.W,
                  reinterpret_cast<const T*>(p.down) + (int64_t)e * p.W * p.F, p.W, p.F, wgt, xs, hs, acc);
  }
  if (p.sgate)
    expert_row<T>(reinterpret_cast<const T*>(p.sgate), reinterpret_cast<const T*>(p.sup),
                  reinterpret_cast<const T*>(p.sdown), p.W, p.Fs, 1.0f, xs, hs, acc);
  for (int d = threadIdx.x; d < p.W; d += blockDim.x) p.out[(int64_t)row * p.W + d] = acc[d];
}


// ---------------------------------------------------------------------------------------------------------------------
// Grouped form: rows sorted by expert, MFMA tiles of 16 rows of ONE expert.  An "id" is a (row, slot) pair,
// id = row * S + k with S = top (+ 1 when the design has a shared expert: slot `top` is the shared expert, weight 1,
// expert index E with its own hidden width).  Each expert's weights are read once per 64 of its rows (four 16-row MFMA tiles; empty ones are skipped), so the same two
// GEMM launches serve a decode step (a few rows per expert) and a prompt portion (hundreds).
//
//   moe_align     one workgroup: per-expert counts -> tile-padded offsets -> sorted ids (pads -1), the expert of every
//                 tile and the tile count.  The order of ids inside an expert is whatever the atomics give; a row's
//                 result does not depend on its place in a tile.
//   moe_gate_up   h[id, f] = silu(gate_e[f] . x[row]) * (up_e[f] . x[row])       (element type)
//   moe_down      o[id, :] = weight(id) * down_e . h[id]                          (fp32)
// The residual norm that follows sums a row's S slots (scalar_norm nsum).

constexpr int kMoeRows = 64;  // rows of one expert per workgroup tile: four 16-row MFMA tiles share every weight fragment

__global__ __launch_bounds__(256) void moe_align_kernel(MoeGroupedParams p) {
  extern __shared__ int sm[];
  const int NE = p.E + (p.S > p.top ? 1 : 0);
  int* cnt = sm;            // [NE]
  int* off = sm + NE;       // [NE + 1] first sorted position of each expert (multiples of kMoeRows)
  int* fill = off + NE + 1; // [NE]
  const int n = p.M * p.S;
  for (int e = threadIdx.x; e < NE; e += blockDim.x) cnt[e] = 0, fill[e] = 0;
  __syncthreads();
  for (int id = threadIdx.x; id < n; id += blockDim.x) {
    const int row = id / p.S, k = id % p.S;
    int e = k < p.top ? p.topk_idx[row * p.top + k] : p.E;
    e = (unsigned)e < (unsigned)NE ? e : 0;
    atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < NE; ++e) {
      off[e] = at;
      at += (cnt[e] + kMoeRows - 1) / kMoeRows * kMoeRows;
    }
    off[NE] = at;
    *p.num_tiles = at / kMoeRows;
  }
  __syncthreads();
  const int total = off[NE];
  for (int i = threadIdx.x; i < total; i += blockDim.x) p.sorted[i] = -1;
  for (int e = threadIdx.x; e < NE; e += blockDim.x)
    for (int t = off[e] / kMoeRows; t < off[e + 1] / kMoeRows; ++t) p.tile_expert[t] = e;
  __syncthreads();
  for (int id = threadIdx.x; id < n; id += blockDim.x) {
    const int row = id / p.S, k = id % p.S;
    int e = k < p.top ? p.topk_idx[row * p.top + k] : p.E;
    e = (unsigned)e < (unsigned)NE ? e : 0;
    p.sorted[off[e] + atomicAdd(&fill[e], 1)] = id;
  }
}

// Both expert GEMMs: a workgroup owns 16 output columns of one 64-row tile; its four waves split the K axis (k-steps
// w, w + 4, ...) and meet in LDS, where wave i finishes the tile's i-th 16-row sub-tile.  Sixteen columns per workgroup
// give a decode step (17 tiles or so) thousands of workgroups to hide the weight stream's latency with.
DEV void reduce4(f32x4 (&acc)[4], float* red, int wave, int lane) {
  // red [wave][sub][reg][lane]; afterwards acc[wave] of every wave holds the sum over the four waves of sub-tile `wave`
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) red[((wave * 4 + i) * 4 + j) * 64 + lane] = acc[i][j];
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) v += red[((w * 4 + wave) * 4 + j) * 64 + lane];
    acc[0][j] = v;
  }
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(MoeGroupedParams p) {
  using F = Frag<T>;
  __shared__ float red[4 * 4 * 4 * 64];
  const int t = blockIdx.y;
  if (t >= *p.num_tiles) return;
  const int e = p.tile_expert[t];
  const bool sh = e >= p.E;
  const int Fe = sh ? p.Fs : p.F;
  if ((int)blockIdx.x * 16 >= Fe) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const bool gated = p.gate != nullptr;  // uniform: experts without a gate are down(relu(up x)^2)
  const T* up = sh ? reinterpret_cast<const T*>(p.sup) : reinterpret_cast<const T*>(p.up) + (int64_t)e * p.F * p.W;
  const T* gate = !gated ? up
                         : (sh ? reinterpret_cast<const T*>(p.sgate)
                               : reinterpret_cast<const T*>(p.gate) + (int64_t)e * p.F * p.W);
  const int* ids = p.sorted + t * kMoeRows;
  // an expert's ids fill its tiles from the front: a 16-row sub-tile is empty when its first id is a pad
  const T* xr[4];
  bool xv[4], live[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int id = ids[16 * i + r];
    live[i] = ids[16 * i] >= 0;
    xv[i] = id >= 0;
    xr[i] = reinterpret_cast<const T*>(p.x) + (int64_t)(xv[i] ? id / p.S : 0) * p.W;
  }
  const int f = blockIdx.x * 16 + r;
  const bool fv = f < Fe;
  const T* gr = gate + (int64_t)(fv ? f : 0) * p.W;
  const T* ur = up + (int64_t)(fv ? f : 0) * p.W;
  const bool vec = p.vec_w != 0;
  f32x4 ag[4], au[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) ag[i] = au[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = wave * F::KS; k0 < p.W; k0 += 4 * F::KS) {
    const int k = k0 + F::PER * g;
    const typename F::V bu = load_frag<T>(ur, k, p.W, fv, vec);
    const typename F::V bg = gated ? load_frag<T>(gr, k, p.W, fv, vec) : bu;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (!live[i]) continue;  // uniform over the workgroup
      const typename F::V a = load_frag<T>(xr[i], k, p.W, xv[i], vec);
      if (gated) ag[i] = mma(a, bg, ag[i]);
      au[i] = mma(a, bu, au[i]);
    }
  }
  if (gated) reduce4(ag, red, wave, lane);
  reduce4(au, red, wave, lane);
  if (!fv || !live[wave]) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int id2 = ids[16 * wave + 4 * g + j];
    if (id2 < 0) continue;
    const float gv = ag[0][j], uv = au[0][j];
    reinterpret_cast<T*>(p.h)[(int64_t)id2 * p.ldh + f] =
        (T)(gated ? gv / (1.0f + expf(-gv)) * uv : (uv > 0.0f ? uv * uv : 0.0f));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(MoeGroupedParams p) {
  using F = Frag<T>;
  __shared__ float red[4 * 4 * 4 * 64];
  const int t = blockIdx.y;
  if (t >= *p.num_tiles) return;
  const int e = p.tile_expert[t];
  const bool sh = e >= p.E;
  const int Fe = sh ? p.Fs : p.F;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const T* down = sh ? reinterpret_cast<const T*>(p.sdown) : reinterpret_cast<const T*>(p.down) + (int64_t)e * p.W * p.F;
  const int* ids = p.sorted + t * kMoeRows;
  const T* hr[4];
  bool hv[4], live[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int id = ids[16 * i + r];
    live[i] = ids[16 * i] >= 0;
    hv[i] = id >= 0;
    hr[i] = reinterpret_cast<const T*>(p.h) + (int64_t)(hv[i] ? id : 0) * p.ldh;
  }
  const int d = blockIdx.x * 16 + r;
  const bool dv = d < p.W;
  const T* dr = down + (int64_t)(dv ? d : 0) * Fe;
  const bool vech = p.vec_h != 0, vecd = p.vec_h != 0 && Fe % F::PER == 0;
  f32x4 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = wave * F::KS; k0 < Fe; k0 += 4 * F::KS) {
    const int k = k0 + F::PER * g;
    const typename F::V b = load_frag<T>(dr, k, Fe, dv, vecd);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (!live[i]) continue;
      acc[i] = mma(load_frag<T>(hr[i], k, Fe, hv[i], vech), b, acc[i]);
    }
  }
  reduce4(acc, red, wave, lane);
  if (!dv || !live[wave]) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int id2 = ids[16 * wave + 4 * g + j];
    if (id2 < 0) continue;
    const int row = id2 / p.S, k = id2 % p.S;
    const float wgt = k < p.top ? p.topk_w[row * p.top + k] : 1.0f;
    p.o[(int64_t)id2 * p.W + d] = wgt * acc[0][j];
  }
}

// Prompt-sized row counts (bf16, widths multiples of 8): the same two GEMMs with both operands staged through LDS.
// A workgroup owns a 64-row tile of one expert times 128 weight rows (MODE 0: 64 hidden units' gate rows and the same
// units' up rows; MODE 1: 128 output columns of the down projection) and walks K in chunks of 64: 256 threads copy the
// next chunk global -> registers while the MFMAs read the current one from LDS (two buffers, rows padded to 144 bytes so
// that a fragment read touches every bank once).  Each wave holds 4 row tiles x 2 weight tiles of accumulators: 8 MFMAs
// per 6 fragment reads from LDS, and every weight element leaves global memory once per 64 rows instead of once per
// wave.
constexpr int kLdsK = 64;            // K elements per chunk
constexpr int kLdsRow = kLdsK + 8;   // padded LDS row, bf16 elements

template <int MODE>
__global__ __launch_bounds__(256) void moe_tile_lds_kernel(MoeGroupedParams p) {
  __shared__ __align__(16) bf16 sa[2][64 * kLdsRow];
  __shared__ __align__(16) bf16 sb[2][128 * kLdsRow];
  const int t = blockIdx.y;
  if (t >= *p.num_tiles) return;
  const int e = p.tile_expert[t];
  const bool sh = e >= p.E;
  const int Fe = sh ? p.Fs : p.F;
  const int K = MODE == 1 ? Fe : p.W;          // reduction length
  const int N = MODE == 1 ? p.W : Fe;          // weight rows of one kind
  const int n0 = blockIdx.x * (MODE == 0 ? 64 : 128);
  if (n0 >= N) return;
  const int* ids = p.sorted + t * kMoeRows;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
  const bf16* X = reinterpret_cast<const bf16*>(MODE == 1 ? p.h : p.x);
  const int ldx = MODE == 1 ? p.ldh : p.W;
  const bf16 *w0, *w1;  // MODE 0: gate, up; MODE 1: down (w1 unused); MODE 2: up alone (experts without a gate)
  if (MODE == 2) {
    w0 = w1 = reinterpret_cast<const bf16*>(p.up) + (int64_t)e * p.F * p.W;
  } else if (MODE == 0) {
    w0 = sh ? reinterpret_cast<const bf16*>(p.sgate) : reinterpret_cast<const bf16*>(p.gate) + (int64_t)e * p.F * p.W;
    w1 = sh ? reinterpret_cast<const bf16*>(p.sup) : reinterpret_cast<const bf16*>(p.up) + (int64_t)e * p.F * p.W;
  } else {
    w0 = sh ? reinterpret_cast<const bf16*>(p.sdown) : reinterpret_cast<const bf16*>(p.down) + (int64_t)e * p.W * p.F;
    w1 = w0;
  }
  // this thread's copies per chunk: 2 of the A tile (64 rows x 8 sixteen-byte pieces), 4 of the B tile (128 rows x 8)
  const bf16* ap[2];
  const bf16* bp[4];
  int ak[2], bk[4], ao[2], bo[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = tid + 256 * i, row = idx >> 3, pc = idx & 7;
    const int id = ids[row];
    ap[i] = id >= 0 ? X + (int64_t)(MODE == 1 ? id : id / p.S) * ldx : nullptr;
    ak[i] = 8 * pc;
    ao[i] = row * kLdsRow + 8 * pc;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = tid + 256 * i, row = idx >> 3, pc = idx & 7;
    int n;
    const bf16* base;
    if (MODE == 0) {
      n = n0 + (row & 63);
      base = row < 64 ? w0 : w1;
    } else {
      n = n0 + row;
      base = w0;
    }
    bp[i] = n < N ? base + (int64_t)n * K : nullptr;
    bk[i] = 8 * pc;
    bo[i] = row * kLdsRow + 8 * pc;
  }
  bf16x8 ra[2], rb[4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      ra[i] = (ap[i] && k0 + ak[i] < K) ? ld_global<bf16x8>(ap[i] + k0 + ak[i]) : zero_bf16x8();
#pragma unroll
    for (int i = 0; i < 4; ++i)
      rb[i] = (bp[i] && k0 + bk[i] < K) ? ld_global<bf16x8>(bp[i] + k0 + bk[i]) : zero_bf16x8();
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<bf16x8*>(&sa[buf][ao[i]]) = ra[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<bf16x8*>(&sb[buf][bo[i]]) = rb[i];
  };
  f32x4 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i][0] = acc[i][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  // this wave's two weight tiles inside the B tile
  const int br0 = MODE == 0 ? 16 * wave : 32 * wave;
  const int br1 = MODE == 0 ? 64 + 16 * wave : 32 * wave + 16;
  fetch(0);
  stash(0);
  __syncthreads();
  const int nchunks = (K + kLdsK - 1) / kLdsK;
  for (int c = 0; c < nchunks; ++c) {
    const int buf = c & 1;
    if (c + 1 < nchunks) fetch((c + 1) * kLdsK);
#pragma unroll
    for (int ks = 0; ks < kLdsK; ks += 32) {
      const bf16x8 b0 = *reinterpret_cast<const bf16x8*>(&sb[buf][(br0 + r) * kLdsRow + ks + 8 * g]);
      const bf16x8 b1 = *reinterpret_cast<const bf16x8*>(&sb[buf][(br1 + r) * kLdsRow + ks + 8 * g]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&sa[buf][(16 * i + r) * kLdsRow + ks + 8 * g]);
        acc[i][0] = mfma16x16x32(a, b0, acc[i][0]);
        acc[i][1] = mfma16x16x32(a, b1, acc[i][1]);
      }
    }
    if (c + 1 < nchunks) stash(buf ^ 1);  // the other buffer: its readers finished before the previous barrier
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int id = ids[16 * i + 4 * g + j];
      if (id < 0) continue;
      if (MODE == 0) {
        const int f = n0 + 16 * wave + r;
        if (f >= N) continue;
        const float gv = acc[i][0][j];
        reinterpret_cast<bf16*>(p.h)[(int64_t)id * p.ldh + f] = (bf16)(gv / (1.0f + expf(-gv)) * acc[i][1][j]);
      } else if (MODE == 2) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const int f = n0 + 32 * wave + 16 * q + r;
          const float uv = acc[i][q][j];
          if (f < N) reinterpret_cast<bf16*>(p.h)[(int64_t)id * p.ldh + f] = (bf16)(uv > 0.0f ? uv * uv : 0.0f);
        }
      } else {
        const int row = id / p.S, k = id % p.S;
        const float wgt = k < p.top ? p.topk_w[row * p.top + k] : 1.0f;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const int d = n0 + 32 * wave + 16 * q + r;
          if (d < N) p.o[(int64_t)id * p.W + d] = wgt * acc[i][q][j];
        }
      }
    }
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_moe_router(const dsse::MoeRouterParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  const size_t lds = sizeof(float) * p->E;
  if (p->f32) hipLaunchKernelGGL(dsse::moe_router_kernel<float>, dim3(p->M), dim3(64), lds, st, *p);
  else hipLaunchKernelGGL(dsse::moe_router_kernel<bf16>, dim3(p->M), dim3(64), lds, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_moe_ffn(const dsse::MoeFfnParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  const int fmax = p->F > p->Fs ? p->F : p->Fs;
  const size_t lds = sizeof(float) * (2 * (size_t)p->W + fmax);
  if (lds > 64 * 1024) return hipErrorInvalidValue;
  if (p->f32) hipLaunchKernelGGL(dsse::moe_ffn_kernel<float>, dim3(p->M), dim3(256), lds, st, *p);
  else hipLaunchKernelGGL(dsse::moe_ffn_kernel<bf16>, dim3(p->M), dim3(256), lds, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_moe_grouped(const dsse::MoeGroupedParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  const int NE = p->E + (p->S > p->top ? 1 : 0);
  hipLaunchKernelGGL(dsse::moe_align_kernel, dim3(1), dim3(256), sizeof(int) * (3 * NE + 1), st, *p);
  const int fmax = p->F > p->Fs ? p->F : p->Fs;
  dim3 g1((fmax + 15) / 16, p->max_tiles), g2((p->W + 15) / 16, p->max_tiles);
  // prompt-sized steps in bf16 with 16-byte-aligned rows: operands staged through LDS
  if (!p->f32 && p->lds_tiles && p->W % 8 == 0 && p->F % 8 == 0 && p->Fs % 8 == 0 && p->ldh % 8 == 0) {
    dim3 l1((fmax + 63) / 64, p->max_tiles), l2((p->W + 127) / 128, p->max_tiles), l3((fmax + 127) / 128, p->max_tiles);
    if (p->gate) hipLaunchKernelGGL(dsse::moe_tile_lds_kernel<0>, l1, dim3(256), 0, st, *p);
    else hipLaunchKernelGGL(dsse::moe_tile_lds_kernel<2>, l3, dim3(256), 0, st, *p);
    hipLaunchKernelGGL(dsse::moe_tile_lds_kernel<1>, l2, dim3(256), 0, st, *p);
    return hipGetLastError();
  }
  if (p->f32) {
    hipLaunchKernelGGL(dsse::moe_gate_up_kernel<float>, g1, dim3(256), 0, st, *p);
    hipLaunchKernelGGL(dsse::moe_down_kernel<float>, g2, dim3(256), 0, st, *p);
  } else {
    hipLaunchKernelGGL(dsse::moe_gate_up_kernel<bf16>, g1, dim3(256), 0, st, *p);
    hipLaunchKernelGGL(dsse::moe_down_kernel<bf16>, g2, dim3(256), 0, st, *p);
  }
  return hipGetLastError();
}

extern "C" hipError_t dsse_moe_topk(const float* z, int M, int E, int top, int* topk_idx, float* topk_w, hipStream_t st) {
  if (M <= 0) return hipSuccess;
  hipLaunchKernelGGL(dsse::moe_topk_kernel, dim3((M + 255) / 256), dim3(256), 0, st, z, M, E, top, topk_idx, topk_w);
  return hipGetLastError();
}
