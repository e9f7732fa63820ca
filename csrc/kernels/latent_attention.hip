// Latent (compressed-KV) attention with a sliding window over the engine's paged cache.
//
// The cache holds, per token and layer, one row [normed latent c (rk) | rotated shared key part (dr)] -- nothing per
// head.  Attention runs in the folded form: with q_abs[h] = W_uk[h]^T q_unrotated[h] (a per-head GEMM before this
// kernel), the score of head h against token j is (q_abs[h] . c_j + rot(q_rot[h]) . kr_j) * scale, and the head's output
// is W_uv[h] (sum_j p_j c_j) (a per-head GEMM after it).  So every head reads the same rk + dr numbers per key and the
// kernel is multi-query attention with key width rk + dr and value width rk.
//
//   latent_kv_write   c = rms-norm(down-projection[:rk]) * w, kr = rot(down-projection[rk:]) -> cache row of the token
//                     (and c once more into the transposed page that the MFMA form reads its values from)
//   latent_attention  generic row kernel (any element type, any sizes): one workgroup per (query tile, head), the
//                     tile's rows one after the other; keys max(0, pos - window + 1) .. pos through the block table,
//                     256 keys per pass (one key per thread for the scores, one latent coordinate per thread for the
//                     weighted sum), online softmax in fp32.  Decode is a one-row tile.
//
// Rotation: interleaved pairs (2i, 2i + 1) of the rotated part, angle from a host-made fp32 (cos, sin) table per
// position that already carries the frequency scaling and amplitude of the design.
#include "api_layers.h"

namespace dsse {
namespace {

DEV float block_reduce_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) s += red[i];
  return s;
}
DEV float block_reduce_max(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = red[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) s = fmaxf(s, red[i]);
  return s;
}

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(LatentKvWriteParams p, T* __restrict__ vt) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  const int slot = p.slots[row];
  if (slot < 0 || slot >= p.num_slots) return;  // uniform per workgroup
  const int D = p.rk + p.dr;
  const float* src = p.ckr + (int64_t)row * p.ld;
  T* dst = reinterpret_cast<T*>(p.cache) + (int64_t)slot * D;
  float ss = 0.f;
  for (int d = threadIdx.x; d < p.rk; d += blockDim.x) ss += src[d] * src[d];
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)p.rk + p.eps);
  const T* nw = reinterpret_cast<const T*>(p.norm_w);
  // vt (optional): the latent once more in the transposed page of the MFMA attention form, key order of that form
  const int off = slot % kBS;
  T* vdst = vt ? vt + (int64_t)(slot / kBS) * p.rk * kBS + (((off & 15) >> 2) * 8 + ((off >> 4) & 1) * 4 + (off & 3))
               : nullptr;
  for (int d = threadIdx.x; d < p.rk; d += blockDim.x) {
    const T v = (T)(src[d] * inv * (float)nw[d]);
    dst[d] = v;
    if (vdst) vdst[(int64_t)d * kBS] = v;
  }
  int pos = p.positions[row];
  pos = pos < 0 ? 0 : (pos >= p.rope_len ? p.rope_len - 1 : pos);
  const float2* cs = p.rope + (int64_t)pos * (p.dr / 2);
  for (int i = threadIdx.x; i < p.dr / 2; i += blockDim.x) {
    const float u = src[p.rk + 2 * i], v = src[p.rk + 2 * i + 1];
    const float2 a = cs[i];
    dst[p.rk + 2 * i] = (T)(u * a.x - v * a.y);
    dst[p.rk + 2 * i + 1] = (T)(v * a.x + u * a.y);
  }
}

constexpr int kAccMax = 4;  // latent coordinates per thread: rk <= 1024

template <typename T>
__global__ __launch_bounds__(256) void latent_attention_rows_kernel(LatentAttnParams p) {
  extern __shared__ float smem[];
  const int D = p.rk + p.dr;
  float* qv = smem;               // [D]
  float* sc = smem + D;           // [256] scores, then weights
  int* sl = reinterpret_cast<int*>(sc + 256);  // [256] cache rows of the pass's keys
  float* red = reinterpret_cast<float*>(sl + 256);  // [4]
  const int tid = threadIdx.x;
  const int seq = p.work_seq[blockIdx.x], tile = p.work_tile[blockIdx.x], h = blockIdx.y;
  const int ql = p.q_len[seq];
  const int* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const T* cache = reinterpret_cast<const T*>(p.cache);
  for (int i = 0; i < p.qt; ++i) {
    const int off = tile * p.qt + i;
    if (off >= ql) break;  // uniform
    const int row = p.q_start[seq] + off;
    const int pos = p.ctx_len[seq] - ql + off;
    __syncthreads();
    for (int d = tid; d < p.rk; d += 256) qv[d] = p.q_abs[((int64_t)row * p.H + h) * p.rk + d];
    {
      const T* qr = reinterpret_cast<const T*>(p.q) + ((int64_t)row * p.H + h) * (p.dn + p.dr) + p.dn;
      const int pp = pos < 0 ? 0 : (pos >= p.rope_len ? p.rope_len - 1 : pos);
      const float2* cs = p.rope + (int64_t)pp * (p.dr / 2);
      for (int k = tid; k < p.dr / 2; k += 256) {
        const float u = (float)qr[2 * k], v = (float)qr[2 * k + 1];
        const float2 a = cs[k];
        qv[p.rk + 2 * k] = u * a.x - v * a.y;
        qv[p.rk + 2 * k + 1] = v * a.x + u * a.y;
      }
    }
    __syncthreads();
    const int lo = pos - p.window + 1 > 0 ? pos - p.window + 1 : 0;
    float m = -INFINITY, l = 0.f;
    float acc[kAccMax];
#pragma unroll
    for (int a = 0; a < kAccMax; ++a) acc[a] = 0.f;
    for (int kb = lo; kb <= pos; kb += 256) {
      const int j = kb + tid;
      float s = -INFINITY;
      int slot = 0;
      if (j <= pos) {
        int blk = bt[j / kBS];
        blk = (unsigned)blk < (unsigned)p.num_blocks ? blk : 0;  // a stale table entry never leaves the cache
        slot = blk * kBS + j % kBS;
        const T* e = cache + (int64_t)slot * D;
        float dot = 0.f;
        for (int d = 0; d < D; ++d) dot += qv[d] * (float)e[d];
        s = dot * p.scale;
      }
      sl[tid] = slot;
      const float bm = block_reduce_max(s, red);
      const float mn = fmaxf(m, bm);
      const float corr = m == -INFINITY ? 0.f : expf(m - mn);
      const float pj = j <= pos ? expf(s - mn) : 0.f;
      sc[tid] = pj;
      const float bs = block_reduce_sum(pj, red);  // its barriers also publish sc / sl
      l = l * corr + bs;
      m = mn;
      const int nk = pos - kb + 1 < 256 ? pos - kb + 1 : 256;
#pragma unroll
      for (int a = 0; a < kAccMax; ++a) {
        const int d = tid + 256 * a;
        if (d < p.rk) {
          float v = acc[a] * corr;
          for (int jj = 0; jj < nk; ++jj) v += sc[jj] * (float)cache[(int64_t)sl[jj] * D + d];
          acc[a] = v;
        }
      }
      __syncthreads();
    }
    T* out = reinterpret_cast<T*>(p.out) + ((int64_t)row * p.H + h) * p.rk;
    const float inv = 1.0f / l;
#pragma unroll
    for (int a = 0; a < kAccMax; ++a) {
      const int d = tid + 256 * a;
      if (d < p.rk) out[d] = (T)(acc[a] * inv);
    }
  }
}

}  // namespace

// ---------------------------------------------------------------------------------------------------------------------
// MFMA form (bf16): one wave per work item, 16 query columns, 32 keys (one cache page) per step, no LDS for keys or
// values.  A column is a (row, head) pair: a decode step puts 16 heads of its one row side by side (the page is read
// once for all of them), a prompt portion puts 16 rows of one head (or rt rows x hp heads).
//
//   S^T[key, col] = K[key, :] . Q[col, :]     A = the page's key rows straight from global memory (16 B per lane),
//                                              B = the columns' query vectors [q_abs | rot(q_rot)] staged in LDS as bf16
//   online softmax per column in fp32 (a column's 32 scores sit in 8 registers of its 4 lanes: rows4_max / rows4_sum)
//   O^T[dim, col] += V^T[dim, key] . P^T[key, col]
//                                              A = the TRANSPOSED latent page vt[page][dim][32 keys] (16 B per lane),
//                                              B = the probabilities exactly as the score accumulators hold them
//
// The last step needs no shuffle because which key a (lane group g, element j) pair of the k axis stands for only has
// to agree between A and B: the scores of lane group g are keys 4g..4g+3 of both 16-key halves, so the transposed page
// stores key k at position 8 ((k & 15) >> 2) + 4 (k >> 4) + (k & 3) (the dense KV cache's V pages use the same order).
// A workgroup is up to four such waves: the head tiles of the SAME rows, which walk the same pages at the same time and
// so share them in the CU's L1 instead of each pulling the whole window from L2 (the launch is L2-bound otherwise).
template <int NT>  // rk / 16 value tiles
__global__ __launch_bounds__(256) void latent_flash_kernel(LatentAttnParams p, const bf16* __restrict__ vt, int rt, int hp,
                                                           int head_tiles) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int D = p.rk + p.dr;
  const int ldq = D + 8;  // bf16 elements per LDS row (16 B of padding)
  const int wave = threadIdx.x >> 6;
  const int hy = blockIdx.y * (blockDim.x >> 6) + wave;  // this wave's head tile
  bf16* qs = reinterpret_cast<bf16*>(smem_raw) + wave * 16 * ldq;  // [16][ldq] per wave
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int seq = p.work_seq[blockIdx.x], tile = p.work_tile[blockIdx.x];
  const int ql = p.q_len[seq];
  if (tile * rt >= ql) return;
  const int q0 = p.q_start[seq], pos0 = p.ctx_len[seq] - ql;
  // this lane's column
  const int c_off = tile * rt + r / hp, c_head = hy * hp + r % hp;
  const bool c_ok = c_off < ql && c_head < p.H && hy < head_tiles;
  const int c_pos = c_ok ? pos0 + c_off : -1;
  const int64_t c_row = q0 + (c_ok ? c_off : 0);
  // stage the 16 query vectors: lane group g fills coordinates g, g + 4, ... (in chunks of 8) of column r
  {
    const float* qa = p.q_abs + (c_row * p.H + (c_ok ? c_head : 0)) * p.rk;
    for (int d = 8 * g; d < p.rk; d += 32) {  // rk % 32 == 0: the eight floats are two aligned 16-byte loads
      const f32x4 lo4 = c_ok ? *reinterpret_cast<const f32x4*>(qa + d) : f32x4{0.f, 0.f, 0.f, 0.f};
      const f32x4 hi4 = c_ok ? *reinterpret_cast<const f32x4*>(qa + d + 4) : f32x4{0.f, 0.f, 0.f, 0.f};
      bf16x8 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (bf16)lo4[j], v[4 + j] = (bf16)hi4[j];
      *reinterpret_cast<bf16x8*>(qs + r * ldq + d) = v;
    }
    const bf16* qr = reinterpret_cast<const bf16*>(p.q) + (c_row * p.H + (c_ok ? c_head : 0)) * (p.dn + p.dr) + p.dn;
    const int pp = c_pos < 0 ? 0 : (c_pos >= p.rope_len ? p.rope_len - 1 : c_pos);
    const float2* cs = p.rope + (int64_t)pp * (p.dr / 2);
    for (int d = 8 * g; d < p.dr; d += 32) {
      // eight rotated coordinates: one 16-byte load when the head's row allows it (dn and dr multiples of 8)
      bf16x8 raw = zero_bf16x8();
      if (c_ok) {
        if (((p.dn + p.dr) % 8 == 0) && (p.dn % 8 == 0)) raw = ld_bf16x8(qr + d);
        else
#pragma unroll
          for (int j = 0; j < 8; ++j) raw[j] = qr[d + j];
      }
      bf16x8 v;
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        const float a = (float)raw[j], b = (float)raw[j + 1];
        const float2 t = cs[(d + j) / 2];
        v[j] = (bf16)(a * t.x - b * t.y);
        v[j + 1] = (bf16)(b * t.x + a * t.y);
      }
      *reinterpret_cast<bf16x8*>(qs + r * ldq + p.rk + d) = v;
    }
  }
  __syncthreads();
  if (hy >= head_tiles) return;
  // key range of the tile: from the first row's window start to the last row's position
  const int last_off = (tile * rt + rt - 1 < ql ? tile * rt + rt - 1 : ql - 1);
  const int hi = pos0 + last_off;
  int lo = pos0 + tile * rt - p.window + 1;
  lo = lo > 0 ? lo : 0;
  const int* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const bf16* rows = reinterpret_cast<const bf16*>(p.cache);
  f32x4 O[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) O[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int nks = D / 32;
  int pg0 = lo / kBS, pg1 = hi / kBS;
  const int np = p.nparts > 1 ? p.nparts : 1;
  if (np > 1) {  // this partition's share of the pages (even split of the item's own range)
    const int per = (pg1 - pg0 + np) / np;
    pg0 += blockIdx.z * per;
    pg1 = pg0 + per - 1 < pg1 ? pg0 + per - 1 : pg1;
  }
  for (int pg = pg0; pg <= pg1; ++pg) {
    int blk = bt[pg];
    blk = (unsigned)blk < (unsigned)p.num_blocks ? blk : 0;
    const bf16* krow0 = rows + ((int64_t)blk * kBS + r) * D + 8 * g;        // key r of the page's first half
    const bf16* krow1 = krow0 + (int64_t)16 * D;                             // key 16 + r
    // the page's value fragments are requested first: they arrive while the scores are computed (a single wave per
    // SIMD has nothing else to hide their latency behind)
    const bf16* vrow = vt + ((int64_t)blk * p.rk + r) * kBS + 8 * g;  // dim r of value tile 0, positions 8g..8g+7
    bf16x8 vf[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) vf[n] = ld_global<bf16x8>(vrow + (int64_t)n * 16 * kBS);
    f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
    // six k-steps at a time: their twelve key loads are issued before the first MFMA needs one (a single wave per
    // work item has nothing else to hide the load latency behind)
    for (int sb = 0; sb < nks; sb += 6) {
      bf16x8 ka[6], kb[6], qb[6];
#pragma unroll
      for (int u = 0; u < 6; ++u) {
        const int s = sb + u < nks ? sb + u : nks - 1;  // past the end: a valid address, the product is skipped
        ka[u] = ld_global<bf16x8>(krow0 + 32 * s);
        kb[u] = ld_global<bf16x8>(krow1 + 32 * s);
        qb[u] = *reinterpret_cast<const bf16x8*>(qs + r * ldq + 32 * s + 8 * g);
      }
#pragma unroll
      for (int u = 0; u < 6; ++u) {
        if (sb + u < nks) {
          s0 = mfma16x16x32(ka[u], qb[u], s0);
          s1 = mfma16x16x32(kb[u], qb[u], s1);
        }
      }
    }
    // lane (r, g): column r, keys pg * 32 + 4 g + i (s0) and + 16 (s1)
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int key = pg * kBS + (i < 4 ? 4 * g + i : 16 + 4 * g + (i - 4));
      const bool seen = c_ok && key <= c_pos && c_pos - key < p.window;
      sv[i] = seen ? (i < 4 ? s0[i] : s1[i - 4]) * p.scale : -INFINITY;
      mx = fmaxf(mx, sv[i]);
    }
    mx = rows4_max(mx);
    const float mn = fmaxf(m, mx);
    const float corr = mn == -INFINITY ? 1.0f : expf(m - mn);  // m = -inf, mn finite: exp(-inf) = 0
    bf16x8 pf;
    float ps = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float e = sv[i] == -INFINITY ? 0.0f : expf(sv[i] - mn);
      ps += e;
      pf[i] = (bf16)e;
    }
    l = l * corr + rows4_sum(ps);
    m = mn;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      f32x4 o = O[n];
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] *= corr;
      O[n] = mfma16x16x32(vf[n], pf, o);
    }
  }
  if (np > 1) {
    float* po = p.part + (((int64_t)blockIdx.x * head_tiles + hy) * np + blockIdx.z) * (16 * (p.rk + 2));
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) po[r * p.rk + 16 * n + 4 * g + i] = O[n][i];
    if (g == 0) {
      po[16 * p.rk + 2 * r] = m;
      po[16 * p.rk + 2 * r + 1] = l;
    }
    return;
  }
  if (c_ok) {
    bf16* out = reinterpret_cast<bf16*>(p.out) + (c_row * p.H + c_head) * p.rk;
    const float inv = l > 0.f ? 1.0f / l : 0.0f;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (bf16)(O[n][i] * inv);
      *reinterpret_cast<bf16x4*>(out + 16 * n + 4 * g) = v;
    }
  }
}

// Merge of the key partitions of latent_flash_kernel: per column, M = max of the partitions' maxima,
// out = sum_z e^(m_z - M) O_z / sum_z e^(m_z - M) l_z.
__global__ __launch_bounds__(256) void latent_flash_combine_kernel(LatentAttnParams p, int rt, int hp) {
  // one workgroup per (item, head tile, column)
  const int seq = p.work_seq[blockIdx.x], tile = p.work_tile[blockIdx.x];
  const int ql = p.q_len[seq];
  const int ht = blockIdx.y / 16, col = blockIdx.y % 16;
  const int off = tile * rt + col / hp, head = ht * hp + col % hp;
  if (off >= ql || head >= p.H) return;
  const int np = p.nparts;
  const int stride = 16 * (p.rk + 2);
  const float* base = p.part + ((int64_t)blockIdx.x * (gridDim.y / 16) + ht) * np * stride;
  const float* ml = base + 16 * p.rk + 2 * col;
  float M = -INFINITY;
  for (int z = 0; z < np; ++z) M = fmaxf(M, ml[z * stride]);
  float den = 0.f;
  for (int z = 0; z < np; ++z) {
    const float mz = ml[z * stride];
    if (mz != -INFINITY) den += expf(mz - M) * ml[z * stride + 1];
  }
  const float inv = den > 0.f ? 1.0f / den : 0.0f;
  bf16* out = reinterpret_cast<bf16*>(p.out) + ((int64_t)(p.q_start[seq] + off) * p.H + head) * p.rk;
  for (int d = threadIdx.x; d < p.rk; d += blockDim.x) {
    float num = 0.f;
    for (int z = 0; z < np; ++z) {
      const float mz = ml[z * stride];
      if (mz != -INFINITY) num += expf(mz - M) * base[z * stride + col * p.rk + d];
    }
    out[d] = (bf16)(num * inv);
  }
}

}  // namespace dsse

extern "C" hipError_t dsse_latent_kv_write(const dsse::LatentKvWriteParams* p, void* vt, hipStream_t st) {
  if (p->T <= 0) return hipSuccess;
  if (p->f32)
    hipLaunchKernelGGL(dsse::latent_kv_write_kernel<float>, dim3(p->T), dim3(256), 0, st, *p, reinterpret_cast<float*>(vt));
  else
    hipLaunchKernelGGL(dsse::latent_kv_write_kernel<bf16>, dim3(p->T), dim3(256), 0, st, *p, reinterpret_cast<bf16*>(vt));
  return hipGetLastError();
}

extern "C" hipError_t dsse_latent_attention(int num_work, const dsse::LatentAttnParams* p, hipStream_t st) {
  if (num_work <= 0) return hipSuccess;
  if (p->rk > 256 * dsse::kAccMax) return hipErrorInvalidValue;
  const size_t lds = sizeof(float) * (p->rk + p->dr + 256 + 256 + 4);
  dim3 grid(num_work, p->H);
  if (p->f32) hipLaunchKernelGGL(dsse::latent_attention_rows_kernel<float>, grid, dim3(256), lds, st, *p);
  else hipLaunchKernelGGL(dsse::latent_attention_rows_kernel<bf16>, grid, dim3(256), lds, st, *p);
  return hipGetLastError();
}

// rt rows x hp heads = 16 columns per work item; work_tile counts tiles of rt rows
extern "C" hipError_t dsse_latent_flash(int num_work, const dsse::LatentAttnParams* p, const void* vt, int rt, int hp,
                                        hipStream_t st) {
  if (num_work <= 0) return hipSuccess;
  if (p->f32 || rt * hp != 16 || p->rk % 32 || p->dr % 32) return hipErrorInvalidValue;
  const int np = p->nparts > 1 ? p->nparts : 1;
  if (np > 1 && !p->part) return hipErrorInvalidValue;
  const int gy = (p->H + hp - 1) / hp;          // head tiles
  const int wy = gy < 4 ? gy : 4;               // of them, waves per workgroup
  const size_t lds = wy * 16 * (size_t)(p->rk + p->dr + 8) * sizeof(bf16);
  dim3 grid(num_work, (gy + wy - 1) / wy, np), block(64 * wy);
  const bf16* v = reinterpret_cast<const bf16*>(vt);
  switch (p->rk / 16) {
    case 4: hipLaunchKernelGGL(dsse::latent_flash_kernel<4>, grid, block, lds, st, *p, v, rt, hp, gy); break;
    case 8: hipLaunchKernelGGL(dsse::latent_flash_kernel<8>, grid, block, lds, st, *p, v, rt, hp, gy); break;
    case 16: hipLaunchKernelGGL(dsse::latent_flash_kernel<16>, grid, block, lds, st, *p, v, rt, hp, gy); break;
    case 32: hipLaunchKernelGGL(dsse::latent_flash_kernel<32>, grid, block, lds, st, *p, v, rt, hp, gy); break;
    default: return hipErrorInvalidValue;
  }
  if (np > 1)
    hipLaunchKernelGGL(dsse::latent_flash_combine_kernel, dim3(num_work, 16 * ((p->H + hp - 1) / hp)), dim3(256), 0, st, *p, rt,
                       hp);
  return hipGetLastError();
}
