// Causal softmax attention with a sink over paged keys and values of any head width (grouped key/value heads).
//
//   score_j = scale (q . k_j),  j in [max(0, pos - window + 1), pos]
//   out     = sum_j exp(score_j - m) v_j / (sum_j exp(score_j - m) + exp(sink_h - m)),  m = max(max_j score_j, sink_h)
//   out    *= sigmoid(gate[row, h])                                                      (optional)
//
// Options for designs that ask for them: capped scores, score_j = cap * tanh(scale (q . k_j) / cap); and an output
// rotation -- every head's sum is turned back by the query row's own position over the whole value width (rotate-half
// pairs (m, m + V / 2), angles from a (cos, sin) table), before the gate: with values that were rotated by THEIR
// positions when they were cached, a value then enters the output rotated by its distance to the query.
//
// The sink is a learned logit with no key and no value: it only enlarges the denominator, so a head can attend to
// "nothing".  Scores, the running maximum, the weights and the output sums are fp32 in both element types; queries
// arrive in fp32 (normed and rotated), keys and values are read from their pages in the cache's element type.
//
// Row kernel (any sizes, both element types; every decode step): a workgroup serves `qt` query rows of one head; for each row its four waves split the keys in chunks of
// 64 (one key per lane for the scores, then one output coordinate per lane and 64 broadcast weights for the values),
// keep their own running (max, sum, output) and are merged through LDS.  A decode row and a prompt row take the same
// path, so a position's result does not depend on how the prompt was cut.
#include "api_mixers.h"

namespace dsse {
namespace {

constexpr int kMaxV = 512;
constexpr int kAccs = kMaxV / 64;

// q (LDS, fp32) . key row (global): 16-byte loads when the row width allows
DEV float dot_row(const float* q, const bf16* k, int D) {
  float s = 0.f;
  int d = 0;
  if (D % 8 == 0) {
    for (; d < D; d += 8) {
      const bf16x8 kv = *reinterpret_cast<const bf16x8*>(k + d);
#pragma unroll
      for (int e = 0; e < 8; ++e) s += q[d + e] * (float)kv[e];
    }
  }
  for (; d < D; ++d) s += q[d] * (float)k[d];
  return s;
}
DEV float dot_row(const float* q, const float* k, int D) {
  float s = 0.f;
  int d = 0;
  if (D % 4 == 0) {
    for (; d < D; d += 4) {
      const f32x4 kv = *reinterpret_cast<const f32x4*>(k + d);
#pragma unroll
      for (int e = 0; e < 4; ++e) s += q[d + e] * kv[e];
    }
  }
  for (; d < D; ++d) s += q[d] * k[d];
  return s;
}

template <typename T>
__global__ __launch_bounds__(256) void sink_attention_kernel(SinkAttnParams p) {
  __shared__ float qs[512];
  __shared__ float m_s[4], l_s[4];
  __shared__ float acc_s[4][kMaxV];
  const int work = blockIdx.x, h = blockIdx.y;
  const int seq = p.work_seq[work], tile = p.work_tile[work];
  const int ql = p.q_len[seq];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = h / (p.H / p.G);
  const int D = p.D, V = p.V;
  const int* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const T* kc = reinterpret_cast<const T*>(p.k);
  const T* vc = reinterpret_cast<const T*>(p.v);
  const float sink = p.sink ? p.sink[h] : -INFINITY;
  for (int i = 0; i < p.qt; ++i) {
    const int off = tile * p.qt + i;
    if (off >= ql) break;  // uniform for the workgroup
    const int row = p.q_start[seq] + off;
    const int pos = p.ctx_len[seq] - ql + off;
    const int lo = pos - p.window + 1 > 0 ? pos - p.window + 1 : 0;
    const int nkeys = pos - lo + 1;
    __syncthreads();  // the previous row's merge has read qs / acc_s
    for (int d = threadIdx.x; d < D; d += blockDim.x) qs[d] = p.q[((int64_t)row * p.H + h) * D + d];
    __syncthreads();
    float m = -INFINITY, l = 0.f;
    float acc[kAccs];
#pragma unroll
    for (int a = 0; a < kAccs; ++a) acc[a] = 0.f;
    for (int c = wave; c * 64 < nkeys; c += 4) {
      const int jj = c * 64 + lane;
      const bool on = jj < nkeys;
      const int j = lo + (on ? jj : 0);
      int page = bt[j / kBS];
      page = (unsigned)page < (unsigned)p.num_blocks ? page : 0;
      const int krow = (page * kBS + j % kBS) * p.G + g;
      const float s_dot = dot_row(qs, kc + (int64_t)krow * D, D);
      float s = s_dot * p.scale;
      if (p.softcap > 0.f) s = p.softcap * tanhf(s / p.softcap);
      s = on ? s : -INFINITY;
      const float m_new = fmaxf(m, wave_max(s));  // finite: the chunk holds at least one key
      const float w = on ? expf(s - m_new) : 0.f;
      const float f = expf(m - m_new);            // 0 when m was -inf
      l = l * f + wave_sum(w);
      m = m_new;
#pragma unroll
      for (int a = 0; a < kAccs; ++a) acc[a] *= f;
      const int cnt = nkeys - c * 64 < 64 ? nkeys - c * 64 : 64;
      for (int t = 0; t < cnt; ++t) {
        const float wt = __shfl(w, t);
        const int vrow = __shfl(krow, t);
        const T* vp = vc + (int64_t)vrow * V;
#pragma unroll
        for (int a = 0; a < kAccs; ++a)
          if (a * 64 + lane < V) acc[a] += wt * (float)vp[a * 64 + lane];
      }
    }
    if (lane == 0) {
      m_s[wave] = m;
      l_s[wave] = l;
    }
#pragma unroll
    for (int a = 0; a < kAccs; ++a)
      if (a * 64 + lane < V) acc_s[wave][a * 64 + lane] = acc[a];
    __syncthreads();
    float mm = sink;
    for (int w = 0; w < 4; ++w) mm = fmaxf(mm, m_s[w]);
    float den = p.sink ? expf(sink - mm) : 0.f;
    float fw[4];
    for (int w = 0; w < 4; ++w) {
      fw[w] = m_s[w] == -INFINITY ? 0.f : expf(m_s[w] - mm);
      den += l_s[w] * fw[w];
    }
    const float gate = p.gate ? 1.0f / (1.0f + expf(-p.gate[(int64_t)row * p.ldg + h])) : 1.0f;
    T* out = reinterpret_cast<T*>(p.out) + ((int64_t)row * p.H + h) * V;
    const int half = V >> 1;
    const float2* orp = p.out_rope ? p.out_rope + (int64_t)(pos < p.out_rope_len ? pos : p.out_rope_len - 1) * half : nullptr;
    for (int d = threadIdx.x; d < V; d += blockDim.x) {
      float o = 0.f;
      for (int w = 0; w < 4; ++w) o += acc_s[w][d] * fw[w];
      if (orp) {  // back by the row's position: (a, b) -> (a cos + b sin, b cos - a sin)
        const bool lo_half = d < half;
        const int dp = lo_half ? d + half : d - half;
        float op = 0.f;
        for (int w = 0; w < 4; ++w) op += acc_s[w][dp] * fw[w];
        const float2 c = orp[lo_half ? d : dp];
        o = lo_half ? o * c.x + op * c.y : o * c.x - op * c.y;
      }
      out[d] = (T)(o / den * gate);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// MFMA form for prompt portions (bf16; D % 32 == 0, V % 16 == 0): one wave per (16 query rows, head), 32 keys (one
// page) per step, a workgroup = up to four heads of the same rows (heads of one key/value group read the same pages,
// which then come from the CU's L1).
//
//   S^T[key, row] = K[key, :] . Q[row, :]    A = the page's key rows straight from global memory (16 B per lane),
//                                             B = the 16 rows' query vectors staged in LDS as bf16
//   online softmax per row in fp32 (a row's 32 scores sit in 8 registers of its 4 lanes)
//   O^T[dim, row] += V^T[dim, key] . P^T[key, row]
//                                             A = the TRANSPOSED value page vt[page][G][V][32 keys] (16 B per lane),
//                                             B = the weights exactly as the score accumulators hold them
//
// Which key an (lane group g, element j) pair of the k axis stands for only has to agree between A and B: the scores of
// lane group g are keys 4g..4g+3 of both 16-key halves, so the transposed page stores key k at position
// 8 ((k & 15) >> 2) + 4 (k >> 4) + (k & 3).  The sink enters once, when the row is finished: it only enlarges the
// denominator.
//
// SPLIT (decode steps: few rows, long contexts): the four waves of a workgroup serve the SAME (tile, head) and take
// every fourth page each; their (max, sum, O) are merged through LDS, so a sequence's keys are walked by four waves at
// once and the launch has four times the waves.
// tanh through one exponential: the bf16 form's scores carry bf16 operand rounding, far above this form's error
DEV float tanh_fast(float x) {
  const float c = fminf(fmaxf(x, -15.0f), 15.0f);
  const float e = __expf(2.0f * c);
  return (e - 1.0f) / (e + 1.0f);
}

template <int NT, bool SPLIT>  // V / 16 value tiles
__global__ __launch_bounds__(256) void sink_flash_kernel(SinkAttnParams p, const bf16* __restrict__ vt, int head_tiles) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int D = p.D, V = p.V;
  const int ldq = D + 8;  // bf16 elements per LDS row (16 B of padding)
  const int wave = threadIdx.x >> 6;
  const int h = SPLIT ? blockIdx.y : blockIdx.y * (blockDim.x >> 6) + wave;
  bf16* qs = reinterpret_cast<bf16*>(smem_raw) + wave * 16 * ldq;
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int seq = p.work_seq[blockIdx.x], tile = p.work_tile[blockIdx.x];
  const int ql = p.q_len[seq];
  if (tile * 16 >= ql) return;
  const bool h_ok = h < head_tiles;
  const int hh = h_ok ? h : 0;
  const int kvh = hh / (p.H / p.G);
  const int q0 = p.q_start[seq], pos0 = p.ctx_len[seq] - ql;
  const int c_off = tile * 16 + r;
  const bool c_ok = c_off < ql && h_ok;
  const int c_pos = c_ok ? pos0 + c_off : -1;
  const int64_t c_row = q0 + (c_off < ql ? c_off : 0);
  {
    const float* qa = p.q + (c_row * p.H + hh) * D;
    for (int d = 8 * g; d < D; d += 32) {
      const f32x4 lo4 = c_ok ? *reinterpret_cast<const f32x4*>(qa + d) : f32x4{0.f, 0.f, 0.f, 0.f};
      const f32x4 hi4 = c_ok ? *reinterpret_cast<const f32x4*>(qa + d + 4) : f32x4{0.f, 0.f, 0.f, 0.f};
      bf16x8 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (bf16)lo4[j], v[4 + j] = (bf16)hi4[j];
      *reinterpret_cast<bf16x8*>(qs + r * ldq + d) = v;
    }
  }
  __syncthreads();
  if (!SPLIT && !h_ok) return;
  const int last_off = tile * 16 + 15 < ql ? tile * 16 + 15 : ql - 1;
  const int hi = pos0 + last_off;
  int lo = pos0 + tile * 16 - p.window + 1;
  lo = lo > 0 ? lo : 0;
  const int* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const bf16* kc = reinterpret_cast<const bf16*>(p.k);
  f32x4 O[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) O[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const float cap_inv = p.softcap > 0.f ? 1.0f / p.softcap : 0.f;
  const int nks = D / 32;
  for (int pg = lo / kBS + (SPLIT ? wave : 0); pg <= hi / kBS; pg += SPLIT ? 4 : 1) {
    int blk = bt[pg];
    blk = (unsigned)blk < (unsigned)p.num_blocks ? blk : 0;
    const bf16* krow0 = kc + (((int64_t)blk * kBS + r) * p.G + kvh) * D + 8 * g;  // key r of the page's first half
    const bf16* krow1 = krow0 + (int64_t)16 * p.G * D;                              // key 16 + r
    const bf16* vrow = vt + (((int64_t)blk * p.G + kvh) * V + r) * kBS + 8 * g;   // dim r of value tile 0
    bf16x8 vf[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) vf[n] = ld_global<bf16x8>(vrow + (int64_t)n * 16 * kBS);
    f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
    for (int sb = 0; sb < nks; sb += 4) {  // four k-steps of key loads are requested before the first MFMA needs one
      bf16x8 ka[4], kb[4], qb[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int s = sb + u < nks ? sb + u : nks - 1;
        ka[u] = ld_global<bf16x8>(krow0 + 32 * s);
        kb[u] = ld_global<bf16x8>(krow1 + 32 * s);
        qb[u] = *reinterpret_cast<const bf16x8*>(qs + r * ldq + 32 * s + 8 * g);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (sb + u < nks) {
          s0 = mfma16x16x32(ka[u], qb[u], s0);
          s1 = mfma16x16x32(kb[u], qb[u], s1);
        }
      }
    }
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int key = pg * kBS + (i < 4 ? 4 * g + i : 16 + 4 * g + (i - 4));
      const bool seen = c_ok && key <= c_pos && c_pos - key < p.window;
      float sc = (i < 4 ? s0[i] : s1[i - 4]) * p.scale;
      if (p.softcap > 0.f) sc = p.softcap * tanh_fast(sc * cap_inv);
      sv[i] = seen ? sc : -INFINITY;
      mx = fmaxf(mx, sv[i]);
    }
    mx = rows4_max(mx);
    const float mn = fmaxf(m, mx);
    const float corr = mn == -INFINITY ? 1.0f : expf(m - mn);
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
  if (SPLIT) {
    // merge the four waves' partial results: [wave][16 columns][V + 2] floats, after every wave has read its queries
    float* mg = reinterpret_cast<float*>(smem_raw) + 4 * 16 * ((ldq + 1) / 2);
    const int ldm = V + 2;
    float* mine = mg + (wave * 16 + r) * ldm;
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[16 * n + 4 * g + i] = O[n][i];
    if (g == 0) {
      mine[V] = m;
      mine[V + 1] = l;
    }
    __syncthreads();
    const int rows_on = ql - tile * 16 < 16 ? ql - tile * 16 : 16;
    for (int idx = threadIdx.x; idx < rows_on * V; idx += blockDim.x) {
      const int col = idx / V, d = idx - col * V;
      const int64_t row = q0 + tile * 16 + col;
      float mm = p.sink ? p.sink[h] : -INFINITY;
      for (int w = 0; w < 4; ++w) mm = fmaxf(mm, mg[(w * 16 + col) * ldm + V]);
      float den = p.sink ? expf(p.sink[h] - mm) : 0.f, num = 0.f, nump = 0.f;
      const int half = V >> 1;
      const bool lo_half = d < half;
      const int dp = lo_half ? d + half : d - half;
      for (int w = 0; w < 4; ++w) {
        const float* src = mg + (w * 16 + col) * ldm;
        const float f = src[V] == -INFINITY ? 0.f : expf(src[V] - mm);
        den += src[V + 1] * f;
        num += src[d] * f;
        nump += src[dp] * f;
      }
      if (p.out_rope) {  // back by the row's position
        const int ps = pos0 + tile * 16 + col;
        const float2 c = p.out_rope[(int64_t)(ps < p.out_rope_len ? ps : p.out_rope_len - 1) * half + (lo_half ? d : dp)];
        num = lo_half ? num * c.x + nump * c.y : num * c.x - nump * c.y;
      }
      float o = den > 0.f ? num / den : 0.f;
      if (p.gate) o *= 1.0f / (1.0f + expf(-p.gate[row * p.ldg + h]));
      reinterpret_cast<bf16*>(p.out)[(row * p.H + h) * V + d] = (bf16)o;
    }
    return;
  }
  if (c_ok) {
    float den = l, f = 1.0f;
    if (p.sink) {  // the sink joins the denominator under the common maximum
      const float sk = p.sink[h];
      const float mm = fmaxf(m, sk);
      f = expf(m - mm);
      den = l * f + expf(sk - mm);
    }
    float inv = den > 0.f ? f / den : 0.0f;
    if (p.gate) inv *= 1.0f / (1.0f + expf(-p.gate[c_row * p.ldg + h]));
    if (p.out_rope) {  // NT is even (the host checks V % 32 == 0): dimension m = 16 n + 4 g + i pairs with tile n + NT / 2
      const float2* orp = p.out_rope + (int64_t)(c_pos < p.out_rope_len ? c_pos : p.out_rope_len - 1) * (V >> 1);
#pragma unroll
      for (int n = 0; n < NT / 2; ++n)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float2 c = orp[16 * n + 4 * g + i];
          const float a = O[n][i], b = O[n + NT / 2][i];
          O[n][i] = a * c.x + b * c.y;
          O[n + NT / 2][i] = b * c.x - a * c.y;
        }
    }
    bf16* out = reinterpret_cast<bf16*>(p.out) + (c_row * p.H + h) * V;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (bf16)(O[n][i] * inv);
      *reinterpret_cast<bf16x4*>(out + 16 * n + 4 * g) = v;
    }
  }
}

template <int NT>
void launch_flash(int num_work, const SinkAttnParams& p, const bf16* vt, int split, hipStream_t st) {
  const size_t qbytes = 16 * (size_t)(p.D + 8) * sizeof(bf16);
  if (split) {  // one head per workgroup, its four waves share the keys; LDS: 4 query tiles + the merge area
    const size_t lds = 4 * 16 * (size_t)((p.D + 8 + 1) / 2) * sizeof(float) + 4 * 16 * (size_t)(p.V + 2) * sizeof(float);
    hipLaunchKernelGGL((sink_flash_kernel<NT, true>), dim3(num_work, p.H), dim3(256), lds, st, p, vt, p.H);
    return;
  }
  const int wy = p.H < 4 ? p.H : 4;
  dim3 grid(num_work, (p.H + wy - 1) / wy), block(64 * wy);
  hipLaunchKernelGGL((sink_flash_kernel<NT, false>), grid, block, wy * qbytes, st, p, vt, p.H);
}

}  // namespace
}  // namespace dsse

// work_tile counts tiles of 16 rows; vt: transposed value pages [pages, G, V, kBS], keys permuted inside a page
extern "C" hipError_t dsse_sink_flash(int num_work, const dsse::SinkAttnParams* p, const void* vt, int split,
                                      hipStream_t st) {
  if (num_work <= 0 || p->H <= 0) return hipSuccess;
  if (p->f32 || p->D % 32 || p->V % 16 || p->V > 512 || p->D > 512 || p->H % p->G) return hipErrorInvalidValue;
  if (split && p->V > 128) return hipErrorInvalidValue;  // the merge area has to fit 64 KB of LDS
  if (p->out_rope && p->V % 32) return hipErrorInvalidValue;  // both halves of a rotation pair are whole 16-wide tiles
  const bf16* v = reinterpret_cast<const bf16*>(vt);
  switch (p->V / 16) {
#define DSSE_FLASH_CASE(n) case n: dsse::launch_flash<n>(num_work, *p, v, split, st); break;
    DSSE_FLASH_CASE(1) DSSE_FLASH_CASE(2) DSSE_FLASH_CASE(3) DSSE_FLASH_CASE(4) DSSE_FLASH_CASE(5) DSSE_FLASH_CASE(6)
    DSSE_FLASH_CASE(7) DSSE_FLASH_CASE(8) DSSE_FLASH_CASE(10) DSSE_FLASH_CASE(12) DSSE_FLASH_CASE(16)
    DSSE_FLASH_CASE(20) DSSE_FLASH_CASE(24) DSSE_FLASH_CASE(32)
#undef DSSE_FLASH_CASE
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

extern "C" hipError_t dsse_sink_attention(int num_work, const dsse::SinkAttnParams* p, hipStream_t st) {
  if (num_work <= 0 || p->H <= 0) return hipSuccess;
  if (p->D > 512 || p->V > dsse::kMaxV || p->H % p->G) return hipErrorInvalidValue;
  if (p->out_rope && p->V % 2) return hipErrorInvalidValue;
  dim3 grid(num_work, p->H);
  if (p->f32) hipLaunchKernelGGL(dsse::sink_attention_kernel<float>, grid, dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::sink_attention_kernel<bf16>, grid, dim3(256), 0, st, *p);
  return hipGetLastError();
}
