// torch operator registrations (namespace torch.ops.dsse) of the layer-mechanism kernels in api_layers.h: the general
// row-major GEMM, the one-number output norm, latent attention, the gated linear recurrence and the routed experts.
//
// As in bindings.cpp, every op validates device, dtype and the shapes its kernel's grid assumes before launching, and
// launches on torch's current HIP stream (graph-capturable).  The element type (bf16 or fp32) is taken from the
// activations; weights must match it.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <algorithm>
#include <climits>
#include <cstdint>

#include "api_layers.h"

namespace {

using at::Tensor;
using OptTensor = c10::optional<Tensor>;

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define DSSE_CHECK_HIP(expr)                                                             \
  do {                                                                                   \
    hipError_t _e = (expr);                                                              \
    TORCH_CHECK(_e == hipSuccess, "dsse kernel launch failed: ", hipGetErrorString(_e)); \
  } while (0)

void gpu(const Tensor& t, const char* name, bool contiguous = true) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  if (contiguous) TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}
void i32(const Tensor& t, const char* name) {
  gpu(t, name);
  TORCH_CHECK(t.scalar_type() == at::kInt, name, " must be int32");
}
void f32t(const Tensor& t, const char* name, bool contiguous = true) {
  gpu(t, name, contiguous);
  TORCH_CHECK(t.scalar_type() == at::kFloat, name, " must be fp32");
}
// element type flag of an activation / weight pair: 1 = fp32, 0 = bf16
int elem(const Tensor& a, const char* name) {
  TORCH_CHECK(a.scalar_type() == at::kFloat || a.scalar_type() == at::kBFloat16, name, " must be bf16 or fp32");
  return a.scalar_type() == at::kFloat ? 1 : 0;
}
void same(const Tensor& a, const Tensor& b, const char* name) {
  TORCH_CHECK(a.scalar_type() == b.scalar_type(), name, " has dtype ", b.scalar_type(), ", expected ", a.scalar_type());
}

// x [M, K] or [Z, M, K]; w [N, K] or [Z, N, K]; out [M, N] or [Z, M, N]; bias [N] or [Z, N]: strided views with a
// unit innermost stride (a head's or a block's slice of a wider buffer is passed as a view, not copied).
void gemm_rm(const Tensor& x, const Tensor& w, Tensor& out, const OptTensor& bias, int64_t act) {
  gpu(x, "x", false);
  gpu(w, "w", false);
  gpu(out, "out", false);
  const int f32 = elem(x, "x");
  same(x, w, "w");
  TORCH_CHECK(out.scalar_type() == at::kFloat || out.scalar_type() == x.scalar_type(), "out must be fp32 or x's type");
  const bool batched = x.dim() == 3;
  TORCH_CHECK((x.dim() == 2 || x.dim() == 3) && w.dim() == x.dim() && out.dim() == x.dim(), "x, w, out: all 2-D or all 3-D");
  const int o = batched ? 1 : 0;
  const int64_t Z = batched ? x.size(0) : 1;
  const int64_t M = x.size(o), K = x.size(o + 1), N = w.size(o);
  TORCH_CHECK(w.size(o + 1) == K && out.size(o) == M && out.size(o + 1) == N, "gemm_rm shape mismatch");
  if (batched) TORCH_CHECK(w.size(0) == Z && out.size(0) == Z, "gemm_rm batch mismatch");
  TORCH_CHECK(M < (1 << 30) && N < (1 << 30) && K < (1 << 30) && Z <= 65535, "gemm_rm sizes out of range");
  TORCH_CHECK((K == 1 || x.stride(o + 1) == 1) && (K == 1 || w.stride(o + 1) == 1) && (N == 1 || out.stride(o + 1) == 1),
              "gemm_rm needs unit innermost strides");
  dsse::GemmRmParams p{};
  p.x = x.data_ptr();
  p.w = w.data_ptr();
  p.out = out.data_ptr();
  p.M = (int)M, p.N = (int)N, p.K = (int)K, p.batch = (int)Z;
  p.ldx = (int)x.stride(o), p.ldw = (int)w.stride(o), p.ldo = (int)out.stride(o);
  p.xbs = batched ? x.stride(0) : 0, p.wbs = batched ? w.stride(0) : 0, p.obs = batched ? out.stride(0) : 0;
  if (bias.has_value()) {
    gpu(*bias, "bias", false);
    same(x, *bias, "bias");
    TORCH_CHECK(bias->dim() == (batched ? 2 : 1) && bias->size(-1) == N && (N == 1 || bias->stride(-1) == 1), "bias shape");
    p.bias = bias->data_ptr();
    p.bbs = batched ? bias->stride(0) : 0;
  }
  TORCH_CHECK(act == 0 || act == 1, "act: 0 none, 1 gelu");
  p.act = (int)act;
  p.out_f32 = out.scalar_type() == at::kFloat;
  p.f32 = f32;
  const int per = f32 ? 4 : 8;
  auto aligned = [&](const Tensor& t, int64_t ld, int64_t bs) {
    return reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0 && ld % per == 0 && bs % per == 0;
  };
  p.vecx = aligned(x, p.ldx, p.xbs);
  p.vecw = aligned(w, p.ldw, p.wbs);
  DSSE_CHECK_HIP(dsse_gemm_rm(&p, cur_stream()));
}

void scalar_norm(const OptTensor& y, const Tensor& g, Tensor& resid, Tensor& xb, double eps, int64_t nsum) {
  f32t(resid, "resid");
  gpu(xb, "xb");
  gpu(g, "g");
  same(xb, g, "g");
  TORCH_CHECK(resid.dim() == 2 && xb.sizes() == resid.sizes() && g.numel() == 1, "scalar_norm shapes");
  dsse::ScalarNormParams p{};
  if (y.has_value()) {
    f32t(*y, "y");
    TORCH_CHECK(nsum >= 1 && y->dim() == 2 && y->size(0) == resid.size(0) * nsum && y->size(1) == resid.size(1),
                "y must be [M * nsum, W]");
    p.y = y->data_ptr<float>();
    p.nsum = (int)nsum;
  }
  p.mode = y.has_value() ? 0 : 1;
  p.g = g.data_ptr();
  p.resid = resid.data_ptr<float>();
  p.xb = xb.data_ptr();
  p.M = (int)resid.size(0), p.W = (int)resid.size(1);
  p.eps = (float)eps;
  p.f32 = elem(xb, "xb");
  DSSE_CHECK_HIP(dsse_scalar_norm(&p, cur_stream()));
}

void embed_rows(const Tensor& ids, const Tensor& embed, Tensor& resid, Tensor& xb) {
  i32(ids, "ids");
  gpu(embed, "embed");
  f32t(resid, "resid");
  gpu(xb, "xb");
  same(embed, xb, "xb");
  const int M = (int)resid.size(0), W = (int)resid.size(1);
  TORCH_CHECK(embed.dim() == 2 && embed.size(1) == W && ids.numel() >= M && xb.sizes() == resid.sizes(), "embed shapes");
  DSSE_CHECK_HIP(dsse_embed_rows(M, W, (int)embed.size(0), ids.data_ptr<int>(), embed.data_ptr(),
                                 resid.data_ptr<float>(), xb.data_ptr(), elem(xb, "xb"), cur_stream()));
}

void latent_kv_write(const Tensor& ckr, const Tensor& norm_w, const Tensor& positions, const Tensor& slots,
                     const Tensor& rope, Tensor& cache, double eps, const OptTensor& vt) {
  f32t(ckr, "ckr", false);
  gpu(norm_w, "norm_w");
  i32(positions, "positions");
  i32(slots, "slots");
  f32t(rope, "rope");
  gpu(cache, "cache");
  same(cache, norm_w, "norm_w");
  TORCH_CHECK(ckr.dim() == 2, "ckr must be [T, rk + dr]");
  const int T = (int)ckr.size(0), D = (int)ckr.size(1), rk = (int)norm_w.numel(), dr = D - rk;
  TORCH_CHECK(dr >= 0 && dr % 2 == 0, "ckr must be [T, rk + dr], dr even");
  TORCH_CHECK((D == 1 || ckr.stride(1) == 1) && (T <= 1 || ckr.stride(0) >= D), "ckr: unit innermost stride, rows apart");
  TORCH_CHECK(cache.dim() == 3 && cache.size(1) == dsse::kBS && cache.size(2) == D, "cache must be [pages, 32, rk + dr]");
  TORCH_CHECK(rope.dim() == 3 && rope.size(1) == dr / 2 && rope.size(2) == 2, "rope must be [P, dr / 2, 2]");
  TORCH_CHECK(positions.numel() >= T && slots.numel() >= T, "metadata too short");
  dsse::LatentKvWriteParams p{};
  p.ckr = ckr.data_ptr<float>();
  p.norm_w = norm_w.data_ptr();
  p.positions = positions.data_ptr<int>();
  p.slots = slots.data_ptr<int>();
  p.rope = reinterpret_cast<const float2*>(rope.data_ptr<float>());
  p.cache = cache.data_ptr();
  p.T = T, p.rk = rk, p.dr = dr, p.rope_len = (int)rope.size(0);
  p.ld = T > 1 ? (int)ckr.stride(0) : D;
  p.num_slots = (int)(cache.size(0) * dsse::kBS);
  p.eps = (float)eps;
  p.f32 = elem(cache, "cache");
  void* vtp = nullptr;
  if (vt.has_value()) {
    gpu(*vt, "vt");
    same(cache, *vt, "vt");
    TORCH_CHECK(vt->dim() == 3 && vt->size(0) == cache.size(0) && vt->size(1) == rk && vt->size(2) == dsse::kBS,
                "vt must be [pages, rk, 32]");
    vtp = vt->data_ptr();
  }
  DSSE_CHECK_HIP(dsse_latent_kv_write(&p, vtp, cur_stream()));
}

void latent_attention(const Tensor& q, const Tensor& q_abs, const Tensor& cache, const Tensor& block_tables,
                      const Tensor& q_start, const Tensor& q_len, const Tensor& ctx_len, const Tensor& work_seq,
                      const Tensor& work_tile, const Tensor& rope, Tensor& out, int64_t window, double scale,
                      int64_t qt, const OptTensor& vt, int64_t hp, const OptTensor& part, int64_t nparts) {
  gpu(q, "q");
  f32t(q_abs, "q_abs");
  gpu(cache, "cache");
  gpu(out, "out");
  same(q, cache, "cache");
  same(q, out, "out");
  i32(block_tables, "block_tables");
  i32(q_start, "q_start");
  i32(q_len, "q_len");
  i32(ctx_len, "ctx_len");
  i32(work_seq, "work_seq");
  i32(work_tile, "work_tile");
  f32t(rope, "rope");
  TORCH_CHECK(q.dim() == 3 && q_abs.dim() == 3 && out.dim() == 3, "q [T, H, dn + dr], q_abs / out [T, H, rk]");
  const int T = (int)q.size(0), H = (int)q.size(1), rk = (int)q_abs.size(2);
  const int D = (int)cache.size(2), dr = D - rk, dn = (int)q.size(2) - dr;
  TORCH_CHECK(cache.dim() == 3 && cache.size(1) == dsse::kBS && dr >= 0 && dr % 2 == 0 && dn >= 0, "cache / q widths");
  TORCH_CHECK(q_abs.size(0) == T && q_abs.size(1) == H && out.sizes() == q_abs.sizes(), "q_abs / out shapes");
  TORCH_CHECK(rope.dim() == 3 && rope.size(1) == dr / 2 && rope.size(2) == 2, "rope must be [P, dr / 2, 2]");
  TORCH_CHECK(block_tables.dim() == 2, "block_tables must be [seqs, max_blocks]");
  const int ns = (int)block_tables.size(0);
  TORCH_CHECK(q_start.numel() >= ns && q_len.numel() >= ns && ctx_len.numel() >= ns, "sequence metadata too short");
  TORCH_CHECK(work_tile.numel() == work_seq.numel(), "work lists differ in length");
  TORCH_CHECK(window >= 1 && qt >= 1 && rk <= 1024, "window >= 1, qt >= 1, rk <= 1024");
  dsse::LatentAttnParams p{};
  p.q = q.data_ptr();
  p.q_abs = q_abs.data_ptr<float>();
  p.cache = cache.data_ptr();
  p.block_tables = block_tables.data_ptr<int>();
  p.max_blocks = (int)block_tables.size(1);
  p.num_blocks = (int)cache.size(0);
  p.q_start = q_start.data_ptr<int>();
  p.q_len = q_len.data_ptr<int>();
  p.ctx_len = ctx_len.data_ptr<int>();
  p.work_seq = work_seq.data_ptr<int>();
  p.work_tile = work_tile.data_ptr<int>();
  p.rope = reinterpret_cast<const float2*>(rope.data_ptr<float>());
  p.out = out.data_ptr();
  p.H = H, p.dn = dn, p.dr = dr, p.rk = rk, p.window = (int)std::min<int64_t>(window, INT_MAX), p.qt = (int)qt;
  p.rope_len = (int)rope.size(0);
  p.scale = (float)scale;
  p.f32 = elem(q, "q");
  if (vt.has_value()) {
    // MFMA form: work_tile counts tiles of qt rows, hp heads side by side, qt * hp = 16 columns
    gpu(*vt, "vt");
    TORCH_CHECK(q.scalar_type() == at::kBFloat16 && vt->scalar_type() == at::kBFloat16, "the MFMA form is bf16");
    TORCH_CHECK(vt->dim() == 3 && vt->size(0) == cache.size(0) && vt->size(1) == rk && vt->size(2) == dsse::kBS,
                "vt must be [pages, rk, 32]");
    TORCH_CHECK(qt * hp == 16 && (rk == 64 || rk == 128 || rk == 256 || rk == 512) && dr % 32 == 0,
                "the MFMA form needs qt * hp = 16, rk in {64, 128, 256, 512}, dr % 32 == 0");
    if (nparts > 1) {
      TORCH_CHECK(part.has_value(), "a key split needs the part scratch");
      f32t(*part, "part");
      const int64_t need = (int64_t)work_seq.numel() * ((H + hp - 1) / hp) * nparts * 16 * (rk + 2);
      TORCH_CHECK(part->numel() >= need && nparts <= 64, "part scratch too small: ", part->numel(), " < ", need);
      p.part = part->data_ptr<float>();
      p.nparts = (int)nparts;
    }
    DSSE_CHECK_HIP(dsse_latent_flash((int)work_seq.numel(), &p, vt->data_ptr(), (int)qt, (int)hp, cur_stream()));
    return;
  }
  DSSE_CHECK_HIP(dsse_latent_attention((int)work_seq.numel(), &p, cur_stream()));
}

void seq_meta(const Tensor& q_start, const Tensor& q_len, const Tensor& ctx_len, const Tensor& state_slot, int& nseq) {
  i32(q_start, "q_start");
  i32(q_len, "q_len");
  i32(ctx_len, "ctx_len");
  i32(state_slot, "state_slot");
  nseq = (int)q_len.numel();
  TORCH_CHECK(q_start.numel() >= nseq && ctx_len.numel() >= nseq && state_slot.numel() >= nseq && nseq <= 65535,
              "sequence metadata too short");
}

void conv_state(const Tensor& in, const Tensor& taps, const OptTensor& bias, const OptTensor& tail, const Tensor& q_start,
                const Tensor& q_len, const Tensor& ctx_len, const Tensor& state_slot, const OptTensor& out,
                const OptTensor& out_b, const OptTensor& in_bias, int64_t act, bool single) {
  gpu(in, "in", false);
  TORCH_CHECK(in.scalar_type() == at::kFloat, "in must be fp32");
  gpu(taps, "taps");
  dsse::ConvStateParams p{};
  seq_meta(q_start, q_len, ctx_len, state_slot, p.nseq);
  TORCH_CHECK(in.dim() == 2 && taps.dim() == 2, "in must be [T, C], taps [C, K]");
  const int C = (int)in.size(1), K = (int)taps.size(1);
  TORCH_CHECK(taps.size(0) == C && K >= 1, "taps must be [C, K]");
  TORCH_CHECK(C == 1 || in.stride(1) == 1, "in needs a unit innermost stride");
  if (out.has_value()) {
    f32t(*out, "out");
    TORCH_CHECK(out->sizes() == in.sizes(), "out must match in");
    p.out = out->data_ptr<float>();
  }
  TORCH_CHECK(out.has_value() || out_b.has_value(), "conv_state needs out or out_b");
  if (out_b.has_value()) {
    gpu(*out_b, "out_b");
    same(taps, *out_b, "out_b");
    TORCH_CHECK(out_b->sizes() == in.sizes(), "out_b must match in");
    p.out_b = out_b->data_ptr();
  }
  if (K > 1) {
    TORCH_CHECK(tail.has_value(), "a convolution with more than one tap needs its tail");
    f32t(*tail, "tail");
    TORCH_CHECK(tail->dim() == 3 && tail->size(1) == K - 1 && tail->size(2) == C, "tail must be [slots, K - 1, C]");
    p.tail = tail->data_ptr<float>();
  }
  if (bias.has_value()) {
    gpu(*bias, "bias");
    same(taps, *bias, "bias");
    TORCH_CHECK(bias->numel() == C, "bias must be [C]");
    p.bias = bias->data_ptr();
  }
  p.in = in.data_ptr<float>();
  p.taps = taps.data_ptr();
  p.q_start = q_start.data_ptr<int>();
  p.q_len = q_len.data_ptr<int>();
  p.ctx_len = ctx_len.data_ptr<int>();
  p.state_slot = state_slot.data_ptr<int>();
  p.single = single ? 1 : 0;
  if (in_bias.has_value()) {
    gpu(*in_bias, "in_bias");
    same(taps, *in_bias, "in_bias");
    TORCH_CHECK(in_bias->numel() == C, "in_bias must be [C]");
    p.in_bias = in_bias->data_ptr();
  }
  p.C = C, p.K = K, p.rows = (int)in.size(0);
  p.ld_in = (int)in.stride(0);
  TORCH_CHECK(act >= 0 && act <= 2, "act: 0 none, 1 SiLU, 2 plus the input");
  p.act = (int)act;
  TORCH_CHECK(p.nseq <= 65535 && (p.rows + 7) / 8 <= 65535, "conv_state: grid too large");
  p.f32 = elem(taps, "taps");
  DSSE_CHECK_HIP(dsse_conv_state(&p, cur_stream()));
}

void lru_scan(const Tensor& u, Tensor& gates, const Tensor& y, const Tensor& lam, Tensor& state,
              const Tensor& q_start, const Tensor& q_len, const Tensor& ctx_len, const Tensor& state_slot, Tensor& out,
              double c, const OptTensor& y_bias, bool coeff, const OptTensor& scratch) {
  f32t(u, "u");
  f32t(gates, "gates");
  f32t(y, "y");
  gpu(lam, "lam");
  f32t(state, "state");
  gpu(out, "out");
  same(lam, out, "out");
  dsse::LruScanParams p{};
  seq_meta(q_start, q_len, ctx_len, state_slot, p.nseq);
  const int C = (int)u.size(1);
  TORCH_CHECK(u.dim() == 2 && gates.dim() == 3 && gates.size(0) == u.size(0) && gates.size(1) * gates.size(2) == 2 * C,
              "gates must be [T, blocks, 2 * C / blocks]");
  TORCH_CHECK(y.sizes() == u.sizes() && out.sizes() == u.sizes() && lam.numel() == C, "y / out / lam shapes");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == C, "state must be [slots, C]");
  p.u = u.data_ptr<float>();
  p.gates = gates.data_ptr<float>();
  p.y = y.data_ptr<float>();
  if (y_bias.has_value()) {
    gpu(*y_bias, "y_bias");
    same(lam, *y_bias, "y_bias");
    TORCH_CHECK(y_bias->numel() == C, "y_bias must be [C]");
    p.y_bias = y_bias->data_ptr();
  }
  p.rows = (int)u.size(0);
  p.coeff = coeff ? 1 : 0;
  if (scratch.has_value()) {  // [2, slots, C] with slots >= rows / 32 + sequences + 1: the chunked walk's scratch
    f32t(*scratch, "scratch");
    const int64_t slots = p.rows / 32 + p.nseq + 1;
    TORCH_CHECK(scratch->dim() == 3 && scratch->size(0) == 2 && scratch->size(1) >= slots && scratch->size(2) == C,
                "lru_scan scratch must be [2, >= rows / 32 + sequences + 1, C]");
    p.chunk_a = scratch->data_ptr<float>();
    p.chunk_b = p.chunk_a + scratch->size(1) * (int64_t)C;
    TORCH_CHECK((p.rows + 31) / 32 <= 65535, "lru_scan: too many rows");
  }
  p.lam = lam.data_ptr();
  p.state = state.data_ptr<float>();
  p.q_start = q_start.data_ptr<int>();
  p.q_len = q_len.data_ptr<int>();
  p.ctx_len = ctx_len.data_ptr<int>();
  p.state_slot = state_slot.data_ptr<int>();
  p.out = out.data_ptr();
  p.C = C, p.bw = (int)gates.size(2) / 2;
  p.c = (float)c;
  p.f32 = elem(lam, "lam");
  DSSE_CHECK_HIP(dsse_lru_scan(&p, cur_stream()));
}

void moe_router(const Tensor& x, const Tensor& w, const OptTensor& b, Tensor& topk_idx, Tensor& topk_w) {
  gpu(x, "x");
  gpu(w, "w");
  same(x, w, "w");
  i32(topk_idx, "topk_idx");
  f32t(topk_w, "topk_w");
  dsse::MoeRouterParams p{};
  p.M = (int)x.size(0), p.W = (int)x.size(1), p.E = (int)w.size(0), p.top = (int)topk_idx.size(1);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && w.size(1) == p.W && topk_idx.dim() == 2 && topk_idx.size(0) == p.M &&
                  topk_w.sizes() == topk_idx.sizes() && p.top >= 1 && p.top <= p.E && p.E <= 8192,
              "router shapes");
  if (b.has_value()) {
    gpu(*b, "b");
    same(x, *b, "b");
    TORCH_CHECK(b->numel() == p.E, "router bias must be [E]");
    p.b = b->data_ptr();
  }
  p.x = x.data_ptr();
  p.w = w.data_ptr();
  p.topk_idx = topk_idx.data_ptr<int>();
  p.topk_w = topk_w.data_ptr<float>();
  p.f32 = elem(x, "x");
  DSSE_CHECK_HIP(dsse_moe_router(&p, cur_stream()));
}

void moe_ffn(const Tensor& x, const Tensor& topk_idx, const Tensor& topk_w, const Tensor& gate, const Tensor& up,
             const Tensor& down, const OptTensor& sgate, const OptTensor& sup, const OptTensor& sdown, Tensor& out) {
  gpu(x, "x");
  i32(topk_idx, "topk_idx");
  f32t(topk_w, "topk_w");
  gpu(gate, "gate");
  gpu(up, "up");
  gpu(down, "down");
  f32t(out, "out");
  same(x, gate, "gate");
  same(x, up, "up");
  same(x, down, "down");
  dsse::MoeFfnParams p{};
  p.M = (int)x.size(0), p.W = (int)x.size(1);
  TORCH_CHECK(gate.dim() == 3 && gate.size(2) == p.W && up.sizes() == gate.sizes(), "gate / up must be [E, F, W]");
  p.E = (int)gate.size(0), p.F = (int)gate.size(1), p.top = (int)topk_idx.size(1);
  TORCH_CHECK(down.dim() == 3 && down.size(0) == p.E && down.size(1) == p.W && down.size(2) == p.F, "down must be [E, W, F]");
  TORCH_CHECK(topk_idx.size(0) == p.M && topk_w.sizes() == topk_idx.sizes() && out.sizes() == x.sizes(), "row shapes");
  if (sgate.has_value()) {
    TORCH_CHECK(sup.has_value() && sdown.has_value(), "the shared expert needs gate, up and down");
    gpu(*sgate, "sgate");
    gpu(*sup, "sup");
    gpu(*sdown, "sdown");
    same(x, *sgate, "sgate");
    same(x, *sup, "sup");
    same(x, *sdown, "sdown");
    p.Fs = (int)sgate->size(0);
    TORCH_CHECK(sgate->dim() == 2 && sgate->size(1) == p.W && sup->sizes() == sgate->sizes() && sdown->dim() == 2 &&
                    sdown->size(0) == p.W && sdown->size(1) == p.Fs,
                "shared expert shapes");
    p.sgate = sgate->data_ptr();
    p.sup = sup->data_ptr();
    p.sdown = sdown->data_ptr();
  }
  TORCH_CHECK(sizeof(float) * (2 * (size_t)p.W + std::max(p.F, p.Fs)) <= 64 * 1024, "moe_ffn: row does not fit the LDS");
  p.x = x.data_ptr();
  p.topk_idx = topk_idx.data_ptr<int>();
  p.topk_w = topk_w.data_ptr<float>();
  p.gate = gate.data_ptr();
  p.up = up.data_ptr();
  p.down = down.data_ptr();
  p.out = out.data_ptr<float>();
  p.f32 = elem(x, "x");
  DSSE_CHECK_HIP(dsse_moe_ffn(&p, cur_stream()));
}

// Grouped form of the routed experts: o [M * S, W] (fp32) = per-(row, slot) expert outputs times their weights, S = top
// (+ 1 with a shared expert); the caller sums a row's S parts (scalar_norm nsum).  Scratch: sorted [tiles * 64],
// tile_expert [tiles], num_tiles [1] (int32), h [M * S, ldh] (element type), tiles >= ceil(M S / 64) + experts + 1.
void moe_grouped(const Tensor& x, const Tensor& topk_idx, const Tensor& topk_w, const OptTensor& gate, const Tensor& up,
                 const Tensor& down, const OptTensor& sgate, const OptTensor& sup, const OptTensor& sdown, Tensor& sorted,
                 Tensor& tile_expert, Tensor& num_tiles, Tensor& h, Tensor& o) {
  gpu(x, "x");
  i32(topk_idx, "topk_idx");
  f32t(topk_w, "topk_w");
  gpu(up, "up");
  gpu(down, "down");
  i32(sorted, "sorted");
  i32(tile_expert, "tile_expert");
  i32(num_tiles, "num_tiles");
  gpu(h, "h");
  f32t(o, "o");
  same(x, up, "up");
  same(x, down, "down");
  same(x, h, "h");
  dsse::MoeGroupedParams p{};
  p.M = (int)x.size(0), p.W = (int)x.size(1);
  TORCH_CHECK(x.dim() == 2 && up.dim() == 3 && up.size(2) == p.W, "up must be [E, F, W]");
  if (gate.has_value()) {
    gpu(*gate, "gate");
    same(x, *gate, "gate");
    TORCH_CHECK(gate->sizes() == up.sizes(), "gate must be [E, F, W] like up");
  } else {
    TORCH_CHECK(!sgate.has_value(), "experts without a gate have no shared expert");
  }
  p.E = (int)up.size(0), p.F = (int)up.size(1), p.top = (int)topk_idx.size(1);
  TORCH_CHECK(down.dim() == 3 && down.size(0) == p.E && down.size(1) == p.W && down.size(2) == p.F, "down must be [E, W, F]");
  TORCH_CHECK(topk_idx.dim() == 2 && topk_idx.size(0) == p.M && topk_w.sizes() == topk_idx.sizes(), "routing shapes");
  p.S = p.top;
  if (sgate.has_value()) {
    TORCH_CHECK(sup.has_value() && sdown.has_value(), "the shared expert needs gate, up and down");
    gpu(*sgate, "sgate");
    gpu(*sup, "sup");
    gpu(*sdown, "sdown");
    same(x, *sgate, "sgate");
    same(x, *sup, "sup");
    same(x, *sdown, "sdown");
    p.Fs = (int)sgate->size(0);
    TORCH_CHECK(sgate->dim() == 2 && sgate->size(1) == p.W && sup->sizes() == sgate->sizes() && sdown->dim() == 2 &&
                    sdown->size(0) == p.W && sdown->size(1) == p.Fs,
                "shared expert shapes");
    p.sgate = sgate->data_ptr();
    p.sup = sup->data_ptr();
    p.sdown = sdown->data_ptr();
    p.S = p.top + 1;
  }
  const int64_t ids = (int64_t)p.M * p.S;
  p.max_tiles = (int)tile_expert.numel();
  TORCH_CHECK(p.max_tiles >= (ids + 63) / 64 + p.E + 1 && sorted.numel() >= (int64_t)p.max_tiles * 64 && p.max_tiles <= 65535,
              "moe_grouped: scratch too small for ", ids, " ids");
  TORCH_CHECK(h.dim() == 2 && h.size(0) >= ids && h.size(1) >= std::max(p.F, p.Fs) && o.dim() == 2 && o.size(0) == ids &&
                  o.size(1) == p.W && p.E + 1 <= 4096,
              "moe_grouped: h / o shapes");
  p.ldh = (int)h.size(1);
  p.x = x.data_ptr();
  p.topk_idx = topk_idx.data_ptr<int>();
  p.topk_w = topk_w.data_ptr<float>();
  p.gate = gate.has_value() ? gate->data_ptr() : nullptr;
  p.up = up.data_ptr();
  p.down = down.data_ptr();
  p.sorted = sorted.data_ptr<int>();
  p.tile_expert = tile_expert.data_ptr<int>();
  p.num_tiles = num_tiles.data_ptr<int>();
  p.h = h.data_ptr();
  p.o = o.data_ptr<float>();
  p.f32 = elem(x, "x");
  const int per = p.f32 ? 4 : 8;
  p.vec_w = p.W % per == 0;
  p.vec_h = p.ldh % per == 0 && p.F % per == 0;
  p.lds_tiles = ids >= 256;  // prompt-sized: most 64-row tiles are full
  DSSE_CHECK_HIP(dsse_moe_grouped(&p, cur_stream()));
}

void moe_topk(const Tensor& logits, Tensor& topk_idx, Tensor& topk_w) {
  f32t(logits, "logits");
  i32(topk_idx, "topk_idx");
  f32t(topk_w, "topk_w");
  const int M = (int)logits.size(0), E = (int)logits.size(1), top = (int)topk_idx.size(1);
  TORCH_CHECK(logits.dim() == 2 && topk_idx.dim() == 2 && topk_idx.size(0) == M && topk_w.sizes() == topk_idx.sizes() &&
                  top >= 1 && top <= E,
              "moe_topk shapes");
  DSSE_CHECK_HIP(dsse_moe_topk(logits.data_ptr<float>(), M, E, top, topk_idx.data_ptr<int>(), topk_w.data_ptr<float>(),
                               cur_stream()));
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(dsse, m) {
  m.def("gemm_rm(Tensor x, Tensor w, Tensor(a!) out, Tensor? bias=None, int act=0) -> ()");
  m.def("scalar_norm(Tensor? y, Tensor g, Tensor(a!) resid, Tensor(b!) xb, float eps, int nsum=1) -> ()");
  m.def("moe_grouped(Tensor x, Tensor topk_idx, Tensor topk_w, Tensor? gate, Tensor up, Tensor down, Tensor? sgate, "
        "Tensor? sup, Tensor? sdown, Tensor(a!) sorted, Tensor(b!) tile_expert, Tensor(c!) num_tiles, Tensor(d!) h, "
        "Tensor(e!) o) -> ()");
  m.def("embed_rows(Tensor ids, Tensor embed, Tensor(a!) resid, Tensor(b!) xb) -> ()");
  m.def("latent_kv_write(Tensor ckr, Tensor norm_w, Tensor positions, Tensor slots, Tensor rope, Tensor(a!) cache, "
        "float eps, Tensor(b!)? vt=None) -> ()");
  m.def("latent_attention(Tensor q, Tensor q_abs, Tensor cache, Tensor block_tables, Tensor q_start, Tensor q_len, "
        "Tensor ctx_len, Tensor work_seq, Tensor work_tile, Tensor rope, Tensor(a!) out, int window, float scale, "
        "int qt, Tensor? vt=None, int hp=1, Tensor(b!)? part=None, int nparts=1) -> ()");
  m.def("conv_state(Tensor inp, Tensor taps, Tensor? bias, Tensor(a!)? tail, Tensor q_start, Tensor q_len, "
        "Tensor ctx_len, Tensor state_slot, Tensor(b!)? out, Tensor(c!)? out_b, Tensor? in_bias=None, int act=0, "
        "bool single=False) -> ()");
  m.def("lru_scan(Tensor u, Tensor(c!) gates, Tensor y, Tensor lam, Tensor(a!) state, Tensor q_start, Tensor q_len, "
        "Tensor ctx_len, Tensor state_slot, Tensor(b!) out, float c, Tensor? y_bias=None, bool coeff=True, "
        "Tensor(d!)? scratch=None) -> ()");
  m.def("moe_router(Tensor x, Tensor w, Tensor? b, Tensor(a!) topk_idx, Tensor(b!) topk_w) -> ()");
  m.def("moe_topk(Tensor logits, Tensor(a!) topk_idx, Tensor(b!) topk_w) -> ()");
  m.def("moe_ffn(Tensor x, Tensor topk_idx, Tensor topk_w, Tensor gate, Tensor up, Tensor down, Tensor? sgate, "
        "Tensor? sup, Tensor? sdown, Tensor(a!) out) -> ()");
}

TORCH_LIBRARY_IMPL(dsse, CUDA, m) {
  m.impl("gemm_rm", &gemm_rm);
  m.impl("scalar_norm", &scalar_norm);
  m.impl("embed_rows", &embed_rows);
  m.impl("latent_kv_write", &latent_kv_write);
  m.impl("latent_attention", &latent_attention);
  m.impl("conv_state", &conv_state);
  m.impl("lru_scan", &lru_scan);
  m.impl("moe_router", &moe_router);
  m.impl("moe_topk", &moe_topk);
  m.impl("moe_ffn", &moe_ffn);
  m.impl("moe_grouped", &moe_grouped);
}
