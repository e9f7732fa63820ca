// torch operator registrations (namespace torch.ops.dsse) of the kernels in api_mixers.h: the residual stream's step
// with the element-wise tanh norm, the gated activation, per-row norms with rotation, softmax attention with a sink
// over paged keys and values, gate math, the matrix-state recurrence, the gated per-head output norm, the normed mix
// of two mixers and the logit cap.
//
// As in the other binding files, every op validates device, dtype and the shapes and strides its kernel's indexing
// assumes before launching, and launches on torch's current HIP stream (graph-capturable).  Column slices of wider
// fp32 buffers are passed as views (unit innermost stride); nothing is copied here.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <algorithm>
#include <climits>
#include <cstdint>

#include "api_mixers.h"

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
int elem(const Tensor& a, const char* name) {
  TORCH_CHECK(a.scalar_type() == at::kFloat || a.scalar_type() == at::kBFloat16, name, " must be bf16 or fp32");
  return a.scalar_type() == at::kFloat ? 1 : 0;
}
const float* opt_f32(const OptTensor& t, const char* name, int64_t numel) {
  if (!t.has_value()) return nullptr;
  f32t(*t, name);
  TORCH_CHECK(t->numel() == numel, name, " must hold ", numel, " numbers");
  return t->data_ptr<float>();
}
// a [rows, heads, width] fp32 view whose heads are adjacent columns of a row-major buffer
void head_view(const Tensor& t, const char* name) {
  f32t(t, name, false);
  TORCH_CHECK(t.dim() == 3 && (t.size(2) == 1 || t.stride(2) == 1) && (t.size(1) == 1 || t.stride(1) == t.size(2)),
              name, " must be [rows, heads, width] with adjacent heads");
  TORCH_CHECK(t.stride(0) >= t.size(1) * t.size(2), name, ": rows overlap");
}
// a [rows, cols] fp32 view with a unit innermost stride
void col_view(const Tensor& t, const char* name) {
  f32t(t, name, false);
  TORCH_CHECK(t.dim() == 2 && (t.size(1) == 1 || t.stride(1) == 1) && t.stride(0) >= t.size(1), name,
              " must be [rows, cols] with a unit innermost stride");
}
void seq_meta(const Tensor& q_start, const Tensor& q_len, const Tensor& ctx_len, int ns) {
  i32(q_start, "q_start");
  i32(q_len, "q_len");
  i32(ctx_len, "ctx_len");
  TORCH_CHECK(q_start.numel() >= ns && q_len.numel() >= ns && ctx_len.numel() >= ns, "sequence metadata too short");
}

void stream_step(const OptTensor& y, double mult, Tensor& resid, const OptTensor& ids, const OptTensor& embed,
                 const OptTensor& vec, const OptTensor& alpha, const OptTensor& w, const OptTensor& b,
                 const OptTensor& xb) {
  f32t(resid, "resid");
  TORCH_CHECK(resid.dim() == 2, "resid must be [M, W]");
  dsse::StreamStepParams p{};
  p.M = (int)resid.size(0), p.W = (int)resid.size(1);
  p.resid = resid.data_ptr<float>();
  p.mult = (float)mult;
  p.f32 = 1;
  if (y.has_value()) {
    f32t(*y, "y");
    TORCH_CHECK(y->sizes() == resid.sizes(), "y must match resid");
    p.y = y->data_ptr<float>();
  }
  if (embed.has_value()) {
    TORCH_CHECK(ids.has_value(), "embed needs ids");
    i32(*ids, "ids");
    gpu(*embed, "embed");
    TORCH_CHECK(embed->dim() == 2 && embed->size(1) == p.W && ids->numel() >= p.M, "embed must be [vocab, W]");
    p.ids = ids->data_ptr<int>();
    p.embed = embed->data_ptr();
    p.vocab = (int)embed->size(0);
    p.f32 = elem(*embed, "embed");
  }
  p.vec = opt_f32(vec, "vec", p.W);
  if (w.has_value()) {
    TORCH_CHECK(alpha.has_value() && b.has_value() && xb.has_value(), "a norm needs alpha, w, b and xb");
    p.alpha = opt_f32(alpha, "alpha", 1);
    p.w = opt_f32(w, "w", p.W);
    p.b = opt_f32(b, "b", p.W);
    gpu(*xb, "xb");
    TORCH_CHECK(xb->sizes() == resid.sizes(), "xb must match resid");
    const int f = elem(*xb, "xb");
    TORCH_CHECK(!embed.has_value() || f == p.f32, "embed and xb differ in type");
    p.f32 = f;
    p.xb = xb->data_ptr();
  }
  DSSE_CHECK_HIP(dsse_stream_step(&p, cur_stream()));
}

void gated_act(const Tensor& gu, Tensor& h, int64_t kind) {
  col_view(gu, "gu");
  gpu(h, "h");
  TORCH_CHECK(h.dim() == 2 && gu.size(0) == h.size(0) && gu.size(1) == 2 * h.size(1), "gu must be [M, 2 F], h [M, F]");
  TORCH_CHECK(kind == 0 || kind == 1, "kind: 0 SiLU, 1 gelu");
  DSSE_CHECK_HIP(dsse_gated_act(gu.data_ptr<float>(), (int)gu.stride(0), h.data_ptr(), (int)h.size(0), (int)h.size(1),
                                (int)kind, elem(h, "h"), cur_stream()));
}

void norm_rope_rows(const Tensor& x, const OptTensor& norm_w, const Tensor& positions, const OptTensor& rope, Tensor& out,
                    const OptTensor& out_rows, int64_t kind, double eps, double scale, const OptTensor& out_t) {
  head_view(x, "x");
  dsse::NormRopeParams p{};
  p.T = (int)x.size(0), p.nh = (int)x.size(1), p.D = (int)x.size(2);
  p.ldx = (int)x.stride(0);
  p.x = x.data_ptr<float>();
  TORCH_CHECK(kind >= 0 && kind <= 3 && p.D <= 512, "kind 0..3, head width <= 512");
  p.kind = (int)kind;
  p.norm_w = opt_f32(norm_w, "norm_w", kind == 3 ? (int64_t)p.D : (int64_t)p.nh * p.D);
  TORCH_CHECK(kind != 1 || p.norm_w, "kind 1 needs norm_w");
  if (rope.has_value() && rope->numel() > 0) {
    f32t(*rope, "rope");
    i32(positions, "positions");
    TORCH_CHECK(rope->dim() == 3 && rope->size(2) == 2 && 2 * rope->size(1) <= p.D, "rope must be [P, dims / 2, 2]");
    TORCH_CHECK(positions.numel() >= p.T, "positions too short");
    p.rope = reinterpret_cast<const float2*>(rope->data_ptr<float>());
    p.positions = positions.data_ptr<int>();
    p.half = (int)rope->size(1), p.rope_len = (int)rope->size(0);
  }
  gpu(out, "out", false);
  TORCH_CHECK(out.scalar_type() == at::kFloat || out.scalar_type() == at::kBFloat16, "out must be fp32 or bf16");
  p.out_f32 = out.scalar_type() == at::kFloat;
  p.out = out.data_ptr();
  if (out_rows.has_value()) {  // out: contiguous rows of [nh, D] (a cache: [pages, page, nh, D])
    i32(*out_rows, "out_rows");
    TORCH_CHECK(out.is_contiguous() && out.dim() >= 3 && out.size(-1) == p.D && out.size(-2) == p.nh,
                "out must be contiguous [..., heads, width]");
    TORCH_CHECK(out_rows->numel() >= p.T, "out_rows too short");
    p.out_rows = out_rows->data_ptr<int>();
    p.ldo = p.nh * p.D;
    p.num_out_rows = (int)(out.numel() / p.ldo);
    if (out_t.has_value()) {  // transposed pages [pages, nh, D, 32] beside the row-major ones
      gpu(*out_t, "out_t");
      TORCH_CHECK(out_t->scalar_type() == out.scalar_type() && out_t->dim() == 4 && out_t->size(1) == p.nh &&
                      out_t->size(2) == p.D && out_t->size(3) == dsse::kBS &&
                      out_t->size(0) * dsse::kBS == p.num_out_rows,
                  "out_t must be [pages, heads, width, 32] over the same pages as out");
      p.out_t = out_t->data_ptr();
    }
  } else {
    TORCH_CHECK(!out_t.has_value(), "out_t needs out_rows");
    TORCH_CHECK(out.dim() == 3 && out.sizes() == x.sizes() && (p.D == 1 || out.stride(2) == 1) &&
                    (p.nh == 1 || out.stride(1) == p.D) && out.stride(0) >= (int64_t)p.nh * p.D,
                "out must be [rows, heads, width] with adjacent heads");
    p.ldo = (int)out.stride(0);
    p.num_out_rows = p.T;
  }
  p.eps = (float)eps, p.scale = (float)scale;
  DSSE_CHECK_HIP(dsse_norm_rope_rows(&p, cur_stream()));
}

void sink_attention(const Tensor& q, const Tensor& kcache, const Tensor& vcache, const Tensor& block_tables,
                    const Tensor& q_start, const Tensor& q_len, const Tensor& ctx_len, const Tensor& work_seq,
                    const Tensor& work_tile, const OptTensor& sink, const OptTensor& gate, Tensor& out, int64_t window,
                    double scale, int64_t qt, const OptTensor& vt, bool split, double softcap, const OptTensor& out_rope) {
  f32t(q, "q");
  gpu(kcache, "kcache");
  gpu(vcache, "vcache");
  gpu(out, "out");
  TORCH_CHECK(kcache.scalar_type() == vcache.scalar_type() && out.scalar_type() == kcache.scalar_type(),
              "kcache, vcache and out share the element type");
  i32(block_tables, "block_tables");
  i32(work_seq, "work_seq");
  i32(work_tile, "work_tile");
  TORCH_CHECK(q.dim() == 3 && kcache.dim() == 4 && vcache.dim() == 4 && out.dim() == 3, "q [T, H, D], caches 4-D");
  dsse::SinkAttnParams p{};
  const int T = (int)q.size(0);
  p.H = (int)q.size(1), p.D = (int)q.size(2), p.G = (int)kcache.size(2), p.V = (int)vcache.size(3);
  TORCH_CHECK(kcache.size(1) == dsse::kBS && vcache.size(1) == dsse::kBS && kcache.size(3) == p.D &&
                  vcache.size(2) == p.G && vcache.size(0) == kcache.size(0),
              "caches must be [pages, 32, G, D] and [pages, 32, G, V]");
  TORCH_CHECK(p.G >= 1 && p.H % p.G == 0 && p.D <= 512 && p.V <= 512, "heads must be a multiple of kv heads, widths <= 512");
  TORCH_CHECK(out.size(0) == T && out.size(1) == p.H && out.size(2) == p.V, "out must be [T, H, V]");
  TORCH_CHECK(block_tables.dim() == 2, "block_tables must be [seqs, max_blocks]");
  const int ns = (int)block_tables.size(0);
  seq_meta(q_start, q_len, ctx_len, ns);
  TORCH_CHECK(work_tile.numel() == work_seq.numel() && window >= 1 && qt >= 1, "work lists, window >= 1, qt >= 1");
  TORCH_CHECK(kcache.size(0) * dsse::kBS * p.G < INT_MAX, "cache rows out of range");
  p.q = q.data_ptr<float>();
  p.k = kcache.data_ptr();
  p.v = vcache.data_ptr();
  p.block_tables = block_tables.data_ptr<int>();
  p.max_blocks = (int)block_tables.size(1);
  p.num_blocks = (int)kcache.size(0);
  p.q_start = q_start.data_ptr<int>();
  p.q_len = q_len.data_ptr<int>();
  p.ctx_len = ctx_len.data_ptr<int>();
  p.work_seq = work_seq.data_ptr<int>();
  p.work_tile = work_tile.data_ptr<int>();
  p.sink = opt_f32(sink, "sink", p.H);
  if (gate.has_value()) {
    col_view(*gate, "gate");
    TORCH_CHECK(gate->size(0) == T && gate->size(1) == p.H, "gate must be [T, H]");
    p.gate = gate->data_ptr<float>();
    p.ldg = (int)gate->stride(0);
  }
  p.out = out.data_ptr();
  p.window = (int)std::min<int64_t>(window, INT_MAX), p.qt = (int)qt;
  p.scale = (float)scale;
  p.f32 = elem(kcache, "kcache");
  TORCH_CHECK(softcap >= 0, "softcap >= 0");
  p.softcap = (float)softcap;
  if (out_rope.has_value()) {
    f32t(*out_rope, "out_rope");
    TORCH_CHECK(out_rope->dim() == 3 && out_rope->size(2) == 2 && 2 * out_rope->size(1) == p.V && out_rope->size(0) >= 1,
                "out_rope must be [P, V / 2, 2]");
    TORCH_CHECK(!vt.has_value() || p.V % 32 == 0, "the MFMA form turns outputs back only for V % 32 == 0");
    p.out_rope = reinterpret_cast<const float2*>(out_rope->data_ptr<float>());
    p.out_rope_len = (int)out_rope->size(0);
  }
  if (vt.has_value()) {  // MFMA form: work_tile counts tiles of 16 rows
    gpu(*vt, "vt");
    TORCH_CHECK(kcache.scalar_type() == at::kBFloat16 && vt->scalar_type() == at::kBFloat16, "the MFMA form is bf16");
    TORCH_CHECK(vt->dim() == 4 && vt->size(0) == vcache.size(0) && vt->size(1) == p.G && vt->size(2) == p.V &&
                    vt->size(3) == dsse::kBS,
                "vt must be [pages, G, V, 32]");
    TORCH_CHECK(qt == 16 && p.D % 32 == 0 && p.V % 16 == 0, "the MFMA form needs qt = 16, D % 32 == 0, V % 16 == 0");
    TORCH_CHECK(!split || p.V <= 128, "the key split of the MFMA form needs V <= 128");
    DSSE_CHECK_HIP(dsse_sink_flash((int)work_seq.numel(), &p, vt->data_ptr(), split ? 1 : 0, cur_stream()));
    return;
  }
  DSSE_CHECK_HIP(dsse_sink_attention((int)work_seq.numel(), &p, cur_stream()));
}

void gate_math(Tensor& x, int64_t kind, const OptTensor& p1, const OptTensor& p2, double c) {
  col_view(x, "x");
  const int M = (int)x.size(0), N = (int)x.size(1);
  TORCH_CHECK(kind >= 0 && kind <= 2, "kind 0..2");
  // p1 / p2 hold one number per column, or one per run of neighbouring columns
  const int64_t n1 = p1.has_value() ? p1->numel() : N, n2 = p2.has_value() ? p2->numel() : N;
  TORCH_CHECK(n1 >= 1 && n2 >= 1 && N % n1 == 0 && N % n2 == 0, "p1 and p2 must divide the row into equal runs");
  const float* a = opt_f32(p1, "p1", n1);
  const float* b = opt_f32(p2, "p2", n2);
  TORCH_CHECK(kind != 0 || (a && b), "kind 0 needs p1 and p2");
  TORCH_CHECK(kind != 2 || c > 0, "kind 2 needs c > 0");
  DSSE_CHECK_HIP(dsse_gate_math(x.data_ptr<float>(), (int)x.stride(0), M, N, (int)kind, a, (int)(N / n1), b, (int)(N / n2),
                                (float)c, cur_stream()));
}

void matrix_scan(const Tensor& q, const Tensor& k, const Tensor& v, const OptTensor& decay, const OptTensor& beta,
                 Tensor& state, const Tensor& q_start, const Tensor& q_len, const Tensor& ctx_len,
                 const Tensor& state_slot, Tensor& out, double q_scale) {
  head_view(q, "q");
  head_view(k, "k");
  head_view(v, "v");
  f32t(state, "state");
  f32t(out, "out");
  dsse::MatrixScanParams p{};
  const int T = (int)v.size(0);
  p.H = (int)v.size(1), p.V = (int)v.size(2), p.G = (int)k.size(1), p.D = (int)k.size(2);
  TORCH_CHECK(q.sizes() == k.sizes() && q.size(0) == T && p.G >= 1 && p.H % p.G == 0, "q, k [T, G, D], v [T, H, V]");
  TORCH_CHECK(p.D <= 512, "key width <= 512");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == p.H && state.size(2) == p.D && state.size(3) == p.V,
              "state must be [slots, H, D, V]");
  TORCH_CHECK(out.dim() == 3 && out.sizes() == v.sizes(), "out must be [T, H, V]");
  p.nseq = (int)q_len.numel();
  seq_meta(q_start, q_len, ctx_len, p.nseq);
  i32(state_slot, "state_slot");
  TORCH_CHECK(state_slot.numel() >= p.nseq && p.nseq <= 65535 && p.H <= 65535, "state_slot too short / grid too large");
  p.q = q.data_ptr<float>(), p.k = k.data_ptr<float>(), p.v = v.data_ptr<float>();
  p.ldq = (int)q.stride(0), p.ldk = (int)k.stride(0), p.ldv = (int)v.stride(0);
  if (decay.has_value()) {
    const Tensor& d = *decay;
    f32t(d, "decay", false);
    if (d.dim() == 1) {
      TORCH_CHECK(d.size(0) == p.H && (p.H == 1 || d.stride(0) == 1), "decay [H]");
      p.decay_kind = 1;
    } else if (d.dim() == 2) {
      col_view(d, "decay");
      TORCH_CHECK(d.size(0) == T && d.size(1) == p.H, "decay [T, H]");
      p.decay_kind = 2;
      p.ldd = (int)d.stride(0);
    } else {
      head_view(d, "decay");
      TORCH_CHECK(d.size(0) == T && d.size(1) == p.H && d.size(2) == p.D, "decay [T, H, D]");
      p.decay_kind = 3;
      p.ldd = (int)d.stride(0);
    }
    p.decay = d.data_ptr<float>();
  }
  if (beta.has_value()) {
    col_view(*beta, "beta");
    TORCH_CHECK(beta->size(0) == T && beta->size(1) == p.H, "beta [T, H]");
    p.beta = beta->data_ptr<float>();
    p.ldb = (int)beta->stride(0);
  }
  p.state = state.data_ptr<float>();
  p.q_start = q_start.data_ptr<int>();
  p.q_len = q_len.data_ptr<int>();
  p.ctx_len = ctx_len.data_ptr<int>();
  p.state_slot = state_slot.data_ptr<int>();
  p.out = out.data_ptr<float>();
  p.q_scale = (float)q_scale;
  p.portions = T > 2 * p.nseq;  // more than a row or two per sequence: prompt portions, not a decode step
  DSSE_CHECK_HIP(dsse_matrix_scan(&p, cur_stream()));
}

// Two-level walk of long prompt portions without the delta rule: (1) every chunk but a sequence's last is walked from
// zeros and leaves its end state in `scratch`; (2) the carry turns those into each chunk's incoming state; (3) every
// chunk is walked from its incoming state and writes its outputs, the last chunk of a sequence also the slot's state.
// cmeta [7, chunks]: first row, tokens, tokens in pass 1 (0 for a sequence's last chunk), -1s, pass-1 destination
// (own entry or -1), own entry, pass-3 destination (the state slot for a sequence's last chunk, else -1).
void matrix_scan_chunked(const Tensor& q, const Tensor& k, const Tensor& v, const OptTensor& decay, Tensor& state,
                         const Tensor& q_len, const Tensor& ctx_len, const Tensor& state_slot, const Tensor& s_first,
                         const Tensor& s_count, const Tensor& cmeta, Tensor& scratch, const OptTensor& a_scratch,
                         Tensor& out, double q_scale) {
  head_view(q, "q");
  head_view(k, "k");
  head_view(v, "v");
  f32t(state, "state");
  f32t(out, "out");
  f32t(scratch, "scratch");
  i32(cmeta, "cmeta");
  i32(q_len, "q_len");
  i32(ctx_len, "ctx_len");
  i32(state_slot, "state_slot");
  i32(s_first, "s_first");
  i32(s_count, "s_count");
  dsse::MatrixScanParams p{};
  const int T = (int)v.size(0);
  p.H = (int)v.size(1), p.V = (int)v.size(2), p.G = (int)k.size(1), p.D = (int)k.size(2);
  TORCH_CHECK(q.sizes() == k.sizes() && q.size(0) == T && p.G >= 1 && p.H % p.G == 0 && p.D <= 512, "q, k [T, G, D], v [T, H, V]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == p.H && state.size(2) == p.D && state.size(3) == p.V,
              "state must be [slots, H, D, V]");
  TORCH_CHECK(out.dim() == 3 && out.sizes() == v.sizes(), "out must be [T, H, V]");
  TORCH_CHECK(cmeta.dim() == 2 && cmeta.size(0) == 7, "cmeta must be [7, chunks]");
  const int N = (int)cmeta.size(1), ns = (int)q_len.numel();
  const int64_t entry = (int64_t)p.H * p.D * p.V;
  TORCH_CHECK(scratch.numel() >= N * entry, "scratch must hold [chunks, H, D, V]");
  TORCH_CHECK(ctx_len.numel() >= ns && state_slot.numel() >= ns && s_first.numel() >= ns && s_count.numel() >= ns &&
                  N <= 65535 && ns <= 65535,
              "sequence metadata too short / too many chunks");
  p.q = q.data_ptr<float>(), p.k = k.data_ptr<float>(), p.v = v.data_ptr<float>();
  p.ldq = (int)q.stride(0), p.ldk = (int)k.stride(0), p.ldv = (int)v.stride(0);
  dsse::ScanCarryParams cp{};
  if (decay.has_value()) {
    const Tensor& d = *decay;
    f32t(d, "decay", false);
    if (d.dim() == 1) {
      TORCH_CHECK(d.size(0) == p.H && (p.H == 1 || d.stride(0) == 1), "decay [H]");
      p.decay_kind = 1;
      cp.decay = d.data_ptr<float>();
    } else {
      head_view(d, "decay");
      TORCH_CHECK(d.dim() == 3 && d.size(0) == T && d.size(1) == p.H && d.size(2) == p.D, "decay [T, H, D]");
      TORCH_CHECK(a_scratch.has_value(), "per-channel decays need a_scratch");
      f32t(*a_scratch, "a_scratch");
      TORCH_CHECK(a_scratch->numel() >= (int64_t)N * p.H * p.D, "a_scratch must hold [chunks, H, D]");
      p.decay_kind = 3;
      p.ldd = (int)d.stride(0);
      p.a_out = a_scratch->data_ptr<float>();
      cp.a_chunk = p.a_out;
    }
    p.decay = d.data_ptr<float>();
  }
  const int* cm = cmeta.data_ptr<int>();
  p.state = state.data_ptr<float>();
  p.nseq = N;
  p.q_start = cm;
  p.ctx_len = cm + N;  // unused by the chunked walk (src_idx decides where a chunk starts from)
  p.state_slot = cm + 5 * N;
  p.out = out.data_ptr<float>();
  p.q_scale = (float)q_scale;
  p.portions = 1;
  // pass 1: from zeros, end states into scratch
  p.q_len = cm + 2 * N;
  p.src_idx = cm + 3 * N, p.dst_idx = cm + 4 * N;
  p.src = scratch.data_ptr<float>(), p.dst = scratch.data_ptr<float>();
  p.no_out = 1;
  DSSE_CHECK_HIP(dsse_matrix_scan(&p, cur_stream()));
  // carry
  cp.scratch = scratch.data_ptr<float>();
  cp.state = state.data_ptr<float>();
  cp.q_len = q_len.data_ptr<int>(), cp.ctx_len = ctx_len.data_ptr<int>(), cp.state_slot = state_slot.data_ptr<int>();
  cp.s_first = s_first.data_ptr<int>(), cp.s_count = s_count.data_ptr<int>();
  cp.cq_len = cm + N;
  cp.nseq = ns, cp.H = p.H, cp.D = p.D, cp.V = p.V, cp.decay_kind = p.decay_kind;
  DSSE_CHECK_HIP(dsse_scan_carry(&cp, cur_stream()));
  // pass 2: from the incoming states, outputs; a sequence's last chunk leaves the slot's state
  p.q_len = cm + N;
  p.src_idx = cm + 5 * N, p.dst_idx = cm + 6 * N;
  p.dst = state.data_ptr<float>();
  p.no_out = 0;
  p.a_out = nullptr;
  DSSE_CHECK_HIP(dsse_matrix_scan(&p, cur_stream()));
}

void gated_head_norm(const Tensor& o, const OptTensor& w, const Tensor& gate, double eps, Tensor& out, int64_t kind) {
  f32t(o, "o");
  col_view(gate, "gate");
  gpu(out, "out");
  TORCH_CHECK(o.dim() == 3 && out.dim() == 2, "o [T, H, V], out [T, H V]");
  const int M = (int)o.size(0), H = (int)o.size(1), V = (int)o.size(2);
  TORCH_CHECK(gate.size(0) == M && gate.size(1) == (int64_t)H * V && out.size(0) == M && out.size(1) == (int64_t)H * V,
              "gate and out must be [T, H V]");
  DSSE_CHECK_HIP(dsse_gated_head_norm(o.data_ptr<float>(), opt_f32(w, "w", V), gate.data_ptr<float>(),
                                      (int)gate.stride(0), out.data_ptr(), M, H, V, (float)eps, (int)kind, elem(out, "out"),
                                      cur_stream()));
}

void rms_mix(const Tensor& ya, const Tensor& wa, const Tensor& yb, const Tensor& wb, double eps, double coef, Tensor& out) {
  f32t(ya, "ya");
  f32t(yb, "yb");
  f32t(out, "out");
  TORCH_CHECK(ya.dim() == 2 && yb.sizes() == ya.sizes() && out.sizes() == ya.sizes(), "ya, yb, out must be [M, W]");
  const int M = (int)ya.size(0), W = (int)ya.size(1);
  f32t(wa, "wa");
  f32t(wb, "wb");
  TORCH_CHECK(wa.numel() == W && wb.numel() == W, "gains must be [W]");
  DSSE_CHECK_HIP(dsse_rms_mix(ya.data_ptr<float>(), wa.data_ptr<float>(), yb.data_ptr<float>(), wb.data_ptr<float>(),
                              out.data_ptr<float>(), M, W, (float)eps, (float)coef, cur_stream()));
}

void logit_cap(Tensor& logits, double scale, double cap) {
  f32t(logits, "logits");
  DSSE_CHECK_HIP(dsse_logit_cap(logits.data_ptr<float>(), (long long)logits.numel(), (float)scale, (float)cap,
                                cur_stream()));
}

}  // namespace

void stream_mix(const OptTensor& y, int64_t nsum, double mult, Tensor& streams, const OptTensor& ids,
                const OptTensor& embed, double embed_scale, const OptTensor& out_w, const OptTensor& mix,
                const OptTensor& in_w, const OptTensor& norm_w, double eps, const OptTensor& h, const OptTensor& total) {
  f32t(streams, "streams", false);
  TORCH_CHECK(streams.dim() == 3, "streams must be [M, S, W]");
  dsse::StreamMixParams p{};
  p.M = (int)streams.size(0), p.S = (int)streams.size(1), p.W = (int)streams.size(2);
  TORCH_CHECK(p.S >= 1 && p.S <= 8, "1..8 streams");
  TORCH_CHECK((p.W == 1 || streams.stride(2) == 1) && (p.S == 1 || streams.stride(1) == p.W) &&
                  (p.M <= 1 || streams.stride(0) >= (int64_t)p.S * p.W),
              "streams: adjacent copies of contiguous rows");
  p.ld = p.M > 1 ? (int)streams.stride(0) : p.S * p.W;
  p.streams = streams.data_ptr<float>();
  p.nsum = (int)nsum, p.mult = (float)mult, p.embed_scale = (float)embed_scale, p.eps = (float)eps;
  TORCH_CHECK(nsum >= 1, "nsum >= 1");
  p.f32 = 1;
  bool typed = false;
  if (y.has_value()) {
    f32t(*y, "y");
    TORCH_CHECK(y->dim() == 2 && y->size(0) == (int64_t)p.M * nsum && y->size(1) == p.W, "y must be [M * nsum, W]");
    p.y = y->data_ptr<float>();
    p.out_w = opt_f32(out_w, "out_w", p.S);
    p.mix = opt_f32(mix, "mix", (int64_t)p.S * p.S);
  }
  if (embed.has_value()) {
    TORCH_CHECK(ids.has_value(), "embed needs ids");
    i32(*ids, "ids");
    gpu(*embed, "embed");
    TORCH_CHECK(embed->dim() == 2 && embed->size(1) == p.W && ids->numel() >= p.M, "embed must be [vocab, W]");
    p.ids = ids->data_ptr<int>();
    p.embed = embed->data_ptr();
    p.vocab = (int)embed->size(0);
    p.f32 = elem(*embed, "embed");
    typed = true;
  }
  if (h.has_value()) {
    TORCH_CHECK(in_w.has_value() && norm_w.has_value(), "h needs in_w and norm_w");
    p.in_w = opt_f32(in_w, "in_w", p.S);
    p.norm_w = opt_f32(norm_w, "norm_w", p.W);
    gpu(*h, "h");
    TORCH_CHECK(h->dim() == 2 && h->size(0) == p.M && h->size(1) == p.W, "h must be [M, W]");
    const int f = elem(*h, "h");
    if (f) {
      p.h_f32 = 1;  // an fp32 h beside a bf16 embedding is the mixed kernel
    } else {
      TORCH_CHECK(!typed || p.f32 == 0, "a bf16 h needs a bf16 embedding");
      p.f32 = 0;
    }
    p.h = h->data_ptr();
  }
  if (total.has_value()) {
    f32t(*total, "total");
    TORCH_CHECK(total->dim() == 2 && total->size(0) == p.M && total->size(1) == p.W, "total must be [M, W]");
    p.total = total->data_ptr<float>();
  }
  DSSE_CHECK_HIP(dsse_stream_mix(&p, cur_stream()));
}

void act_rows(const Tensor& x, Tensor& out, int64_t kind, const OptTensor& params, const OptTensor& gate) {
  col_view(x, "x");
  gpu(out, "out");
  TORCH_CHECK(out.dim() == 2 && out.sizes() == x.sizes(), "out must be [M, F] like x");
  TORCH_CHECK(kind >= 0 && kind <= 2, "kind: 0 identity, 1 xIELU, 2 relu^2");
  const float* pp = opt_f32(params, "params", 2);
  TORCH_CHECK(kind != 1 || pp, "xIELU needs its two constants");
  const float* g = nullptr;
  int ldg = 0;
  if (gate.has_value()) {
    col_view(*gate, "gate");
    TORCH_CHECK(gate->sizes() == x.sizes(), "gate must be [M, F] like x");
    g = gate->data_ptr<float>();
    ldg = (int)gate->stride(0);
  }
  DSSE_CHECK_HIP(dsse_act_rows(x.data_ptr<float>(), (int)x.stride(0), out.data_ptr(), (int)x.size(0), (int)x.size(1),
                               (int)kind, pp, g, ldg, elem(out, "out"), cur_stream()));
}

void moe_route(const Tensor& z, const OptTensor& correction, Tensor& topk_idx, Tensor& topk_w, int64_t groups,
               int64_t keep, double scale, int64_t kind) {
  f32t(z, "z");
  TORCH_CHECK(kind == 0 || kind == 1, "kind: 0 sigmoid scores, 1 softmax scores");
  TORCH_CHECK(kind == 1 || correction.has_value(), "sigmoid routing needs its correction");
  i32(topk_idx, "topk_idx");
  f32t(topk_w, "topk_w");
  TORCH_CHECK(z.dim() == 2 && topk_idx.dim() == 2, "z must be [M, E], topk_idx [M, top]");
  const int M = (int)z.size(0), E = (int)z.size(1), top = (int)topk_idx.size(1);
  TORCH_CHECK(topk_idx.size(0) == M && topk_w.sizes() == topk_idx.sizes(), "routing shapes");
  const float* corr = opt_f32(correction, "correction", E);
  TORCH_CHECK(E >= 1 && E <= 256 && groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && top >= 1 &&
                  top <= keep * (E / groups),
              "routing: E <= 256, equal groups, 1 <= keep <= groups, top <= experts of the kept groups");
  DSSE_CHECK_HIP(dsse_moe_route(z.data_ptr<float>(), corr, M, E, top, (int)groups, (int)keep, (float)scale, (int)kind,
                                topk_idx.data_ptr<int>(), topk_w.data_ptr<float>(), cur_stream()));
}

void embed_pair_rows(const Tensor& ids, const OptTensor& prev, const Tensor& positions, const Tensor& embed,
                     const OptTensor& pair, int64_t mul_prev, int64_t mul_cur, int64_t buckets, Tensor& resid,
                     const OptTensor& x0, const OptTensor& prev_out, const OptTensor& keep) {
  f32t(resid, "resid");
  gpu(embed, "embed");
  i32(ids, "ids");
  TORCH_CHECK(resid.dim() == 2 && embed.dim() == 2 && embed.size(1) == resid.size(1), "resid [M, W], embed [vocab, W]");
  dsse::EmbedPairParams p{};
  p.M = (int)resid.size(0), p.W = (int)resid.size(1);
  p.f32 = elem(embed, "embed");
  TORCH_CHECK(ids.numel() >= p.M, "ids too short");
  p.ids = ids.data_ptr<int>();
  p.embed = embed.data_ptr();
  p.vocab = (int)embed.size(0);
  if (pair.has_value()) {
    gpu(*pair, "pair");
    TORCH_CHECK(prev.has_value(), "the pair table needs each row's previous token");
    i32(*prev, "prev");
    i32(positions, "positions");
    TORCH_CHECK(pair->scalar_type() == embed.scalar_type() && pair->dim() == 2 && pair->size(1) == p.W && buckets >= 1 &&
                    pair->size(0) == buckets + 1,
                "pair must be [buckets + 1, W] in embed's type");
    TORCH_CHECK(prev->numel() >= p.M && positions.numel() >= p.M && mul_prev >= 0 && mul_cur >= 0, "prev / positions too short");
    p.pair = pair->data_ptr();
    p.prev = prev->data_ptr<int>();
    p.positions = positions.data_ptr<int>();
  }
  p.buckets = (int)buckets, p.mul_prev = mul_prev, p.mul_cur = mul_cur;
  p.resid = resid.data_ptr<float>();
  if (x0.has_value()) {
    gpu(*x0, "x0", false);
    TORCH_CHECK(x0->scalar_type() == embed.scalar_type() && x0->dim() == 2 && x0->size(0) == p.M && x0->size(1) == p.W &&
                    (p.W == 1 || x0->stride(1) == 1) && x0->stride(0) >= p.W,
                "x0 must be [M, W] in embed's type with unit column stride");
    p.x0 = x0->data_ptr();
    p.ldx0 = (int)x0->stride(0);
  }
  if (prev_out.has_value()) {
    i32(*prev_out, "prev_out");
    p.prev_out = prev_out->data_ptr<int>();
    p.n_prev_out = (int)std::min<int64_t>(prev_out->numel(), p.M);
    if (keep.has_value()) {
      i32(*keep, "keep");
      TORCH_CHECK(keep->numel() >= p.n_prev_out, "keep too short");
      p.keep = keep->data_ptr<int>();
    }
  }
  DSSE_CHECK_HIP(dsse_embed_pair_rows(&p, cur_stream()));
}

void add_norm_rows(const OptTensor& y, int64_t nsum, const OptTensor& g_add, Tensor& resid, const OptTensor& g_out,
                   double eps, const OptTensor& out, const OptTensor& out32) {
  f32t(resid, "resid");
  TORCH_CHECK(resid.dim() == 2 && nsum >= 1, "resid [M, W], nsum >= 1");
  dsse::AddNormParams p{};
  p.M = (int)resid.size(0), p.W = (int)resid.size(1);
  p.resid = resid.data_ptr<float>();
  p.nsum = (int)nsum;
  if (y.has_value()) {
    f32t(*y, "y");
    TORCH_CHECK(y->numel() == (int64_t)p.M * nsum * p.W, "y must hold M * nsum rows of W");
    TORCH_CHECK(g_add.has_value(), "y needs its norm's gain");
    p.y = y->data_ptr<float>();
    p.g_add = opt_f32(g_add, "g_add", p.W);
  }
  p.g_out = opt_f32(g_out, "g_out", p.W);
  if (out.has_value()) {
    gpu(*out, "out", false);
    TORCH_CHECK(out->dim() == 2 && out->size(0) == p.M && out->size(1) == p.W && (p.W == 1 || out->stride(1) == 1) &&
                    out->stride(0) >= p.W,
                "out must be [M, W] with unit column stride");
    p.out_f32 = elem(*out, "out");
    p.out = out->data_ptr();
    p.ldo = (int)out->stride(0);
  }
  if (out32.has_value()) {
    f32t(*out32, "out32");
    TORCH_CHECK(out32->numel() == (int64_t)p.M * p.W, "out32 must be [M, W]");
    p.out32 = out32->data_ptr<float>();
  }
  p.eps = (float)eps;
  DSSE_CHECK_HIP(dsse_add_norm_rows(&p, cur_stream()));
}

void token_gate_rows(const Tensor& x, const Tensor& ids, const Tensor& table, int64_t col0, Tensor& out) {
  col_view(x, "x");
  i32(ids, "ids");
  gpu(table, "table");
  gpu(out, "out");
  const int M = (int)x.size(0), F = (int)x.size(1);
  TORCH_CHECK(table.dim() == 2 && col0 >= 0 && col0 + F <= table.size(1), "table [vocab, columns] must hold col0 + F columns");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == M && out.size(1) == F && out.scalar_type() == table.scalar_type(),
              "out must be [M, F] in the table's type");
  TORCH_CHECK(ids.numel() >= M, "ids too short");
  DSSE_CHECK_HIP(dsse_token_gate_rows(x.data_ptr<float>(), (int)x.stride(0), ids.data_ptr<int>(), table.data_ptr(),
                                      (int)table.size(0), (int)table.size(1), (int)col0, out.data_ptr(), M, F,
                                      elem(table, "table"), cur_stream()));
}

void token_side_rows(const OptTensor& y, int64_t nsum, const OptTensor& g_add, Tensor& resid, const Tensor& ids,
                     const Tensor& table, int64_t col0, const Tensor& gate_w, const Tensor& proj_w, const Tensor& side_norm,
                     const OptTensor& g_out, double eps, const OptTensor& out, const OptTensor& out32) {
  f32t(resid, "resid");
  i32(ids, "ids");
  gpu(table, "table");
  gpu(gate_w, "gate_w");
  gpu(proj_w, "proj_w");
  TORCH_CHECK(resid.dim() == 2 && nsum >= 1 && gate_w.dim() == 2 && proj_w.dim() == 2 && table.dim() == 2, "shapes");
  dsse::TokenSideParams p{};
  p.M = (int)resid.size(0), p.W = (int)resid.size(1), p.F = (int)gate_w.size(0);
  TORCH_CHECK(gate_w.size(1) == p.W && proj_w.size(0) == p.W && proj_w.size(1) == p.F, "gate_w [F, W], proj_w [W, F]");
  TORCH_CHECK(gate_w.scalar_type() == proj_w.scalar_type() && table.scalar_type() == gate_w.scalar_type(),
              "gate_w, proj_w and table share the element type");
  TORCH_CHECK(col0 >= 0 && col0 + p.F <= table.size(1) && ids.numel() >= p.M, "table must hold col0 + F columns, one id per row");
  TORCH_CHECK((int64_t)(p.W + p.F + 16) * 4 <= 64 * 1024, "row too wide for the one-launch form");
  p.f32 = elem(gate_w, "gate_w");
  p.resid = resid.data_ptr<float>();
  p.nsum = (int)nsum;
  if (y.has_value()) {
    f32t(*y, "y");
    TORCH_CHECK(y->numel() == (int64_t)p.M * nsum * p.W && g_add.has_value(), "y must hold M * nsum rows of W, with its gain");
    p.y = y->data_ptr<float>();
    p.g_add = opt_f32(g_add, "g_add", p.W);
  }
  p.ids = ids.data_ptr<int>();
  p.table = table.data_ptr();
  p.vocab = (int)table.size(0), p.ldt = (int)table.size(1), p.col0 = (int)col0;
  p.gate_w = gate_w.data_ptr();
  p.proj_w = proj_w.data_ptr();
  f32t(side_norm, "side_norm");
  TORCH_CHECK(side_norm.numel() == p.W, "side_norm must be [W]");
  p.side_norm = side_norm.data_ptr<float>();
  p.g_out = opt_f32(g_out, "g_out", p.W);
  if (out.has_value()) {
    gpu(*out, "out", false);
    TORCH_CHECK(out->scalar_type() == gate_w.scalar_type() && out->dim() == 2 && out->size(0) == p.M && out->size(1) == p.W &&
                    (p.W == 1 || out->stride(1) == 1) && out->stride(0) >= p.W,
                "out must be [M, W] in the weights' type with unit column stride");
    p.out = out->data_ptr();
    p.ldo = (int)out->stride(0);
  }
  if (out32.has_value()) {
    f32t(*out32, "out32");
    TORCH_CHECK(out32->numel() == (int64_t)p.M * p.W, "out32 must be [M, W]");
    p.out32 = out32->data_ptr<float>();
  }
  p.eps = (float)eps;
  DSSE_CHECK_HIP(dsse_token_side_rows(&p, cur_stream()));
}

TORCH_LIBRARY_FRAGMENT(dsse, m) {
  m.def("token_side_rows(Tensor? y, int nsum, Tensor? g_add, Tensor(a!) resid, Tensor ids, Tensor table, int col0, "
        "Tensor gate_w, Tensor proj_w, Tensor side_norm, Tensor? g_out, float eps, Tensor(b!)? out, Tensor(c!)? out32) -> ()");
  m.def("stream_mix(Tensor? y, int nsum, float mult, Tensor(a!) streams, Tensor? ids, Tensor? embed, float embed_scale, "
        "Tensor? out_w, Tensor? mix, Tensor? in_w, Tensor? norm_w, float eps, Tensor(b!)? h, Tensor(c!)? total) -> ()");
  m.def("act_rows(Tensor x, Tensor(a!) out, int kind, Tensor? params=None, Tensor? gate=None) -> ()");
  m.def("moe_route(Tensor z, Tensor? correction, Tensor(a!) topk_idx, Tensor(b!) topk_w, int groups, int keep, "
        "float scale, int kind=0) -> ()");
  m.def("embed_pair_rows(Tensor ids, Tensor? prev, Tensor positions, Tensor embed, Tensor? pair, int mul_prev, "
        "int mul_cur, int buckets, Tensor(a!) resid, Tensor(b!)? x0, Tensor(c!)? prev_out, Tensor? keep) -> ()");
  m.def("add_norm_rows(Tensor? y, int nsum, Tensor? g_add, Tensor(a!) resid, Tensor? g_out, float eps, "
        "Tensor(b!)? out, Tensor(c!)? out32) -> ()");
  m.def("token_gate_rows(Tensor x, Tensor ids, Tensor table, int col0, Tensor(a!) out) -> ()");
  m.def("stream_step(Tensor? y, float mult, Tensor(a!) resid, Tensor? ids, Tensor? embed, Tensor? vec, Tensor? alpha, "
        "Tensor? w, Tensor? b, Tensor(b!)? xb) -> ()");
  m.def("gated_act(Tensor gu, Tensor(a!) h, int kind=1) -> ()");
  m.def("norm_rope_rows(Tensor x, Tensor? norm_w, Tensor positions, Tensor? rope, Tensor(a!) out, Tensor? out_rows, "
        "int kind, float eps, float scale=1.0, Tensor(b!)? out_t=None) -> ()");
  m.def("sink_attention(Tensor q, Tensor kcache, Tensor vcache, Tensor block_tables, Tensor q_start, Tensor q_len, "
        "Tensor ctx_len, Tensor work_seq, Tensor work_tile, Tensor? sink, Tensor? gate, Tensor(a!) out, int window, "
        "float scale, int qt, Tensor? vt=None, bool split=False, float softcap=0.0, Tensor? out_rope=None) -> ()");
  m.def("gate_math(Tensor(a!) x, int kind, Tensor? p1=None, Tensor? p2=None, float c=1.0) -> ()");
  m.def("matrix_scan(Tensor q, Tensor k, Tensor v, Tensor? decay, Tensor? beta, Tensor(a!) state, Tensor q_start, "
        "Tensor q_len, Tensor ctx_len, Tensor state_slot, Tensor(b!) out, float q_scale=1.0) -> ()");
  m.def("matrix_scan_chunked(Tensor q, Tensor k, Tensor v, Tensor? decay, Tensor(a!) state, Tensor q_len, Tensor ctx_len, "
        "Tensor state_slot, Tensor s_first, Tensor s_count, Tensor cmeta, Tensor(b!) scratch, Tensor(c!)? a_scratch, "
        "Tensor(d!) out, float q_scale=1.0) -> ()");
  m.def("gated_head_norm(Tensor o, Tensor? w, Tensor gate, float eps, Tensor(a!) out, int kind=0) -> ()");
  m.def("rms_mix(Tensor ya, Tensor wa, Tensor yb, Tensor wb, float eps, float coef, Tensor(a!) out) -> ()");
  m.def("logit_cap(Tensor(a!) logits, float scale, float cap) -> ()");
}

TORCH_LIBRARY_IMPL(dsse, CUDA, m) {
  m.impl("stream_mix", &stream_mix);
  m.impl("act_rows", &act_rows);
  m.impl("moe_route", &moe_route);
  m.impl("embed_pair_rows", &embed_pair_rows);
  m.impl("add_norm_rows", &add_norm_rows);
  m.impl("token_gate_rows", &token_gate_rows);
  m.impl("token_side_rows", &token_side_rows);
  m.impl("stream_step", &stream_step);
  m.impl("gated_act", &gated_act);
  m.impl("norm_rope_rows", &norm_rope_rows);
  m.impl("sink_attention", &sink_attention);
  m.impl("gate_math", &gate_math);
  m.impl("matrix_scan", &matrix_scan);
  m.impl("matrix_scan_chunked", &matrix_scan_chunked);
  m.impl("gated_head_norm", &gated_head_norm);
  m.impl("rms_mix", &rms_mix);
  m.impl("logit_cap", &logit_cap);
}
