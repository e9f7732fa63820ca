// Host-visible API of the kernels that serve pre-norm designs with matrix-state mixers: the residual stream's step with
// the element-wise tanh norm, the gated activation of a fused gate | up projection, per-row norms with the rotate-half
// rotation (also the write of keys and values into their pages), softmax attention with a sink over paged keys and
// values of any head width, the gate math of decays, the matrix-state recurrence (plain, decayed, delta rule), the
// per-head output norm with its SiLU gate, the normed mix of two mixers, and the logit scale and cap.
//
// Activations between these kernels are fp32; `T` is the engine's element type (bf16 for serving, fp32 for the exact
// mode) and appears only where a projection reads or a page stores.  Small parameter vectors are fp32 in both modes.
// Sequence metadata as in api_layers.h: per sequence q_start, q_len (0 = inactive), ctx_len (tokens after this step).
#pragma once
#include "api.h"

namespace dsse {

struct StreamStepParams {
  const float* y;        // [M, W] sublayer output or null
  float mult;            // resid += mult * y
  float* resid;          // [M, W] fp32 stream
  const int* ids;        // [M] token ids (with embed)
  const void* embed;     // [vocab, W] element type or null: resid += embed[ids]
  int vocab;
  const float* vec;      // [W] or null: resid += vec
  const float* alpha;    // one number
  const float* w;        // [W] or null: no norm, xb untouched
  const float* b;        // [W]
  void* xb;              // [M, W] element type: tanh(alpha * resid) * w + b
  int M, W;
  int f32;
};

struct NormRopeParams {
  const float* x;        // [T, nh, D], rows ldx apart
  const float* norm_w;   // [nh * D] (kind 1) or null
  const int* positions;  // [T]
  const float2* rope;    // [rope_len, half] (cos, sin) or null
  void* out;             // rows ldo apart, [nh, D] each; fp32 when out_f32 else bf16
  const int* out_rows;   // [T] or null (row t); negative = skip
  void* out_t;           // with out_rows: also into transposed pages [pages, nh, D, kBS] (bf16), token permuted, or null
  int T, nh, D, ldx, ldo, half, rope_len, num_out_rows;
  int kind;              // 0 none, 1 RMS over the whole row times norm_w, 2 unit vector per head, 3 RMS per head times
                         // norm_w [D] (one gain vector for all heads)
  float eps, scale;
  int out_f32;
};

struct SinkAttnParams {
  const float* q;        // [T, H, D] fp32 (normed, rotated)
  const void* k;         // [pages * kBS, G, D] element type
  const void* v;         // [pages * kBS, G, V]
  const int* block_tables;
  int max_blocks, num_blocks;
  const int* q_start;
  const int* q_len;
  const int* ctx_len;
  const int* work_seq;
  const int* work_tile;
  const float* sink;     // [H] or null
  const float* gate;     // [T, ..] rows ldg apart, column h: output times sigmoid, or null
  void* out;             // [T, H, V] element type
  int H, G, D, V, window, qt, ldg;
  float scale;
  int f32;
  float softcap;         // > 0: score = softcap * tanh(scale q.k / softcap)
  const float2* out_rope;  // [out_rope_len, V / 2] (cos, sin) or null: each head's sum is turned back by the row's own
  int out_rope_len;        // position, rotate-half pairs (m, m + V / 2), before the gate
};

struct MatrixScanParams {
  const float* q;        // [T, G, D] rows ldq apart
  const float* k;        // rows ldk apart
  const float* v;        // [T, H, V] rows ldv apart
  const float* decay;    // kind 1: [H]; 2: [T, H] rows ldd apart; 3: [T, H, D] rows ldd apart
  const float* beta;     // [T, H] rows ldb apart, or null (no delta rule)
  float* state;          // [slots, H, D, V]
  const int* q_start;
  const int* q_len;
  const int* ctx_len;
  const int* state_slot;
  float* out;            // [T, H, V]
  int nseq, H, G, D, V, ldq, ldk, ldv, ldd, ldb;
  int decay_kind;        // 0 none
  float q_scale;
  // two-level walk of long prompt portions (src_idx null = the plain walk): a "sequence" of the launch is then a CHUNK
  // of a portion, its initial state comes from entry src_idx[i] of `src` (-1 = zeros) and its end state goes to entry
  // dst_idx[i] of `dst` (-1 = nowhere); entries are [H, D, V]
  const int* src_idx;
  const int* dst_idx;
  const float* src;
  float* dst;
  int no_out;            // 1: a pass that only produces end states
  int portions;          // 1: the rows are prompt portions (many rows per sequence): the wave-local kernel
  float* a_out;          // [nseq, H, D] product of the chunk's per-channel decays (decay_kind 3) or null
};

// The carry between the two passes of the two-level walk: per sequence, the incoming state of each of its chunks.
struct ScanCarryParams {
  float* scratch;        // [chunks, H, D, V]: in: a chunk's end state from zeros; out: the chunk's incoming state
  const float* a_chunk;  // [chunks, H, D] per-channel decay products (decay_kind 3) or null
  const float* decay;    // [H] (decay_kind 1) or null
  const float* state;    // [slots, H, D, V]
  const int* q_len;      // per sequence
  const int* ctx_len;
  const int* state_slot;
  const int* s_first;    // first chunk of the sequence
  const int* s_count;    // its chunks
  const int* cq_len;     // [chunks] tokens of a chunk
  int nseq, H, D, V, decay_kind;
};

// One pass over the residual streams of every row between two sublayers of a design that carries several of them.
struct StreamMixParams {
  float* streams;        // [M, S, W] fp32, rows ld apart
  const float* y;        // [M * nsum, W] finished sublayer output (a row's nsum parts are summed) or null
  int nsum;
  float mult;            // x_t = sum_s mix[s][t] x_s + mult * out_w[t] * y
  const float* out_w;    // [S] or null (ones)
  const float* mix;      // [S, S] indexed [from][to], or null (identity)
  const int* ids;        // [M] token ids (with embed)
  const void* embed;     // [vocab, W] element type or null: every stream = embed[ids] * embed_scale
  int vocab;
  float embed_scale;
  const float* in_w;     // [S] or null: with h, u = sum_s in_w[s] x_s
  const float* norm_w;   // [W]
  void* h;               // [M, W]: u / rms(u) * norm_w (fp32 when h_f32, else the element type), or null
  float* total;          // [M, W] sum of the streams, or null
  int M, S, W, ld;
  float eps;
  int f32;               // element type of embed (and of h unless h_f32)
  int h_f32;
};

// The embedding of a design that adds a hashed row per (previous token, token) pair.
struct EmbedPairParams {
  const int* ids;        // [M]
  const int* prev;       // [M] previous token of each row (with pair)
  const int* positions;  // [M]: position 0 takes row `buckets`
  const void* embed;     // [vocab, W] element type
  const void* pair;      // [buckets + 1, W] element type or null
  int vocab, buckets;
  long long mul_prev, mul_cur;
  float* resid;          // [M, W] fp32
  void* x0;              // rows ldx0 apart, element type, or null: the same row once more
  int ldx0;
  int* prev_out;         // [n_prev_out] or null: row i < n_prev_out stores its token when keep[i] > 0 (keep null: always)
  const int* keep;
  int n_prev_out;
  int M, W, f32;
};

// The stream's step of a design with a norm before and after each sublayer.
struct AddNormParams {
  const float* y;        // [M * nsum, W] or null: resid += rms-norm(sum of the row's parts) * g_add
  int nsum;
  const float* g_add;    // [W]
  float* resid;          // [M, W] fp32
  const float* g_out;    // [W] or null: out = resid itself
  void* out;             // rows ldo apart (fp32 when out_f32, else bf16) or null
  float* out32;          // [M, W] fp32 copy of the unrounded output row, or null
  int M, W, ldo, out_f32;
  float eps;
};

// A per-layer token input in one launch (decode-sized steps): stream += norm(y) * g_add; g = gelu_tanh(gate_w x) *
// table[id, col0 : col0 + F] on the rounded stream x; stream += norm(proj_w g) * side_norm; out = norm(stream) * g_out.
struct TokenSideParams {
  const float* y;        // [M * nsum, W] pending sublayer output or null
  int nsum;
  const float* g_add;    // [W]
  float* resid;          // [M, W] fp32
  const int* ids;        // [M]
  const void* table;     // [vocab, ldt] element type
  int vocab, ldt, col0;
  const void* gate_w;    // [F, W] element type
  const void* proj_w;    // [W, F] element type
  const float* side_norm;  // [W]
  const float* g_out;    // [W] or null: out = the stream itself
  void* out;             // rows ldo apart, element type, or null
  float* out32;          // [M, W] or null
  int ldo;
  int M, W, F, f32;
  float eps;
};

}  // namespace dsse

extern "C" {
hipError_t dsse_token_side_rows(const dsse::TokenSideParams* p, hipStream_t st);
hipError_t dsse_embed_pair_rows(const dsse::EmbedPairParams* p, hipStream_t st);
hipError_t dsse_add_norm_rows(const dsse::AddNormParams* p, hipStream_t st);
// out [M, F] = gelu_tanh(x) * table[ids, col0 : col0 + F] (table rows ldt apart)
hipError_t dsse_token_gate_rows(const float* x, int ldx, const int* ids, const void* table, int vocab, int ldt, int col0,
                                void* out, int M, int F, int f32, hipStream_t st);
hipError_t dsse_stream_mix(const dsse::StreamMixParams* p, hipStream_t st);
// out [M, F] = act(x) * sigmoid(gate): kind 0 identity, 1 xIELU with params = (a_p, a_n), 2 relu^2; gate may be null
hipError_t dsse_act_rows(const float* x, int ldx, void* out, int M, int F, int kind, const float* params,
                         const float* gate, int ldg, int f32, hipStream_t st);
// group-limited routing from fp32 logits [M, E] (E <= 256); kind 0: sigmoid scores + correction, groups by the sum of
// their two best, weights renormalised; kind 1: softmax scores (corr may be null), groups by their best, weights as is
hipError_t dsse_moe_route(const float* z, const float* corr, int M, int E, int top, int groups, int keep, float scale,
                          int kind, int* topk_idx, float* topk_w, hipStream_t st);
hipError_t dsse_stream_step(const dsse::StreamStepParams* p, hipStream_t st);
hipError_t dsse_gated_act(const float* gu, int ldg, void* h, int M, int F, int kind, int f32, hipStream_t st);
hipError_t dsse_norm_rope_rows(const dsse::NormRopeParams* p, hipStream_t st);
hipError_t dsse_sink_attention(int num_work, const dsse::SinkAttnParams* p, hipStream_t st);
// MFMA form for prompt portions (bf16, D % 32 == 0, V / 16 in {1..8, 10, 12, 16, 20, 24, 32}): 16-row tiles, values from the
// transposed pages vt [pages, G, V, kBS] (keys permuted inside a page as the MFMA's k axis wants them)
// split (V <= 128): the four waves of a workgroup share one (tile, head) and split its pages -- decode steps
hipError_t dsse_sink_flash(int num_work, const dsse::SinkAttnParams* p, const void* vt, int split, hipStream_t st);
// p1 / p2 hold N / rep1 and N / rep2 numbers: entry j serves columns [j rep, (j + 1) rep)
hipError_t dsse_gate_math(float* x, int ld, int M, int N, int kind, const float* p1, int rep1, const float* p2, int rep2,
                          float c, hipStream_t st);
hipError_t dsse_matrix_scan(const dsse::MatrixScanParams* p, hipStream_t st);
hipError_t dsse_scan_carry(const dsse::ScanCarryParams* p, hipStream_t st);
// gate_kind 0: silu(gate), 1: sigmoid(gate)
hipError_t dsse_gated_head_norm(const float* o, const float* w, const float* gate, int ldg, void* out, int M, int H,
                                int V, float eps, int gate_kind, int f32, hipStream_t st);
hipError_t dsse_rms_mix(const float* ya, const float* wa, const float* yb, const float* wb, float* out, int M, int W,
                        float eps, float coef, hipStream_t st);
hipError_t dsse_logit_cap(float* logits, long long n, float scale, float cap, hipStream_t st);
}
