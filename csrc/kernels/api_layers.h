// Host-visible API of the layer-mechanism kernels that serve configuration-driven designs (layers listed in a
// checkpoint's config.json): the general row-major GEMM, the one-number RMS norm on a sublayer's output, latent
// (compressed-KV) attention with a sliding window, the gated linear recurrence with its short convolution, and the
// routed mixture of experts.  Every kernel takes its sizes and constants as parameters and exists for two element
// types: bf16 (serving) and fp32 (the exact mode: every product and sum in true 32-bit).
//
// Sequence metadata follows the engine's convention (api.h AttnParams): per sequence q_start (first row), q_len (rows
// in this step, 0 = inactive) and ctx_len (tokens after this step); a row's position is ctx_len - q_len + its offset.
#pragma once
#include "api.h"

namespace dsse {

struct GemmRmParams {
  const void* x;     // [M, K] rows ldx apart, batch z at + z * xbs elements
  const void* w;     // [N, K] rows ldw apart (row-major [out, in]), batch z at + z * wbs
  const void* bias;  // [N] of the weight's type or null, batch z at + z * bbs
  void* out;         // [M, N] rows ldo apart, batch z at + z * obs; fp32 when out_f32 else the element type
  int M, N, K, batch;
  int ldx, ldw, ldo;
  long long xbs, wbs, bbs, obs;
  int act;           // 0 none, 1 gelu (tanh form)
  int out_f32;
  int f32;           // element type of x / w / bias: 0 bf16, 1 fp32
  int vecx, vecw;    // 16-byte fragment loads allowed (base, row and batch strides aligned)
};

struct ScalarNormParams {
  const float* y;    // [M * nsum, W] sublayer output, a row's nsum consecutive parts are summed (mode 0) -- unused in mode 1
  int nsum;
  const void* g;     // one number, element type
  float* resid;      // [M, W] fp32 stream
  void* xb;          // [M, W] element type: the stream's rounding (mode 0) / the normed stream (mode 1)
  int M, W;
  float eps;
  int mode;          // 0: resid += y / rms(y) * g, xb = resid;  1: xb = resid / rms(resid) * g
  int f32;
};

struct LatentKvWriteParams {
  const float* ckr;      // [T, rk + dr] down-projection (latent | shared rotated key part), rows ld apart
  const void* norm_w;    // [rk]
  const int* positions;  // [T]
  const int* slots;      // [T] cache row (page * kBS + offset), -1 = skip
  const float2* rope;    // [rope_len, dr / 2] (cos, sin), amplitude folded in
  void* cache;           // [pages * kBS, rk + dr]
  int T, rk, dr, rope_len, num_slots;
  float eps;
  int f32;
  int ld;                // row stride of ckr (a column slice of a wider buffer), rk + dr when contiguous
};

struct LatentAttnParams {
  const void* q;         // [T, H, dn + dr]: the rotated part is read (and rotated) here
  const float* q_abs;    // [T, H, rk]: the unrotated part folded through the key up-projection
  const void* cache;     // [pages * kBS, rk + dr]
  const int* block_tables;
  int max_blocks, num_blocks;
  const int* q_start;
  const int* q_len;
  const int* ctx_len;
  const int* work_seq;
  const int* work_tile;
  const float2* rope;
  void* out;             // [T, H, rk]: softmax-weighted sum of latents (the value up-projection follows)
  int H, dn, dr, rk, window, qt, rope_len;
  float scale;
  int f32;
  // MFMA form with the keys of an item split over gridDim.z partitions (decode: few items, long windows): partition z
  // leaves its unnormalised O^T and (max, sum) per column in part [item][head tile][z][16 x rk | 16 x 2] and a combine
  // kernel merges them.  nparts <= 1: no split.
  float* part;
  int nparts;
};

struct ConvStateParams {
  const float* in;       // [T, C] fp32, rows ld_in apart
  const void* taps;      // [C, K]; taps[c][K - 1] weighs the newest input
  const void* bias;      // [C]
  const void* in_bias;   // [C] or null: added to every input (the input projection's bias; tails hold biased inputs)
  float* tail;           // [slots, K - 1, C] last K - 1 inputs of each sequence
  const int* q_start;
  const int* q_len;
  const int* ctx_len;
  const int* state_slot;
  float* out;            // [T, C] fp32 or null
  void* out_b;           // [T, C] element type (the gates' GEMM input) or null
  int nseq, C, K, rows;  // rows = T
  int f32;
  int ld_in;             // row stride of `in` (a column slice of a wider buffer), C when contiguous
  int act;               // 0 none, 1 SiLU on the output (the tail keeps the raw inputs), 2 the row's input added to it
  int single;            // 1: every sequence has few rows (a decode step: one): the convolution kernel also moves the tail
};

struct LruScanParams {
  const float* u;        // [T, C] convolution output
  const float* gates;    // [T, blocks, 2 * bw]: per block [recurrence gate | input gate] pre-activations (bias added);
                         // overwritten with the recurrence's coefficients (a | b) when coeff is set
  const float* y;        // [T, C] gelu branch before its bias and gelu
  const void* y_bias;    // [C] or null
  const void* lam;       // [C]
  float* state;          // [slots, C]
  const int* q_start;
  const int* q_len;
  const int* ctx_len;
  const int* state_slot;
  void* out;             // [T, C] element type: state * y
  int nseq, C, bw, rows; // rows = T
  int coeff;             // 1: compute (a, b) for all rows first; 0: gates already hold them (a later sequence group)
  float* chunk_a;        // [rows / 32 + nseq + 1, C] scratch of the chunked walk (prompt portions), or null
  float* chunk_b;
  float c;               // 8: log a = -c r softplus(lam)
  int f32;
};

struct MoeRouterParams {
  const void* x;         // [M, W]
  const void* w;         // [E, W]
  const void* b;         // [E]
  int* topk_idx;         // [M, top]
  float* topk_w;         // [M, top]
  int M, W, E, top;
  int f32;
};

struct MoeFfnParams {
  const void* x;         // [M, W]
  const int* topk_idx;
  const float* topk_w;
  const void* gate;      // [E, F, W]
  const void* up;        // [E, F, W]
  const void* down;      // [E, W, F]
  const void* sgate;     // shared expert [Fs, W] or null
  const void* sup;
  const void* sdown;     // [W, Fs]
  float* out;            // [M, W] fp32
  int M, W, F, Fs, E, top;
  int f32;
};

struct MoeGroupedParams {
  const void* x;         // [M, W]
  const int* topk_idx;   // [M, top]
  const float* topk_w;   // [M, top]
  const void* gate;      // [E, F, W], or null: experts without a gate, h = relu(up x)^2
  const void* up;
  const void* down;      // [E, W, F]
  const void* sgate;     // shared expert (slot `top`, expert index E) or null
  const void* sup;
  const void* sdown;
  int* sorted;           // [max_tiles * 64] ids (row * S + slot) grouped by expert, -1 = pad
  int* tile_expert;      // [max_tiles]
  int* num_tiles;        // [1]
  void* h;               // [M * S, ldh] element type
  float* o;              // [M * S, W]
  int M, W, F, Fs, E, top, S, ldh, max_tiles;
  int vec_w, vec_h;      // 16-byte fragment loads allowed on rows W wide / on rows of h
  int lds_tiles;         // 1: enough rows for the LDS-staged tiles (prompt portions); 0: the register-direct kernels
  int f32;
};

}  // namespace dsse

extern "C" {
hipError_t dsse_gemm_rm(const dsse::GemmRmParams* p, hipStream_t st);
hipError_t dsse_scalar_norm(const dsse::ScalarNormParams* p, hipStream_t st);
hipError_t dsse_embed_rows(int M, int W, int vocab, const int* ids, const void* embed, float* resid, void* xb, int f32,
                           hipStream_t st);
hipError_t dsse_latent_kv_write(const dsse::LatentKvWriteParams* p, void* vt, hipStream_t st);  // vt: see below, or null
hipError_t dsse_latent_attention(int num_work, const dsse::LatentAttnParams* p, hipStream_t st);
// transposed latent pages vt [pages, rk, kBS] (keys permuted inside a page) for the MFMA form, and that form itself
// (bf16, rk in {64, 128, 256, 512}, dr % 32 == 0; 16 columns = rt rows x hp heads per work item)
hipError_t dsse_latent_flash(int num_work, const dsse::LatentAttnParams* p, const void* vt, int rt, int hp,
                             hipStream_t st);
hipError_t dsse_conv_state(const dsse::ConvStateParams* p, hipStream_t st);
hipError_t dsse_lru_scan(const dsse::LruScanParams* p, hipStream_t st);
hipError_t dsse_moe_router(const dsse::MoeRouterParams* p, hipStream_t st);
hipError_t dsse_moe_ffn(const dsse::MoeFfnParams* p, hipStream_t st);
hipError_t dsse_moe_grouped(const dsse::MoeGroupedParams* p, hipStream_t st);
hipError_t dsse_moe_topk(const float* z, int M, int E, int top, int* topk_idx, float* topk_w, hipStream_t st);
}
