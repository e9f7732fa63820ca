"""Layer-mechanism ops for configuration-driven designs: HIP kernels on GPU tensors, ``layers_reference`` on CPU tensors.

Dispatch follows ``ops/__init__.py``: a GPU tensor always takes the HIP kernel (the call raises when the kernel library
is missing), a CPU tensor the PyTorch reference.  The element type (bf16, or fp32 for the exact mode) comes with the
tensors; sizes and constants are arguments, so another design reuses the same ops with its own numbers.
"""
from __future__ import annotations

import torch

from . import layers_reference as lref


def _hip(t: torch.Tensor) -> bool:
    if t.is_cuda:
        from . import load_library

        load_library(required=True)
        return True
    return False


def gemm_rm(x, w, out, bias=None, act: int = 0):
    """out = act(x · wᵀ + bias) for row-major w [N, K]; any sizes; 3-D operands are batched over dim 0 (strided views
    of wider buffers are fine: only the innermost stride must be 1).  act: 0 none, 1 gelu (tanh form)."""
    if _hip(x):
        torch.ops.dsse.gemm_rm(x, w, out, bias, act)
    else:
        lref.gemm_rm(x, w, out, bias, act)


def scalar_norm(y, g, resid, xb, eps: float, nsum: int = 1):
    """y given: resid += y / rms(y) · g (one number g), xb = resid rounded; y [M · nsum, W] holds each row in nsum
    consecutive parts that are summed first (the grouped experts' slots).  y None: xb = resid / rms(resid) · g."""
    if _hip(resid):
        torch.ops.dsse.scalar_norm(y, g, resid, xb, eps, nsum)
    else:
        lref.scalar_norm(y, g, resid, xb, eps, nsum)


def embed_rows(ids, embed, resid, xb):
    """resid (fp32) = xb = embed[ids]."""
    if _hip(resid):
        torch.ops.dsse.embed_rows(ids, embed, resid, xb)
    else:
        lref.embed_rows(ids, embed, resid, xb)


def latent_kv_write(ckr, norm_w, positions, slots, rope, cache, eps: float, vt=None):
    """cache[slot] = [rms-norm(ckr[:, :rk]) · norm_w | rot(ckr[:, rk:])] for rows with slot >= 0; vt (optional,
    [pages, rk, 32]) receives the latent once more in transposed pages (the MFMA attention's value operand)."""
    if _hip(ckr):
        torch.ops.dsse.latent_kv_write(ckr, norm_w, positions, slots, rope, cache, eps, vt)
    else:
        lref.latent_kv_write(ckr, norm_w, positions, slots, rope, cache, eps, vt)


def latent_flash_ok(dtype, rk: int, dr: int) -> bool:
    """Shapes the MFMA form of latent_attention covers (everything else takes the row kernel)."""
    return dtype == torch.bfloat16 and rk in (64, 128, 256, 512) and dr % 32 == 0


def latent_flash_part_floats(items: int, heads: int, hp: int, nparts: int, rk: int) -> int:
    """fp32 words of the key-split scratch of latent_attention's MFMA form."""
    return items * (-(-heads // hp)) * nparts * 16 * (rk + 2)


def latent_attention(q, q_abs, cache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile, rope, out,
                     window: int, scale: float, qt: int, vt=None, hp: int = 1, part=None, nparts: int = 1):
    """Sliding-window multi-query attention over the latent cache (folded form), `qt` query rows per work item.
    With vt (transposed latent pages, latent_flash_ok shapes): the MFMA form, qt rows x hp heads = 16 columns per
    item, the item's keys optionally split over `nparts` partitions (fp32 scratch `part`, latent_flash_part_floats)
    and merged by a combine kernel; without vt: the row kernel (any sizes, both element types)."""
    if _hip(q):
        torch.ops.dsse.latent_attention(q, q_abs, cache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile,
                                        rope, out, window, scale, qt, vt, hp, part, nparts)
    else:
        lref.latent_attention(q, q_abs, cache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile, rope, out,
                              window, scale, qt, vt)


def conv_state(inp, taps, bias, tail, q_start, q_len, ctx_len, state_slot, out, out_b, in_bias=None, act: int = 0,
               single: bool = False):
    """Per-channel causal convolution continued from each sequence's slot tail (and the tail's update); in_bias is
    added to every input (the bias of the projection that made `inp`).  `inp` may be a column slice of a wider fp32
    buffer; bias, out (fp32) and out_b (the output in the element type) may be None (not both outputs); act 1 applies
    SiLU to the output, act 2 adds the row's own input to it (inp + conv(inp)).  single: every sequence of the call has
    one row (a decode step), so one launch also moves the tails."""
    if _hip(inp):
        torch.ops.dsse.conv_state(inp, taps, bias, tail, q_start, q_len, ctx_len, state_slot, out, out_b, in_bias, act,
                                  single)
    else:
        lref.conv_state(inp, taps, bias, tail, q_start, q_len, ctx_len, state_slot, out, out_b, in_bias, act)


def lru_scan(u, gates, y, lam, state, q_start, q_len, ctx_len, state_slot, out, c: float, y_bias=None,
             coeff: bool = True, scratch=None):
    """Real-gated linear recurrence continued from each sequence's slot state; out = state · gelu(y + y_bias).
    coeff: turn the gate pre-activations of ALL rows into the recurrence's coefficients first (in place); pass False
    for a further sequence group of the same step.  scratch (fp32 [2, rows / 32 + sequences + 1, C]): steps of 128 rows
    or more walk in three phases over 32-row chunks instead of one thread per sequence and channel."""
    if _hip(u):
        torch.ops.dsse.lru_scan(u, gates, y, lam, state, q_start, q_len, ctx_len, state_slot, out, c, y_bias, coeff,
                                scratch)
    else:
        lref.lru_scan(u, gates, y, lam, state, q_start, q_len, ctx_len, state_slot, out, c, y_bias, coeff)


def moe_topk(logits, topk_idx, topk_w):
    """The top-k experts of fp32 router logits [M, E] and the softmax over the chosen logits."""
    if _hip(logits):
        torch.ops.dsse.moe_topk(logits, topk_idx, topk_w)
    else:
        lref.moe_topk(logits, topk_idx, topk_w)


def moe_router(x, w, b, topk_idx, topk_w):
    """fp32 router logits, the top-k experts per row and the softmax over the chosen logits."""
    if _hip(x):
        torch.ops.dsse.moe_router(x, w, b, topk_idx, topk_w)
    else:
        lref.moe_router(x, w, b, topk_idx, topk_w)


def moe_ffn(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, out):
    """out (fp32) = sum_k w_k · expert_k(x) + shared(x), experts of the gated-SiLU form."""
    if _hip(x):
        torch.ops.dsse.moe_ffn(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, out)
    else:
        lref.moe_ffn(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, out)


def moe_grouped(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, sorted_ids, tile_expert, num_tiles, h, o):
    """Grouped form of the routed experts: rows sorted by expert, 16-row MFMA tiles of one expert each.  o [M · S, W]
    (fp32) = weight · expert output per (row, slot), S = top (+ 1: the shared expert's slot); the norm or stream step
    that follows sums them (nsum=S).  gate None: experts without a gate, down(relu(up x)^2).  sorted_ids / tile_expert /
    num_tiles / h are scratch."""
    if _hip(x):
        torch.ops.dsse.moe_grouped(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, sorted_ids, tile_expert,
                                   num_tiles, h, o)
    else:
        lref.moe_grouped(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, o)


# ---------------------------------------------------------------------------------------------------------------------
# Pre-norm designs with matrix-state mixers.  Small parameter vectors (norm gains, sinks, decay parameters) are fp32
# in both element types.
def stream_step(y, mult: float, resid, ids, embed, vec, alpha, w, b, xb):
    """The residual stream's step between sublayers: resid (fp32) += mult * y (y given) + embed[ids] (embed given) +
    vec (vec [W] given); then, when a norm follows (w given), xb = tanh(alpha * resid) * w + b in the element type."""
    if _hip(resid):
        torch.ops.dsse.stream_step(y, mult, resid, ids, embed, vec, alpha, w, b, xb)
    else:
        lref.stream_step(y, mult, resid, ids, embed, vec, alpha, w, b, xb)


def gated_act(gu, h, kind: int = 1):
    """h = act(gu[:, :F]) * gu[:, F:] for the fused gate | up projection's fp32 output; kind 0 SiLU, 1 gelu (tanh)."""
    if _hip(gu):
        torch.ops.dsse.gated_act(gu, h, kind)
    else:
        lref.gated_act(gu, h, kind)


def norm_rope_rows(x, norm_w, positions, rope, out, out_rows, norm_kind: int, eps: float, scale: float = 1.0, out_t=None):
    """Rows x [T, heads, D] (fp32, may be a column slice of a wider buffer) -> out rows out_rows[t] (or t) in out's
    type: an optional norm (1: RMS over the whole row times norm_w [heads * D]; 2: unit vector per head; 3: RMS per head
    times norm_w [D], one gain vector for all heads), the rotate-half rotation
    of the leading 2 * rope.shape[1] coordinates (rope [positions, dims / 2, 2] or None), times scale.  With out_rows =
    cache rows this writes keys or values straight into their pages [pages, 32, heads, D]; out_t (optional,
    [pages, heads, D, 32]) receives them once more in transposed pages (the MFMA attention's value operand)."""
    if _hip(x):
        torch.ops.dsse.norm_rope_rows(x, norm_w, positions, rope, out, out_rows, norm_kind, eps, scale, out_t)
    else:
        lref.norm_rope_rows(x, norm_w, positions, rope, out, out_rows, norm_kind, eps, scale, out_t)


SINK_FLASH_TILES = (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16, 20, 24, 32)  # value widths / 16 the MFMA form is built for


SINK_SPLIT_MAX_V = 128  # widest value head whose key-split merge area fits LDS


def sink_flash_ok(dtype, dim: int, vdim: int) -> bool:
    """Shapes the MFMA form of sink_attention covers (prompt portions; everything else takes the row kernel)."""
    return dtype == torch.bfloat16 and dim % 32 == 0 and dim <= 512 and vdim % 16 == 0 and vdim // 16 in SINK_FLASH_TILES


def sink_attention(q, kcache, vcache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile, sink, gate, out,
                   window: int, scale: float, qt: int, vt=None, split: bool = False, softcap: float = 0.0, out_rope=None):
    """Causal softmax attention of q [T, H, D] over paged keys [pages, 32, G, D] and values [pages, 32, G, V] (grouped
    heads), scores and weights in fp32; sink [H] adds exp(sink) to each head's denominator, gate [T, H] multiplies the
    head's output by its sigmoid.  `qt` query rows per work item (work_seq, work_tile).  With vt (transposed value
    pages [pages, G, V, 32], sink_flash_ok shapes, qt = 16): the MFMA form; split (V <= 128) lets the four waves of a
    workgroup share one (tile, head) and split its pages, for decode steps.  softcap > 0: scores
    softcap * tanh(scale q.k / softcap).  out_rope ([positions, V / 2, 2] (cos, sin), rotate-half pairs over the whole
    value width): each head's weighted sum is turned back by the query row's own position before the gate -- with
    values that were rotated by THEIR positions when cached, a value enters the output rotated by the distance (the
    MFMA form then needs V % 32 == 0)."""
    if _hip(q):
        torch.ops.dsse.sink_attention(q, kcache, vcache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile,
                                      sink, gate, out, window, scale, qt, vt, split, softcap, out_rope)
    else:
        lref.sink_attention(q, kcache, vcache, block_tables, q_start, q_len, ctx_len, sink, gate, out, window, scale, vt,
                            softcap, out_rope)


def gate_math(x, kind: int, p1=None, p2=None, c: float = 1.0):
    """In place on fp32 x [T, N] (a column slice is fine): 0: exp(-exp(p1) * softplus(x + p2)); 1: sigmoid(x);
    2: sigmoid(x)^(1 / c).  p1 and p2 hold N numbers, or N / k of them: each then serves k neighbouring columns (one
    rate per head beside one bias per head and channel)."""
    if _hip(x):
        torch.ops.dsse.gate_math(x, kind, p1, p2, c)
    else:
        lref.gate_math(x, kind, p1, p2, c)


def matrix_scan(q, k, v, decay, beta, state, q_start, q_len, ctx_len, state_slot, out, q_scale: float = 1.0):
    """Matrix-state recurrence per (sequence, head) continued from the slot state [slots, H, D, V] (fp32; zeros at
    position 0): S = a S; u = beta (v - S^T k) with beta (the delta rule), else u = v; S += k u^T; o = S^T (q_scale q).
    decay: None, [H], [T, H] or [T, H, D]; q, k [T, G, D], v [T, H, V] are fp32 (column slices are fine)."""
    if _hip(v):
        torch.ops.dsse.matrix_scan(q, k, v, decay, beta, state, q_start, q_len, ctx_len, state_slot, out, q_scale)
    else:
        lref.matrix_scan(q, k, v, decay, beta, state, q_start, q_len, ctx_len, state_slot, out, q_scale)


def scan_state_plain(state):
    """A GPU matrix state [slots, H, D, V] as the plain [.., D, V] matrices it stands for.  The scan kernels keep an
    entry tile-major ([H][V / 16][D][16]) when V is a multiple of 16; CPU tensors are plain already."""
    S, H, D, V = state.shape
    if not state.is_cuda or V % 16:
        return state
    return state.view(S, H, V // 16, D, 16).permute(0, 1, 3, 2, 4).reshape(S, H, D, V)


def scan_state_from_plain(plain):
    """The inverse of scan_state_plain for a GPU tensor: plain matrices -> the kernels' layout."""
    S, H, D, V = plain.shape
    if not plain.is_cuda or V % 16:
        return plain
    return plain.view(S, H, D, V // 16, 16).permute(0, 1, 3, 2, 4).reshape(S, H, D, V).contiguous()


SCAN_CHUNK = 64        # tokens per chunk of the two-level walk
SCAN_CHUNKED_FROM = 256  # rows of a prompt group from which matrix_scan_chunked pays


def scan_chunks(q_start: list, q_len: list, slots: list):
    """Host-side chunk lists of matrix_scan_chunked for sequences with the given first rows, lengths and state slots:
    (s_first, s_count, cmeta [7][chunks]) as Python lists (see the op for cmeta's rows)."""
    s_first, s_count = [], []
    rows = [[] for _ in range(7)]
    for r0, n, slot in zip(q_start, q_len, slots):
        k = -(-n // SCAN_CHUNK) if n > 0 else 0
        s_first.append(len(rows[0]))
        s_count.append(k)
        for i in range(k):
            cid, last = len(rows[0]), i == k - 1
            ln = min(SCAN_CHUNK, n - i * SCAN_CHUNK)
            for row, val in zip(rows, (r0 + i * SCAN_CHUNK, ln, 0 if last else ln, -1, -1 if last else cid, cid,
                                       slot if last else -1)):
                row.append(val)
    return s_first, s_count, rows


def matrix_scan_chunked(q, k, v, decay, state, q_start, q_len, ctx_len, state_slot, s_first, s_count, cmeta, scratch,
                        a_scratch, out, q_scale: float = 1.0):
    """matrix_scan without the delta rule for long prompt portions, as a two-level walk: chunks of SCAN_CHUNK tokens are
    walked in parallel from zeros, a carry gives every chunk its incoming state, and a second parallel walk writes the
    outputs and the slots' states.  decay: None, [H] or [T, H, D].  Chunk lists from scan_chunks; scratch
    [chunks, H, D, V] and a_scratch [chunks, H, D] (per-channel decays) are fp32 work areas."""
    if _hip(v):
        torch.ops.dsse.matrix_scan_chunked(q, k, v, decay, state, q_len, ctx_len, state_slot, s_first, s_count, cmeta,
                                           scratch, a_scratch, out, q_scale)
    else:
        lref.matrix_scan(q, k, v, decay, None, state, q_start, q_len, ctx_len, state_slot, out, q_scale)


def gated_head_norm(o, w, gate, eps: float, out, kind: int = 0):
    """out [T, H * V] (element type) = o / rms(o) per head * w (or no gain) * silu(gate); kind 1: * sigmoid(gate)."""
    if _hip(o):
        torch.ops.dsse.gated_head_norm(o, w, gate, eps, out, kind)
    else:
        lref.gated_head_norm(o, w, gate, eps, out, kind)


def rms_mix(ya, wa, yb, wb, eps: float, coef: float, out):
    """out (fp32) = coef * (rms-norm(ya) * wa + rms-norm(yb) * wb)."""
    if _hip(ya):
        torch.ops.dsse.rms_mix(ya, wa, yb, wb, eps, coef, out)
    else:
        lref.rms_mix(ya, wa, yb, wb, eps, coef, out)


def logit_cap(logits, scale: float, cap: float):
    """In place: logits * scale, then cap * tanh(. / cap) when cap > 0."""
    if _hip(logits):
        torch.ops.dsse.logit_cap(logits, scale, cap)
    else:
        lref.logit_cap(logits, scale, cap)


# ---------------------------------------------------------------------------------------------------------------------
# Designs on several residual streams with routed squared-ReLU experts.
def stream_mix(y, nsum: int, mult: float, streams, ids=None, embed=None, embed_scale: float = 1.0, out_w=None, mix=None,
               in_w=None, norm_w=None, eps: float = 0.0, h=None, total=None):
    """One pass over the S residual streams [M, S, W] (fp32) of each row, between two sublayers.  embed given: every
    stream = embed[ids] * embed_scale (a model's first step).  y given ([M * nsum, W] fp32, a row's nsum consecutive
    parts are summed first): x_t = sum_s mix[s, t] x_s + mult * out_w[t] * y for all streams at once.  in_w given: the
    next sublayer's input u = sum_s in_w[s] x_s, RMS-normed with the gain norm_w [W], into h (fp32 or the element
    type).  total given: the sum of the streams (fp32).  out_w, in_w [S], mix [S, S] and norm_w are fp32."""
    if _hip(streams):
        torch.ops.dsse.stream_mix(y, nsum, mult, streams, ids, embed, embed_scale, out_w, mix, in_w, norm_w, eps, h, total)
    else:
        lref.stream_mix(y, nsum, mult, streams, ids, embed, embed_scale, out_w, mix, in_w, norm_w, eps, h, total)


def act_rows(x, out, kind: int, params=None, gate=None):
    """out [M, F] (fp32 or the element type) = act(x) * sigmoid(gate) for fp32 x and gate (column slices are fine; gate
    may be None).  kind 0: identity; 1: xIELU, a_p z^2 + z / 2 for z > 0 else a_n (e^z - 1 - z) + z / 2 with
    params = fp32 (a_p, a_n); 2: relu(z)^2."""
    if _hip(x):
        torch.ops.dsse.act_rows(x, out, kind, params, gate)
    else:
        lref.act_rows(x, out, kind, params, gate)


def moe_route(z, correction, topk_idx, topk_w, groups: int, keep: int, scale: float, kind: int = 0):
    """Group-limited routing from fp32 logits z [M, E].  kind 0 (sigmoid): choice scores sigmoid(z) + correction [E]; of
    `groups` equal groups of neighbouring experts only the `keep` with the largest sum of their two best choice scores
    are eligible; the top experts by choice score get the weights sigmoid(z) / (their sum + 1e-20) * scale.  kind 1
    (softmax): scores softmax(z) over ALL experts (correction may be None), a group's score is its largest score, the
    chosen experts' weights are their scores as they are, times scale."""
    if _hip(z):
        torch.ops.dsse.moe_route(z, correction, topk_idx, topk_w, groups, keep, scale, kind)
    else:
        lref.moe_route(z, correction, topk_idx, topk_w, groups, keep, scale, kind)


# ---------------------------------------------------------------------------------------------------------------------
# Designs with bracketing norms, hashed bigram embeddings and per-layer token inputs.
def embed_pair_rows(ids, prev, positions, embed, pair, mul_prev: int, mul_cur: int, buckets: int, resid, x0=None,
                    prev_out=None, keep=None):
    """resid (fp32) = embed[ids] + pair[row] with row = (prev * mul_prev + ids * mul_cur) mod buckets, or the table's
    last row (`buckets`) at position 0; pair None: the plain embedding.  x0 (optional, element type, may be a column
    slice of a wider buffer) receives the same rows.  prev_out (optional, int32 [B], may be `prev` itself): the first B
    rows store their token there when keep[i] > 0 -- a decode slot's token becomes its next token's predecessor."""
    if _hip(resid):
        torch.ops.dsse.embed_pair_rows(ids, prev, positions, embed, pair, mul_prev, mul_cur, buckets, resid, x0, prev_out,
                                       keep)
    else:
        lref.embed_pair_rows(ids, prev, positions, embed, pair, mul_prev, mul_cur, buckets, resid, x0, prev_out, keep)


def add_norm_rows(y, nsum: int, g_add, resid, g_out, eps: float, out=None, out32=None):
    """The stream's step between sublayers of a design that norms a sublayer's input AND its output, in one pass over
    the row: y given ([M * nsum, W] fp32; a row's nsum consecutive parts are summed first, the grouped experts' slots):
    resid += y / rms(y) * g_add; out given (element type or fp32; a column slice of a wider buffer is fine):
    out = resid / rms(resid) * g_out, or the stream itself when g_out is None; out32 (fp32) receives that row unrounded
    (what a router reads).  Gains are fp32 [W]."""
    if _hip(resid):
        torch.ops.dsse.add_norm_rows(y, nsum, g_add, resid, g_out, eps, out, out32)
    else:
        lref.add_norm_rows(y, nsum, g_add, resid, g_out, eps, out, out32)


def token_gate_rows(x, ids, table, col0: int, out):
    """out [M, F] (element type) = gelu_tanh(x) * table[ids, col0 : col0 + F]: a gate computed from the stream times a
    slice of a per-token table.  x fp32 (a column slice is fine)."""
    if _hip(x):
        torch.ops.dsse.token_gate_rows(x, ids, table, col0, out)
    else:
        lref.token_gate_rows(x, ids, table, col0, out)



SIDE_FUSED_MAX_ROWS = 64   # steps of up to this many rows run a token input as one launch (each row's workgroup reads
                           # both small weights from L2; prompt-sized steps amortise them in two GEMMs instead)


def token_side_fits(rows: int, width: int, cols: int) -> bool:
    """Steps that token_side_rows serves: decode-sized, the row and the gate's columns in 64 KB of LDS."""
    return rows <= SIDE_FUSED_MAX_ROWS and (width + cols + 16) * 4 <= 64 * 1024


def token_side_rows(y, nsum: int, g_add, resid, ids, table, col0: int, gate_w, proj_w, side_norm, g_out, eps: float,
                    out=None, out32=None):
    """A per-layer token input in ONE launch, for decode-sized steps: the pending add_norm_rows (y, nsum, g_add); the
    gate g = gelu_tanh(gate_w x) * table[ids, col0 : col0 + F] on the stream rounded to the weights' type; the
    back-projection proj_w g, RMS-normed, times side_norm, added to the stream; then out (element type; a column slice
    is fine) = the stream normed with g_out (or itself), out32 the same unrounded."""
    if _hip(resid):
        torch.ops.dsse.token_side_rows(y, nsum, g_add, resid, ids, table, col0, gate_w, proj_w, side_norm, g_out, eps, out,
                                       out32)
    else:
        lref.token_side_rows(y, nsum, g_add, resid, ids, table, col0, gate_w, proj_w, side_norm, g_out, eps, out, out32)
