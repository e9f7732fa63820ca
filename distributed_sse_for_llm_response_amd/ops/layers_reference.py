"""Plain-PyTorch references of the layer-mechanism ops (``ops/layers.py``): exact semantics of the HIP kernels in
``csrc/kernels/{gemm_rowmajor,norms,latent_attention,recurrent,moe,stream_ops,sink_attention,matrix_scan,multistream}.hip``,
including the cache and state layouts.

As with ``ops/reference.py`` they are the numerics oracle of the kernel tests and the CPU execution path of the engine
(scheduler, cache and state-slot plumbing run here without a GPU).  Everything is computed in fp32 on whatever element
type the tensors carry.
"""
from __future__ import annotations

import math

import torch

PAGE = 32


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def gemm_rm(x, w, out, bias=None, act=0):
    y = torch.matmul(x.float(), w.float().transpose(-1, -2))
    if bias is not None:
        y = y + bias.float().unsqueeze(-2)
    if act == 1:
        y = gelu_tanh(y)
    out.copy_(y.to(out.dtype))


def scalar_norm(y, g, resid, xb, eps, nsum=1):
    src = resid if y is None else y.view(resid.shape[0], nsum, -1).sum(1)
    n = src * (g.float().reshape(()) / torch.sqrt(src.pow(2).mean(-1, keepdim=True) + eps))
    if y is None:
        xb.copy_(n.to(xb.dtype))
    else:
        resid.add_(n)
        xb.copy_(resid.to(xb.dtype))


def embed_rows(ids, embed, resid, xb):
    M = resid.shape[0]
    idx = ids[:M].long()
    idx = torch.where((idx >= 0) & (idx < embed.shape[0]), idx, torch.zeros_like(idx))
    rows = embed[idx]
    resid.copy_(rows.float())
    xb.copy_(rows)


def _rotate(v, cs):
    """v [..., dr] interleaved pairs, cs [..., dr / 2, 2] (cos, sin)."""
    a, b = v[..., 0::2], v[..., 1::2]
    out = torch.empty_like(v)
    out[..., 0::2] = a * cs[..., 0] - b * cs[..., 1]
    out[..., 1::2] = b * cs[..., 0] + a * cs[..., 1]
    return out


def vt_position(off):
    """Place of token `off` (0..31) inside a transposed latent page (the MFMA attention's key order)."""
    return ((off & 15) >> 2) * 8 + ((off >> 4) & 1) * 4 + (off & 3)


def latent_kv_write(ckr, norm_w, positions, slots, rope, cache, eps, vt=None):
    T, rk = ckr.shape[0], norm_w.numel()
    flat = cache.view(-1, cache.shape[-1])
    c = ckr[:, :rk]
    c = c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    pos = positions[:T].long().clamp(0, rope.shape[0] - 1)
    kr = _rotate(ckr[:, rk:], rope[pos])
    row = torch.cat([c, kr], dim=-1).to(cache.dtype)
    sl = slots[:T].long()
    ok = (sl >= 0) & (sl < flat.shape[0])
    flat[sl[ok]] = row[ok]
    if vt is not None:
        good = sl[ok]
        vt[good // PAGE, :, vt_position(good % PAGE)] = row[ok][:, :rk]


def latent_attention(q, q_abs, cache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile, rope, out, window,
                     scale, qt, vt=None):
    """With vt the values come from the transposed pages (the same numbers in another place), so a wrong place shows."""
    rk = q_abs.shape[2]
    dr = cache.shape[2] - rk
    dn = q.shape[2] - dr
    flat = cache.view(-1, cache.shape[-1]).float()
    done = set()
    for s, t in zip(work_seq.tolist(), work_tile.tolist()):
        ql = int(q_len[s])
        for i in range(qt):
            off = t * qt + i
            if off >= ql or (s, off) in done:
                continue
            done.add((s, off))
            row = int(q_start[s]) + off
            pos = int(ctx_len[s]) - ql + off
            lo = max(0, pos - window + 1)
            j = torch.arange(lo, pos + 1)
            rows = block_tables[s].long()[j // PAGE] * PAGE + j % PAGE
            kv = flat[rows]  # [keys, rk + dr]
            qr = _rotate(q[row, :, dn:].float(), rope[min(max(pos, 0), rope.shape[0] - 1)])
            sc = (q_abs[row].float() @ kv[:, :rk].t() + qr @ kv[:, rk:].t()) * scale
            p = torch.softmax(sc, dim=-1)
            val = kv[:, :rk] if vt is None else vt[rows // PAGE, :, vt_position(rows % PAGE)].float()
            out[row] = (p @ val).to(out.dtype)


def conv_state(inp, taps, bias, tail, q_start, q_len, ctx_len, state_slot, out, out_b, in_bias=None, act=0):
    """inp may be a column slice of a wider buffer; act 1: SiLU on the output (the tail keeps raw inputs); act 2: the
    row's own input is added to its output (inp + conv(inp))."""
    K = taps.shape[1]
    tp = taps.float()
    ib = 0.0 if in_bias is None else in_bias.float()
    for s in range(q_len.numel()):
        ql = int(q_len[s])
        if ql <= 0:
            continue
        r0, slot = int(q_start[s]), int(state_slot[s])
        fresh = int(ctx_len[s]) - ql == 0
        prev = torch.zeros(K - 1, inp.shape[1]) if fresh or K == 1 else tail[slot].clone()
        seq = torch.cat([prev, inp[r0:r0 + ql].float() + ib])
        y = torch.zeros(ql, inp.shape[1]) if bias is None else bias.float().expand(ql, -1).clone()
        for k in range(K):
            y = y + seq[k:k + ql] * tp[:, k]
        if act == 1:
            y = torch.nn.functional.silu(y)
        elif act == 2:
            y = y + seq[K - 1:]
        if out is not None:
            out[r0:r0 + ql] = y
        if out_b is not None:
            out_b[r0:r0 + ql] = y.to(out_b.dtype)
        if K > 1:
            tail[slot] = seq[ql:]


def lru_scan(u, gates, y, lam, state, q_start, q_len, ctx_len, state_slot, out, c, y_bias=None, coeff=True):
    """coeff: first turn every row's gate pre-activations [recurrence | input] into the coefficients (a | b) of
    S = a S + b, in place; then walk each sequence's rows.  y is the gelu branch before its bias and gelu."""
    C = u.shape[1]
    bw = gates.shape[2] // 2
    if coeff:
        sp = torch.nn.functional.softplus(lam.float()).view(1, -1, bw)
        log_a = -c * torch.sigmoid(gates[:, :, :bw]) * sp
        b = torch.sqrt(-torch.expm1(2.0 * log_a)) * torch.sigmoid(gates[:, :, bw:]) * u.view(u.shape[0], -1, bw)
        gates[:, :, :bw] = torch.exp(log_a)
        gates[:, :, bw:] = b
    yb = 0.0 if y_bias is None else y_bias.float()
    for s in range(q_len.numel()):
        ql = int(q_len[s])
        if ql <= 0:
            continue
        r0, slot = int(q_start[s]), int(state_slot[s])
        S = torch.zeros(C) if int(ctx_len[s]) - ql == 0 else state[slot].clone()
        for t in range(ql):
            g = gates[r0 + t]
            S = g[:, :bw].reshape(C) * S + g[:, bw:].reshape(C)
            out[r0 + t] = (S * gelu_tanh(y[r0 + t].float() + yb)).to(out.dtype)
        state[slot] = S


def moe_topk(logits, topk_idx, topk_w):
    z = torch.nan_to_num(logits.float(), nan=0.0)
    val, idx = torch.topk(z, topk_idx.shape[1], dim=-1)
    topk_idx.copy_(idx.to(torch.int32))
    topk_w.copy_(torch.softmax(val, dim=-1))


def moe_router(x, w, b, topk_idx, topk_w):
    z = x.float() @ w.float().t()
    if b is not None:
        z = z + b.float()
    z = torch.nan_to_num(z, nan=0.0)
    val, idx = torch.topk(z, topk_idx.shape[1], dim=-1)
    topk_idx.copy_(idx.to(torch.int32))
    topk_w.copy_(torch.softmax(val, dim=-1))


def moe_ffn(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, out):
    xf = x.float()

    def ffn(h, g, u, d):
        return (torch.nn.functional.silu(h @ g.float().t()) * (h @ u.float().t())) @ d.float().t()

    acc = torch.zeros_like(out)
    for e in range(gate.shape[0]):
        sel = topk_idx == e
        rows = sel.any(-1)
        if rows.any():
            acc[rows] += ffn(xf[rows], gate[e], up[e], down[e]) * (topk_w * sel)[rows].sum(-1, keepdim=True)
    if sgate is not None:
        acc += ffn(xf, sgate, sup, sdown)
    out.copy_(acc)


def moe_grouped(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, o):
    """o [M * S, W]: slot k < top of row r = weight * expert output, slot `top` = the shared expert.  gate None: the
    experts are down(relu(up x)^2), without a gate."""
    xf = x.float()
    M, top = topk_idx.shape
    S = top + (1 if sgate is not None else 0)
    ov = o.view(M, S, -1)

    def ffn(h, g, u, d):
        if g is None:
            return torch.relu(h @ u.float().t()).pow(2).to(x.dtype).float() @ d.float().t()
        return (torch.nn.functional.silu(h @ g.float().t()) * (h @ u.float().t())) @ d.float().t()

    for e in range(up.shape[0]):
        rows, ks = torch.nonzero(topk_idx == e, as_tuple=True)
        if rows.numel():
            ov[rows, ks] = ffn(xf[rows], None if gate is None else gate[e], up[e], down[e]) * topk_w[rows, ks].unsqueeze(-1)
    if sgate is not None:
        ov[:, top] = ffn(xf, sgate, sup, sdown)


# ---------------------------------------------------------------------------------------------------------------------
# Pre-norm designs with matrix-state mixers (models/surodra.py)
def stream_step(y, mult, resid, ids, embed, vec, alpha, w, b, xb):
    """resid += mult * y (y given) + embed[ids] (embed given) + vec (vec given); then, with a norm (w given),
    xb = tanh(alpha * resid) * w + b."""
    M = resid.shape[0]
    if y is not None:
        resid.add_(y.float() * mult)
    if embed is not None:
        idx = ids[:M].long()
        idx = torch.where((idx >= 0) & (idx < embed.shape[0]), idx, torch.zeros_like(idx))
        resid.add_(embed[idx].float())
    if vec is not None:
        resid.add_(vec.float())
    if w is not None:
        xb.copy_((torch.tanh(alpha.float().reshape(()) * resid) * w.float() + b.float()).to(xb.dtype))


def gated_act(gu, h, kind):
    """h = act(gu[:, :F]) * gu[:, F:]; kind 0 SiLU, 1 gelu (tanh form)."""
    F = h.shape[1]
    g, u = gu[:, :F].float(), gu[:, F:].float()
    h.copy_(((torch.nn.functional.silu(g) if kind == 0 else gelu_tanh(g)) * u).to(h.dtype))


def rotate_half_rows(v, cs, dims):
    """v [T, heads, D], cs [T, dims / 2, 2]: coordinate i < dims / 2 pairs with i + dims / 2."""
    half = dims // 2
    a, b = v[..., :half], v[..., half:dims]
    c, s = cs[:, None, :, 0], cs[:, None, :, 1]
    out = v.clone()
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def norm_rope_rows(x, norm_w, positions, rope, out, out_rows, norm_kind, eps, scale, out_t=None):
    """x [T, heads, D] fp32 -> out rows (out_rows[t], or t) as [heads, D] in out's type.  norm_kind 1: RMS norm over
    the whole row (all heads at once) times norm_w [heads * D]; 2: every head divided by sqrt(sum of squares + eps);
    3: RMS norm per head times norm_w [D] (one gain vector for all heads);
    then the rotate-half rotation of the leading 2 * rope.shape[1] coordinates at positions[t]; then times scale.
    Rows whose out_rows entry is negative are skipped."""
    T, nh, D = x.shape
    v = x.float()
    if norm_kind == 1:
        flat = v.reshape(T, nh * D)
        v = (flat / torch.sqrt(flat.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()).view(T, nh, D)
    elif norm_kind == 2:
        v = v / torch.sqrt(v.pow(2).sum(-1, keepdim=True) + eps)
    elif norm_kind == 3:
        v = v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        if norm_w is not None:
            v = v * norm_w.float()
    if rope is not None and rope.shape[1] > 0:
        pos = positions[:T].long().clamp(0, rope.shape[0] - 1)
        v = rotate_half_rows(v, rope[pos], 2 * rope.shape[1])
    v = (v * scale).to(out.dtype)
    if out_rows is None:
        out.copy_(v)
    else:
        flat_out = out.view(-1, nh, D)
        r = out_rows[:T].long()
        ok = (r >= 0) & (r < flat_out.shape[0])
        flat_out[r[ok]] = v[ok]
        if out_t is not None:  # [pages, heads, D, PAGE], the token at vt_position(offset)
            good = r[ok]
            out_t[good // PAGE, :, :, vt_position(good % PAGE)] = v[ok]


def sink_attention(q, kcache, vcache, block_tables, q_start, q_len, ctx_len, sink, gate, out, window, scale, vt=None,
                   softcap=0.0, out_rope=None):
    """Softmax attention over paged keys [pages, PAGE, G, D] and values [pages, PAGE, G, V] with grouped heads; the
    denominator also holds exp(sink[h]) when sink is given; the head's output is multiplied by sigmoid(gate[row, h])
    when gate is given.  With vt the values come from the transposed pages [pages, G, V, PAGE].  softcap > 0: scores
    softcap * tanh(. / softcap).  out_rope [positions, V / 2, 2]: the head's output is turned BACK by the query's
    position (rotate-half pairs), undoing the rotation of a value rotated by that same position."""
    H = q.shape[1]
    G = kcache.shape[2]
    kf = kcache.view(-1, G, kcache.shape[3]).float()
    vf = vcache.view(-1, G, vcache.shape[3]).float()
    grp = torch.arange(H) // (H // G)
    for s in range(q_len.numel()):
        ql = int(q_len[s])
        if ql <= 0:
            continue
        r0, p0 = int(q_start[s]), int(ctx_len[s]) - ql
        bt = block_tables[s].long()
        for i in range(ql):
            pos = p0 + i
            j = torch.arange(max(0, pos - window + 1), pos + 1)
            rows = bt[j // PAGE] * PAGE + j % PAGE
            k, v = kf[rows][:, grp], vf[rows][:, grp]                       # [keys, H, D], [keys, H, V]
            if vt is not None:  # the same numbers from the transposed pages, so a wrong place shows
                v = vt[rows // PAGE, :, :, vt_position(rows % PAGE)].float()[:, grp]
            sc = torch.einsum("hd,jhd->hj", q[r0 + i].float(), k) * scale
            if softcap > 0:
                sc = softcap * torch.tanh(sc / softcap)
            mx = sc.max(-1, keepdim=True).values
            if sink is not None:
                mx = torch.maximum(mx, sink.float()[:, None])
            e = torch.exp(sc - mx)
            den = e.sum(-1, keepdim=True)
            if sink is not None:
                den = den + torch.exp(sink.float()[:, None] - mx)
            o = torch.einsum("hj,jhv->hv", e / den, v)
            if out_rope is not None:
                cs = out_rope[min(pos, out_rope.shape[0] - 1)].float().clone()
                cs[:, 1] = -cs[:, 1]
                o = rotate_half_rows(o[None], cs[None], 2 * out_rope.shape[1])[0]
            if gate is not None:
                o = o * torch.sigmoid(gate[r0 + i].float())[:, None]
            out[r0 + i] = o.to(out.dtype)


def gate_math(x, kind, p1, p2, c):
    """In place on fp32 x [T, N]: kind 0: exp(-exp(p1) * softplus(x + p2)) (p1, p2 [N]); 1: sigmoid(x);
    2: sigmoid(x)^(1 / c) as exp(logsigmoid(x) / c)."""
    if kind == 0:  # p1, p2 may be shorter than a row: each entry then serves a run of neighbouring columns
        N = x.shape[1]
        a = p1.float().repeat_interleave(N // p1.numel())
        b = p2.float().repeat_interleave(N // p2.numel())
        x.copy_(torch.exp(-torch.exp(a) * torch.nn.functional.softplus(x + b)))
    elif kind == 1:
        x.copy_(torch.sigmoid(x))
    else:
        x.copy_(torch.exp(torch.nn.functional.logsigmoid(x) / c))


def matrix_scan(q, k, v, decay, beta, state, q_start, q_len, ctx_len, state_slot, out, q_scale=1.0):
    """Matrix-state recurrence per (sequence, head), continued from the sequence's slot (zeros at position 0):
    S = a S; with beta (delta rule) u = beta (v - S^T k) else u = v; S += k u^T; o = S^T q.  q, k [T, G, D] (head h
    reads group h / (H / G)), v [T, H, V], state [slots, H, D, V] fp32, out [T, H, V] fp32.  decay: None, [H] (fixed
    per head), [T, H] (per row and head) or [T, H, D] (per row, head and key channel).  q is multiplied by q_scale."""
    T, H, V = v.shape
    G, D = k.shape[1], k.shape[2]
    grp = torch.arange(H) // (H // G)
    for s in range(q_len.numel()):
        ql = int(q_len[s])
        if ql <= 0:
            continue
        r0, slot = int(q_start[s]), int(state_slot[s])
        S = torch.zeros(H, D, V) if int(ctx_len[s]) - ql == 0 else state[slot].clone()
        for t in range(r0, r0 + ql):
            kt, qt, vt = k[t].float()[grp], q[t].float()[grp] * q_scale, v[t].float()
            if decay is not None:
                a = decay.float() if decay.dim() == 1 else decay[t].float()
                S = S * (a[:, None, None] if a.dim() == 1 else a[:, :, None])
            if beta is not None:
                vt = beta[t].float()[:, None] * (vt - torch.einsum("hdv,hd->hv", S, kt))
            S = S + kt[:, :, None] * vt[:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, qt)
        state[slot] = S


def gated_head_norm(o, w, gate, eps, out, kind=0):
    """out [T, H * V] = o / rms(o over V) * w (w [V] or None) * silu(gate [T, H * V]) (kind 1: sigmoid(gate))."""
    T, H, V = o.shape
    n = o.float() / torch.sqrt(o.float().pow(2).mean(-1, keepdim=True) + eps)
    if w is not None:
        n = n * w.float()
    g = torch.sigmoid(gate.float()) if kind == 1 else torch.nn.functional.silu(gate.float())
    out.copy_((n.reshape(T, H * V) * g).to(out.dtype))


def rms_mix(ya, wa, yb, wb, eps, coef, out):
    """out (fp32) = coef * (ya / rms(ya) * wa + yb / rms(yb) * wb), rows of the model width."""
    def n(y, w):
        return y.float() / torch.sqrt(y.float().pow(2).mean(-1, keepdim=True) + eps) * w.float()

    out.copy_(coef * (n(ya, wa) + n(yb, wb)))


def logit_cap(logits, scale, cap):
    """In place: logits *= scale; with cap > 0 then cap * tanh(logits / cap)."""
    logits.mul_(scale)
    if cap > 0:
        logits.copy_(cap * torch.tanh(logits / cap))


# ---------------------------------------------------------------------------------------------------------------------
# Designs on several residual streams with routed squared-ReLU experts (models/dironex.py)
def stream_mix(y, nsum, mult, streams, ids, embed, embed_scale, out_w, mix, in_w, norm_w, eps, h, total):
    """streams [M, S, W] fp32.  embed given: every stream = embed[ids] * embed_scale.  y given ([M * nsum, W], a row's
    nsum consecutive parts summed first): x_t = sum_s mix[s, t] x_s + mult * out_w[t] * y, all streams at once from the
    old ones.  in_w given: u = sum_s in_w[s] x_s and h = u / rms(u) * norm_w in h's type.  total given: sum_s x_s."""
    M, S, W = streams.shape
    if embed is not None:
        idx = ids[:M].long()
        idx = torch.where((idx >= 0) & (idx < embed.shape[0]), idx, torch.zeros_like(idx))
        streams.copy_((embed[idx].float() * embed_scale)[:, None, :].expand(M, S, W))
    if y is not None:
        ys = y.float().view(M, nsum, W).sum(1)
        streams.copy_(torch.einsum("st,msw->mtw", mix.float(), streams) + mult * out_w.float()[None, :, None] * ys[:, None])
    if in_w is not None:
        u = torch.einsum("s,msw->mw", in_w.float(), streams)
        h.copy_((u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()).to(h.dtype))
    if total is not None:
        total.copy_(streams.sum(1))


def act_rows(x, out, kind, params, gate):
    """out = act(x) * sigmoid(gate) (gate given).  kind 0: identity; 1: a_p z^2 + z / 2 for z > 0, else
    a_n (e^z - 1 - z) + z / 2, with params = (a_p, a_n); 2: relu(z)^2."""
    z = x.float()
    if kind == 1:
        ap, an = params.float()[0], params.float()[1]
        z = torch.where(z > 0, ap * z * z + 0.5 * z, an * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z)
    elif kind == 2:
        z = torch.relu(z).pow(2)
    if gate is not None:
        z = z * torch.sigmoid(gate.float())
    out.copy_(z.to(out.dtype))


def moe_route(z, correction, topk_idx, topk_w, groups, keep, scale, kind=0):
    """kind 1: scores softmax(z) over all experts, a group's score is its largest score, the weights are the chosen
    scores as they are (times scale).  kind 0: router logits z [M, E] fp32 -> the `top` experts with the largest sigmoid(z) + correction among the experts of
    the `keep` best of `groups` equal groups of neighbours (a group's score: the sum of its two largest such values);
    weights: the chosen sigmoid(z) over their sum (+ 1e-20), times scale.  Ties go to the lower index."""
    M, E = z.shape
    top = topk_idx.shape[1]
    zz = torch.nan_to_num(z.float(), nan=0.0)
    s = torch.softmax(zz, dim=-1) if kind == 1 else torch.sigmoid(zz)
    choice = s + correction.float() if correction is not None else s.clone()
    if groups > 1:
        per = choice.view(M, groups, E // groups)
        gscore = per.max(-1).values if kind == 1 else per.topk(min(2, E // groups), dim=-1).values.sum(-1)
        order = torch.argsort(gscore, dim=-1, descending=True, stable=True)[:, :keep]
        allow = torch.zeros(M, groups, dtype=torch.bool).scatter_(1, order, True)
        choice = per.masked_fill(~allow[:, :, None], float("-inf")).reshape(M, E)
    idx = torch.argsort(choice, dim=-1, descending=True, stable=True)[:, :top]
    w = s.gather(1, idx)
    topk_idx.copy_(idx.to(torch.int32))
    topk_w.copy_(w * scale if kind == 1 else w / (w.sum(-1, keepdim=True) + 1e-20) * scale)


# ---------------------------------------------------------------------------------------------------------------------
# Designs with bracketing norms, hashed bigram embeddings and per-layer token inputs (models/murulorn.py)
def embed_pair_rows(ids, prev, positions, embed, pair, mul_prev, mul_cur, buckets, resid, x0, prev_out, keep):
    """resid (fp32) = embed[ids] + pair[row], row = (prev * mul_prev + ids * mul_cur) mod buckets, or `buckets` (the
    table's last row) at position 0; x0 (optional, element type, may be a column slice) receives the same rows;
    prev_out (optional, [B]): prev_out[i] = ids[i] for the first B rows whose keep[i] > 0 (decode slots remember their
    token as the next one's predecessor)."""
    M = resid.shape[0]
    idx = ids[:M].long()
    idx = torch.where((idx >= 0) & (idx < embed.shape[0]), idx, torch.zeros_like(idx))
    rows = embed[idx].float()
    if pair is not None:
        pv = prev[:M].long().clamp(min=0)
        r = (pv * mul_prev + idx * mul_cur) % buckets
        r = torch.where(positions[:M].long() <= 0, torch.full_like(r, buckets), r)
        rows = rows + pair[r].float()
    if prev_out is not None:
        B = prev_out.shape[0]
        new = torch.where(keep[:B] > 0, ids[:B].to(prev_out.dtype), prev_out) if keep is not None else ids[:B]
        prev_out.copy_(new)
    resid.copy_(rows)
    if x0 is not None:
        x0.copy_(rows.to(x0.dtype))


def add_norm_rows(y, nsum, g_add, resid, g_out, eps, out, out32):
    """The residual stream's step of a design with a norm before AND after each sublayer.  y given ([M * nsum, W] fp32,
    a row's nsum consecutive parts are summed first): resid += y / rms(y) * g_add.  out given (element type or fp32, may
    be a column slice): out = resid / rms(resid) * g_out, or resid itself without g_out; out32 (optional, fp32) receives
    the same row unrounded."""
    if y is not None:
        v = y.float().view(resid.shape[0], nsum, -1).sum(1)
        resid.add_(v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * g_add.float())
    if out is not None or out32 is not None:
        n = resid
        if g_out is not None:
            n = resid / torch.sqrt(resid.pow(2).mean(-1, keepdim=True) + eps) * g_out.float()
        if out is not None:
            out.copy_(n.to(out.dtype))
        if out32 is not None:
            out32.copy_(n)


def token_gate_rows(x, ids, table, col0, out):
    """out [M, F] = gelu_tanh(x) * table[ids, col0 : col0 + F] for fp32 x (a column slice is fine)."""
    F = x.shape[1]
    idx = ids[:x.shape[0]].long()
    idx = torch.where((idx >= 0) & (idx < table.shape[0]), idx, torch.zeros_like(idx))
    out.copy_((gelu_tanh(x.float()) * table[idx, col0:col0 + F].float()).to(out.dtype))


def token_side_rows(y, nsum, g_add, resid, ids, table, col0, gate_w, proj_w, side_norm, g_out, eps, out, out32):
    """A per-layer token input in one call: the pending add + norm; g = gelu_tanh(gate_w x) * table[ids, col0 : col0 + F]
    on the stream rounded to the weights' type; resid += proj_w g, RMS-normed, times side_norm; then out = the stream
    normed with g_out (or itself)."""
    add_norm_rows(y, nsum, g_add, resid, None, eps, None, None)
    F = gate_w.shape[0]
    sg = resid.to(gate_w.dtype).float() @ gate_w.float().t()
    sh = torch.empty(resid.shape[0], F, dtype=gate_w.dtype)
    token_gate_rows(sg, ids, table, col0, sh)
    add_norm_rows(sh.float() @ proj_w.float().t(), 1, side_norm, resid, g_out, eps, out, out32)
