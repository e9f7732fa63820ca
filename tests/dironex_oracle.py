"""Plain float64 oracle of the Dironex design, written from its equations: one function per mechanism, whole sequences,
no cache, no batching, no code shared with the package.  ``forward(config dict, {tensor name: tensor}, tokens)`` returns
(logits [T, vocab], the summed streams after every layer run).

Notation: W x for a stored [out, in] weight; rms(v) = v / sqrt(mean(v^2) + eps).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def softplus(x):
    return torch.nn.functional.softplus(x)


# ------------------------------------------------------------------------------------------------- rotation
def yarn_frequencies(rot: dict) -> tuple:
    """(frequencies [dims / 2], amplitude) of a rotation entry {base, dims, scaling?}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(v, rot: dict, first_pos: int = 0):
    """v [T, ..., D]: the leading rot.dims coordinates rotate, i paired with i + dims / 2; the rest pass."""
    dims = int(rot["dims"])
    f, amp = yarn_frequencies(rot)
    T = v.shape[0]
    ang = (first_pos + torch.arange(T, dtype=F64))[:, None] * f[None, :]
    shape = [T] + [1] * (v.dim() - 2) + [dims // 2]
    c, s = (ang.cos() * amp).view(shape), (ang.sin() * amp).view(shape)
    a, b = v[..., : dims // 2], v[..., dims // 2: dims]
    out = v.clone()
    out[..., : dims // 2] = a * c - b * s
    out[..., dims // 2: dims] = b * c + a * s
    return out


# ------------------------------------------------------------------------------------------------- mixers
def causal_softmax(scores, window=None):
    """scores [H, T, T] -> weights; row i sees j <= i (and i - j < window)."""
    T = scores.shape[-1]
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & (i - j < window)
    return torch.softmax(scores.masked_fill(~ok, float("-inf")), dim=-1)


def latent_attention(h, m: dict, w: dict, eps: float):
    """h [T, W]; w: the mixer's tensors by their last name part."""
    T = h.shape[0]
    H, dn, dr, dv, rk = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    cq = rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(T, H, dn + dr)
    ckr = h @ w["dkv"].T
    c = rms(ckr[:, :rk], eps) * w["dkv.norm"]
    kr = rotate_half(ckr[:, rk:], m["rot"])                         # [T, dr], one for all heads
    qn, qr = q[..., :dn], rotate_half(q[..., dn:], m["rot"])
    kn = (c @ w["uk"].T).view(T, H, dn)
    v = (c @ w["uv"].T).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", qn, kn) + torch.einsum("ihd,jd->hij", qr, kr)) * float(m["scale"])
    p = causal_softmax(scores)
    o = torch.einsum("hij,jhv->ihv", p, v).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ w["g"].T)
    return o @ w["o"].T


def window_attention(h, m: dict, w: dict, eps: float):
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    q = rms((h @ w["q"].T).view(T, H, D), eps) * w["q.norm"]
    k = rms((h @ w["k"].T).view(T, G, D), eps) * w["k.norm"]
    v = (h @ w["v"].T).view(T, G, V)
    grp = torch.arange(H) // (H // G)
    scores = torch.einsum("ihd,jhd->hij", q, k[:, grp]) * float(m["scale"])
    window = (m.get("mask") or {}).get("size")
    p = causal_softmax(scores, None if window is None else int(window))
    o = torch.einsum("hij,jhv->ihv", p, v[:, grp]).reshape(T, H * V)
    return o @ w["o"].T


# ------------------------------------------------------------------------------------------------- feed-forward
def xielu(z, p, q):
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (torch.expm1(z) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def dense_ff(h, w: dict):
    return xielu(h @ w["up"].T, w["act"][0], w["act"][1]) @ w["down"].T


def route(z, correction, r: dict):
    """Router logits z [T, E] -> (chosen experts [T, top], their weights [T, top])."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(z)
    choice = s + correction
    g = r.get("groups")
    if g:
        count, keep = int(g["count"]), int(g["keep"])
        per = choice.view(-1, count, E // count)
        gscore = per.topk(min(2, E // count), dim=-1).values.sum(-1)
        kept = gscore.topk(keep, dim=-1).indices
        allow = torch.zeros_like(gscore, dtype=torch.bool).scatter_(1, kept, True)
        choice = per.masked_fill(~allow[:, :, None], float("-inf")).reshape(-1, E)
    idx = choice.topk(top, dim=-1).indices
    ws = s.gather(1, idx)
    return idx, ws / (ws.sum(-1, keepdim=True) + 1e-20) * float(r["scale"])


def moe_ff(h, f: dict, w: dict):
    idx, wt = route(h @ w["router"].T, w["correction"], f["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wt[t]):
            out[t] += a * (torch.relu(w[f"e{e}.up"] @ h[t]) ** 2) @ w[f"e{e}.down"].T
    return out


# ------------------------------------------------------------------------------------------------- layer
def input_conv(h, taps_w):
    """h + conv(h): conv(h)_t = sum_j w[:, j] h_(t - taps + 1 + j), zeros before the start."""
    T, taps = h.shape[0], taps_w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, h.shape[1], dtype=h.dtype), h])
    out = h.clone()
    for j in range(taps):
        out += pad[j:j + T] * taps_w[:, j]
    return out


def sublayer(streams, hc, norm_w, canon, fn, mult: float, eps: float):
    """streams [S, T, W] -> new streams.  hc = (in [S], out [S], mix [S, S] indexed [from, to]) or None (one stream,
    plain residual)."""
    if hc is None:
        u = streams[0]
    else:
        u = torch.einsum("s,stw->tw", hc[0], streams)
    h = rms(u, eps) * norm_w
    if canon is not None:
        h = input_conv(h, canon)
    y = fn(h)
    if hc is None:
        return streams + mult * y[None]
    return torch.einsum("sr,stw->rtw", hc[2], streams) + mult * hc[1][:, None, None] * y[None]


def layer_order(cfg: dict) -> list:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, k = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * k + list(range(b, n))


def forward(cfg: dict, tensors: dict, tokens):
    t64 = {k: v.to(F64) for k, v in tensors.items()}
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    S = int(cfg.get("streams", 0))
    x = t64["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    streams = torch.stack([x] * max(S, 1))
    trace = []
    for i in layer_order(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        mix_w = {k[len(p) + 4:]: v for k, v in t64.items() if k.startswith(p + "mix.")}
        mlp_w = {k[len(p) + 4:]: v for k, v in t64.items() if k.startswith(p + "mlp.")}
        mixer = {"latent_attention": latent_attention, "attention": window_attention}[L["type"]]
        hc = (lambda q: (t64[p + q + ".in"], t64[p + q + ".out"], t64[p + q + ".mix"])) if S else (lambda q: None)
        canon = (lambda q: t64[p + q]) if cfg.get("canon") else (lambda q: None)
        streams = sublayer(streams, hc("hc1"), t64[p + "norm1"], canon("canon1"),
                           lambda h: mixer(h, L["mixer"], mix_w, eps), mult, eps)
        f = L.get("mlp")
        if f:
            ff = (lambda h: dense_ff(h, mlp_w)) if f["kind"] == "dense" else (lambda h: moe_ff(h, f, mlp_w))
            streams = sublayer(streams, hc("hc2"), t64[p + "norm2"], canon("canon2"), ff, mult, eps)
        trace.append(streams.sum(0))
    x = rms(streams.sum(0), eps) * t64["final.norm"]
    return x @ t64["head"].T, trace
