"""Plain, slow oracle of the Murulorn design: one function per mechanism, whole sequences only, no cache, no batching.

Written from the design's equations in float64 and shares no code with the package: the tests compare the engine (its
kernels, caches, state slots and scheduler) with this.  Inputs: the configuration as the dictionary a checkpoint's
``config.json`` holds, and the weights as {tensor name: tensor}.

Notation: ``x`` is the residual stream [T, W], ``n(v, g) = v / sqrt(mean(v^2) + eps) * g``.  A layer is
``x += n(mixer(n(x, 1 + a1)), 1 + b1); x += n(ff(n(x, 1 + a2)), 1 + b2); x += n(side(x, token), s)``.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def offset_norm(v, gain, eps):
    """RMS norm whose stored gain sits around zero."""
    return rms(v, eps) * (1.0 + gain)


def embedding(cfg: dict, w: dict, tokens):
    """Token rows plus hashed rows of (previous token, token) pairs; a sequence's first token takes the table's last row."""
    x = w["embed"][tokens]
    b = (cfg.get("embedding") or {}).get("bigram")
    if b:
        n = int(b["buckets"])
        rows = [n] + [(int(tokens[t - 1]) * int(b["mul_prev"]) + int(tokens[t]) * int(b["mul_cur"])) % n
                      for t in range(1, len(tokens))]
        x = x + w["bigram"][torch.tensor(rows)]
    return x


def rotate_pairs(v, angle_sign: float, base: float, dims: int, positions):
    """Neighbouring coordinates (2i, 2i + 1) of the first `dims` of v [T, heads, D] turn by sign * pos * base^(-2i/dims)."""
    half = dims // 2
    f = base ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    ang = angle_sign * positions.to(F64)[:, None] * f[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def attention(h, m: dict, w: dict, eps: float):
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    rot = m.get("rot") or {"dims": 0, "base": 10000.0}
    base = float(rot["base"])
    q = rms(h @ w["q"].T, eps) * w["q.norm"]
    k = rms(h @ w["k"].T, eps) * w["k.norm"]
    q = rotate_pairs(q.view(T, H, D), 1.0, base, int(rot["dims"]), pos)
    k = rotate_pairs(k.view(T, G, D), 1.0, base, int(rot["dims"]), pos)
    v = rms((h @ w["v"].T).view(T, G, V), eps)
    v = rotate_pairs(v, 1.0, base, V, pos)
    gate = torch.sigmoid(h @ w["g"].T)
    window = int((m.get("mask") or {}).get("size", T + 1))
    cap = float(m.get("softcap") or 0.0)
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i) & (i - j < window)
    o = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(m["scale"])
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~seen, float("-inf"))
        o[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    o = rotate_pairs(o, -1.0, base, V, pos)
    o = o * gate[:, :, None]
    return o.reshape(T, H * V) @ w["o"].T


def short_conv(x, taps):
    """x [T, C], taps [C, K] (the last column weighs the current token), zeros before the start."""
    T, K = x.shape[0], taps.shape[1]
    pad = torch.cat([torch.zeros(K - 1, x.shape[1], dtype=x.dtype), x])
    out = torch.zeros_like(x)
    for j in range(K):
        out = out + pad[j:j + T] * taps[:, j]
    return out


def channel_delta(h, m: dict, w: dict, eps: float):
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    silu = torch.nn.functional.silu
    q = silu(short_conv(h @ w["q"].T, w["q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ w["k"].T, w["k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ w["v"].T, w["v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)
    step = torch.nn.functional.softplus((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(w["A_log"])[None, :, None] * step)
    o = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(D, V, dtype=h.dtype)
        for t in range(T):
            S = decay[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    o = rms(o, eps) * w["norm"]
    o = o.reshape(T, H * V) * torch.sigmoid((h @ w["g1"].T) @ w["g2"].T)
    return o @ w["o"].T


def expert(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def route(z, r: dict):
    """Softmax scores over all experts; groups of neighbours ranked by their best score; the largest scores among the
    experts of the kept groups, used as weights as they are."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.softmax(z, dim=-1)
    ok = torch.ones_like(s, dtype=torch.bool)
    g = r.get("groups")
    if g:
        n, keep = int(g["count"]), int(g["keep"])
        best = s.view(-1, n, E // n).max(-1).values
        kept = torch.zeros_like(best, dtype=torch.bool)
        kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
        ok = kept[:, :, None].expand(-1, n, E // n).reshape(-1, E)
    idx = s.masked_fill(~ok, -1.0).topk(top, dim=-1).indices
    return idx, s.gather(1, idx)


def feed_forward(h, f: dict, w: dict):
    if f.get("kind", "dense") == "dense":
        return expert(h, w["up"], w["down"])
    idx, wt = route(h @ w["router"].T, f["router"])
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, c in zip(idx[t].tolist(), wt[t]):
            out[t] += c * expert(h[t:t + 1], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    return out


def token_side(x, tokens, i: int, dim: int, side_embed, w: dict, eps: float):
    e = side_embed[tokens][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ w["gate"].T) * e) @ w["proj"].T
    return rms(y, eps) * w["norm"]


def sub(w: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def layer(x, tokens, i: int, cfg: dict, w: dict):
    L, eps = cfg["layers"][i], float(cfg["norm"]["eps"])
    lw = sub(w, f"l{i}.")
    mixer = {"attention": attention, "channel_delta": channel_delta}[L["type"]]
    x = x + offset_norm(mixer(offset_norm(x, lw["norm1"], eps), L["mixer"], sub(lw, "mix."), eps), lw["norm1b"], eps)
    if L.get("mlp"):
        x = x + offset_norm(feed_forward(offset_norm(x, lw["norm2"], eps), L["mlp"], sub(lw, "mlp.")), lw["norm2b"], eps)
    if cfg.get("token_side"):
        x = x + token_side(x, tokens, i, int(cfg["token_side"]["dim"]), w["side.embed"], sub(lw, "side."), eps)
    return x


def layer_order(cfg: dict) -> list:
    """[(layer, opens a pass of the looped span)] in the order the layers run."""
    n, lp = len(cfg["layers"]), cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    a, b, t = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    order = [(i, False) for i in range(a)]
    for _ in range(t):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg: dict, weights: dict, tokens, trace: list | None = None):
    """Logits [T, vocab] of one sequence; `trace` receives the stream after every layer run."""
    w = {k: v.to(F64) if v.is_floating_point() else v for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x0 = embedding(cfg, w, tokens)
    x = x0
    for i, opens in layer_order(cfg):
        if opens:  # every pass of the looped span re-reads the embedding output next to the stream
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T
        x = layer(x, tokens, i, cfg, w)
        if trace is not None:
            trace.append(x.clone())
    x = offset_norm(x, w["final.norm"], float(cfg["norm"]["eps"]))
    return x @ w["embed"].T
