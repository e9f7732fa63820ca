"""Murulorn: a decoder-only family with bracketing norms, hashed bigram embeddings and per-layer token inputs, whose
layer list comes from the checkpoint's ``config.json``.

The embedding output is ``x0 = embed[token] + bigram[hash(previous token, token)]`` with
``hash = (prev * mul_prev + token * mul_cur) mod buckets``; a sequence's first token takes the table's last row (row
``buckets``), so the previous token is part of a sequence's state.  Every layer is

    x += n(mixer(n(x, 1 + a1)), 1 + b1);  x += n(ff(n(x, 1 + a2)), 1 + b2);  x += n(side(x, token), s)

on an fp32 residual stream, ``n(v, g) = v / sqrt(mean(v^2) + eps) * g``: an RMS norm before AND after each sublayer,
gains stored around zero.  ``side`` is the per-layer token input: layer i owns columns ``[i dim, (i + 1) dim)`` of a
second embedding table ``e``, ``side = proj(gelu_tanh(gate x) * e[token])``, normed with a plain gain.  Mixers:

* ``attention`` -- softmax attention with grouped key/value heads; an RMS norm over the WHOLE query and key projection
  (plain gains); rotary on the leading ``rot.dims`` coordinates of each head, neighbouring coordinates (2i, 2i + 1)
  forming a pair; values RMS-normed per head (no gain) and ROTATED by their own position over all ``vdim`` coordinates
  before they are cached, the head's weighted sum turned back by the query's position (so a value enters the output
  rotated by the distance); scores ``softcap * tanh(scale q.k / softcap)``; sliding window; a sigmoid gate per head.
* ``channel_delta`` -- gated delta rule with one decay per head AND key channel: ``S = diag(g) S``,
  ``u = beta (v - S^T k)``, ``S += k u^T``, ``o = S^T q`` with ``g = exp(-exp(A_h) softplus(a2 (a1 h) + dt))``
  laid out heads x dim; q / k / v pass a short causal convolution and SiLU, q and k are unit vectors per head (q / k
  heads may be shared by several value heads); the output is RMS-normed per head and gated by
  ``sigmoid(g2 (g1 h))``.

Feed-forward: dense ``down(relu(up h)^2)``, or routed experts of that form: scores = softmax over ALL experts, experts
in ``groups.count`` groups of neighbours of which the ``groups.keep`` groups with the largest best score are
eligible, the ``top`` largest scores chosen and used as weights as they are.  A span of layers may run several times in
a row with the same weights (``loop``); every pass has its own pages and state and opens with
``x <- W_in [x; x0]``.  The head is the embedding table itself behind the final norm.

This module holds the configuration (parsed from / written to the ``config.json`` dictionary), the checkpoint's tensor
naming, random initialisation for tests and benchmarks, and named configurations.  The forward pass lives in
``engine/layered_runner.py`` on the kernels of ``ops/layers.py``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch

from .surodra import ANY, NO_WINDOW, UNIT_EPS, HalfRotarySpec, LayerRun  # noqa: F401  (UNIT_EPS: the runner's import)


@dataclass(frozen=True)
class RotatedValueAttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int             # leading coordinates of a query / key head that rotate (0 = none)
    rot_base: float           # also the base of the values' rotation over all vdim coordinates
    softcap: float = 0.0      # 0 = scores are not capped
    window: int = NO_WINDOW


@dataclass(frozen=True)
class ChannelDeltaSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int = ANY     # inner widths of the two low-rank projections; a checkpoint's tensors decide them
    gate_rank: int = ANY


@dataclass(frozen=True)
class SquaredReluSpec:
    ff: int


@dataclass(frozen=True)
class SoftmaxRoutedSpec:
    experts: int
    top: int
    ff: int
    groups: int = 1
    keep: int = 1


@dataclass(frozen=True)
class BigramSpec:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class LayerSpec:
    kind: str             # "attention" | "channel_delta"
    mixer: object
    mlp: object           # SquaredReluSpec | SoftmaxRoutedSpec | None


@dataclass(frozen=True)
class MurulornConfig:
    vocab_size: int
    width: int
    eps: float
    layers: tuple
    bigram: BigramSpec | None = None
    side_dim: int = 0              # columns of the side table per layer (0 = no per-layer token input)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0            # 0 = the checkpoint has no loop (and no loop.in)
    name: str = "murulorn"
    max_position: int = 32768
    bos_token_id: int = 1
    eos_token_id: int = 2
    raw: dict = field(default=None, compare=False, hash=False, repr=False)

    family = "murulorn"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """The layer runs in order: layers before the loop, the looped span `loop_times` times, the rest.  pass_no >= 0
        marks the run that opens a pass of the looped span."""
        n = len(self.layers)
        if self.loop_times <= 0:
            order = [(i, -1) for i in range(n)]
        else:
            order = [(i, -1) for i in range(self.loop_start)]
            for t in range(self.loop_times):
                order += [(i, t if i == self.loop_start else -1) for i in range(self.loop_start, self.loop_stop)]
            order += [(i, -1) for i in range(self.loop_stop, n)]
        return [LayerRun(layer=i, index=r, pass_no=t) for r, (i, t) in enumerate(order)]

    # ---- config.json <-> dataclasses
    @classmethod
    def from_dict(cls, d: dict, name: str = "murulorn") -> "MurulornConfig":
        layers = []
        for i, L in enumerate(d["layers"]):
            m = L["mixer"]
            if L["type"] == "attention":
                rot, mask = m.get("rot") or {}, m.get("mask") or {}
                mixer = RotatedValueAttentionSpec(
                    heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                    vdim=int(m["vdim"]), scale=float(m["scale"]), rot_dims=int(rot.get("dims", 0)),
                    rot_base=float(rot.get("base", 10000.0)), softcap=float(m.get("softcap") or 0.0),
                    window=int(mask.get("size", NO_WINDOW)))
            elif L["type"] == "channel_delta":
                mixer = ChannelDeltaSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                                         dim=int(m["dim"]), vdim=int(m["vdim"]), conv=int(m["conv"]))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            f = L.get("mlp")
            mlp = None
            if f:
                kind = f.get("kind", "dense")
                if kind == "dense":
                    mlp = SquaredReluSpec(ff=int(f["ff"]))
                elif kind == "moe":
                    r = f["router"]
                    g = r.get("groups") or {}
                    mlp = SoftmaxRoutedSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(f["expert"]["ff"]),
                                            groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))))
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
            layers.append(LayerSpec(kind=L["type"], mixer=mixer, mlp=mlp))
        b = (d.get("embedding") or {}).get("bigram")
        loop = d.get("loop") or {}
        cfg = cls(vocab_size=int(d["vocab"]), width=int(d["width"]), eps=float(d["norm"]["eps"]), layers=tuple(layers),
                  bigram=BigramSpec(buckets=int(b["buckets"]), mul_prev=int(b["mul_prev"]), mul_cur=int(b["mul_cur"]))
                  if b else None,
                  side_dim=int((d.get("token_side") or {}).get("dim", 0)), loop_start=int(loop.get("start", 0)),
                  loop_stop=int(loop.get("stop", 0)), loop_times=int(loop.get("times", 0)), name=name, raw=d)
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        out = {"architecture": "Murulorn", "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.eps},
               "layers": []}
        if self.bigram:
            out["embedding"] = {"bigram": {"buckets": self.bigram.buckets, "mul_prev": self.bigram.mul_prev,
                                           "mul_cur": self.bigram.mul_cur}}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        if self.loop_times > 0:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        for L in self.layers:
            m = L.mixer
            if L.kind == "attention":
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                         "rot": {"base": m.rot_base, "dims": m.rot_dims}}
                if m.softcap:
                    mixer["softcap"] = m.softcap
                if m.window != NO_WINDOW:
                    mixer["mask"] = {"size": m.window}
            else:
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
            f = L.mlp
            if f is None:
                mlp = None
            elif isinstance(f, SquaredReluSpec):
                mlp = {"kind": "dense", "ff": f.ff}
            else:
                router = {"experts": f.experts, "top": f.top}
                if f.groups > 1:
                    router["groups"] = {"count": f.groups, "keep": f.keep}
                mlp = {"kind": "moe", "expert": {"ff": f.ff}, "router": router}
            out["layers"].append({"type": L.kind, "mixer": mixer, "mlp": mlp})
        return out

    def validate(self, tp: int = 1) -> None:
        if tp != 1:
            raise ValueError("Murulorn runs on one GPU per replica (no tensor-parallel sharding of its layers)")
        n = len(self.layers)
        if self.loop_times > 0 and not 0 <= self.loop_start < self.loop_stop <= n:
            raise ValueError(f"loop span {self.loop_start}..{self.loop_stop} does not fit {n} layers")
        if self.bigram and self.bigram.buckets < 1:
            raise ValueError("bigram.buckets must be positive")
        for i, L in enumerate(self.layers):
            m = L.mixer
            if m.heads % m.kv_heads or max(m.dim, m.vdim) > 512:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads, head widths at most 512")
            if L.kind == "attention":
                if m.rot_dims % 2 or not 0 <= m.rot_dims <= m.dim or m.vdim % 2 or m.window < 1:
                    raise ValueError(f"layer {i}: rot.dims even and at most dim, vdim even, window >= 1")
            elif m.conv < 1:
                raise ValueError(f"layer {i}: conv >= 1")
            f = L.mlp
            if isinstance(f, SoftmaxRoutedSpec):
                if f.experts > 256 or f.experts % f.groups or not 1 <= f.keep <= f.groups or \
                        not 1 <= f.top <= f.keep * (f.experts // f.groups):
                    raise ValueError(f"layer {i}: at most 256 experts in equal groups, 1 <= keep <= groups, top within "
                                     "the kept groups")

    def num_params(self) -> int:
        return sum(math.prod(max(x, 1) for x in s) for s in tensor_shapes(self).values())

    def cache_bytes_per_token(self, elem_bytes: int = 2) -> int:
        """Paged cache bytes per token: keys and values of the attention layers, once per run of their layer."""
        n = 0
        for r in self.runs():
            L = self.layers[r.layer]
            if L.kind == "attention":
                n += L.mixer.kv_heads * (L.mixer.dim + L.mixer.vdim) * elem_bytes
        return n

    def state_bytes_per_sequence(self) -> int:
        """fp32 matrix states and convolution tails of one sequence over all runs (plus its previous token)."""
        n = 1
        for r in self.runs():
            L, m = self.layers[r.layer], self.layers[r.layer].mixer
            if L.kind == "channel_delta":
                n += m.heads * m.dim * m.vdim + (m.conv - 1) * (2 * m.kv_heads * m.dim + m.heads * m.vdim)
        return 4 * n


def layer_tensor_shapes(cfg: MurulornConfig, i: int) -> dict:
    """{tensor name: shape} of layer i (checkpoint naming, linear weights [out, in]); ANY = the checkpoint decides."""
    L, W, p = cfg.layers[i], cfg.width, f"l{i}."
    m = L.mixer
    s = {p + "norm1": (W,), p + "norm1b": (W,)}
    if L.kind == "attention":
        s.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.kv_heads * m.dim, W),
                  p + "mix.v": (m.kv_heads * m.vdim, W), p + "mix.q.norm": (m.heads * m.dim,),
                  p + "mix.k.norm": (m.kv_heads * m.dim,), p + "mix.g": (m.heads, W), p + "mix.o": (W, m.heads * m.vdim)})
    else:
        qk, hv, hd = m.kv_heads * m.dim, m.heads * m.vdim, m.heads * m.dim
        s.update({p + "mix.q": (qk, W), p + "mix.q.conv": (qk, m.conv), p + "mix.k": (qk, W),
                  p + "mix.k.conv": (qk, m.conv), p + "mix.v": (hv, W), p + "mix.v.conv": (hv, m.conv),
                  p + "mix.b": (m.heads, W), p + "mix.A_log": (m.heads,), p + "mix.norm": (m.vdim,),
                  p + "mix.a1": (m.decay_rank, W), p + "mix.a2": (hd, m.decay_rank), p + "mix.dt_bias": (hd,),
                  p + "mix.g1": (m.gate_rank, W), p + "mix.g2": (hv, m.gate_rank), p + "mix.o": (W, hv)})
    f = L.mlp
    if f is not None:
        s.update({p + "norm2": (W,), p + "norm2b": (W,)})
        if isinstance(f, SquaredReluSpec):
            s.update({p + "mlp.up": (f.ff, W), p + "mlp.down": (W, f.ff)})
        else:
            s[p + "mlp.router"] = (f.experts, W)
            for e in range(f.experts):
                s.update({p + f"mlp.e{e}.up": (f.ff, W), p + f"mlp.e{e}.down": (W, f.ff)})
    if cfg.side_dim:
        s.update({p + "side.gate": (cfg.side_dim, W), p + "side.proj": (W, cfg.side_dim), p + "side.norm": (W,)})
    return s


def tensor_shapes(cfg: MurulornConfig) -> dict:
    s = {"embed": (cfg.vocab_size, cfg.width)}
    if cfg.bigram:
        s["bigram"] = (cfg.bigram.buckets + 1, cfg.width)
    if cfg.loop_times > 0:
        s["loop.in"] = (cfg.width, 2 * cfg.width)
    if cfg.side_dim:
        s["side.embed"] = (cfg.vocab_size, cfg.side_dim * len(cfg.layers))
    for i in range(len(cfg.layers)):
        s.update(layer_tensor_shapes(cfg, i))
    s["final.norm"] = (cfg.width,)
    return s


@torch.no_grad()
def init_weights(cfg: MurulornConfig, seed: int = 0, device="cpu", dtype=torch.bfloat16, rank=16) -> dict:
    """Random weights in the checkpoint's naming: projections ~ N(0, 1 / fan-in), stored gains near 0 (bracketing norms)
    or near 1 (plain norms), decay parameters spread so that fast and slow heads and channels occur.  `rank` (one number,
    or one for the decay's and one for the gate's pair) fills the inner widths that the configuration leaves to the
    checkpoint."""
    ranks = (rank, rank) if isinstance(rank, int) else tuple(rank)
    dev = torch.device(device)
    gdev = dev if dev.type == "cuda" else torch.device("cpu")
    g = torch.Generator(device=gdev).manual_seed(seed)
    out = {}

    def randn(shape):
        return torch.randn(tuple(shape), generator=g, device=gdev)

    def rand(shape):
        return torch.rand(tuple(shape), generator=g, device=gdev)

    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        shape = tuple(ranks[leaf in ("g1", "g2")] if x == ANY else x for x in shape)
        if name in ("embed", "bigram", "side.embed"):
            t = randn(shape) * (1.0 if name == "embed" else 0.5)
        elif leaf in ("norm1", "norm2", "norm1b", "norm2b") or name == "final.norm":
            t = 0.2 * randn(shape)
        elif name.endswith(("q.norm", "k.norm", "mix.norm", "side.norm")):
            t = 1.0 + 0.2 * randn(shape)
        elif leaf == "conv":
            t = randn(shape) / math.sqrt(shape[-1]) + 0.3
        elif leaf == "A_log":
            t = torch.log(0.05 + 2.0 * rand(shape))
        elif leaf == "dt_bias":
            t = randn(shape) - 1.0
        elif name == "loop.in":
            t = randn(shape) / math.sqrt(shape[-1] / 2)
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(dtype).to(dev)
    return out


def _named(name: str, vocab: int, width: int, pattern: tuple, heads: int, kv_heads: int, dim: int, vdim: int, ff: int,
           experts: int, expert_ff: int, top: int, groups: int, keep: int, side_dim: int, buckets: int,
           loop: tuple = (0, 0, 0), window: int = 1024, rank: int = 64, max_position: int = 32768) -> MurulornConfig:
    mix = {"attention": RotatedValueAttentionSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                                                  scale=1.0 / math.sqrt(dim), rot_dims=dim // 2, rot_base=10000.0,
                                                  softcap=30.0, window=window),
           "channel_delta": ChannelDeltaSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=4, decay_rank=rank,
                                             gate_rank=rank)}
    layers = tuple(LayerSpec(kind=k, mixer=mix[k],
                             mlp=SquaredReluSpec(ff=ff) if i == 0 else
                             SoftmaxRoutedSpec(experts=experts, top=top, ff=expert_ff, groups=groups, keep=keep))
                   for i, k in enumerate(pattern))
    cfg = MurulornConfig(vocab_size=vocab, width=width, eps=1e-6, layers=layers,
                         bigram=BigramSpec(buckets=buckets, mul_prev=36313, mul_cur=27191), side_dim=side_dim,
                         loop_start=loop[0], loop_stop=loop[1], loop_times=loop[2], name=name, max_position=max_position)
    cfg.validate()
    return cfg


# Named configurations (random weights): a toy for smoke runs, and sizes that resemble real models' layers for the
# benchmark -- "mid" has 2048-wide layers, "wide" the 4096-wide layers of a 7B-class model; six layer runs each (a
# looped pair of channel_delta layers counts twice), like the other families' -mid / -wide models.
PATTERN = ("attention", "channel_delta", "channel_delta", "attention", "channel_delta")
TINY = _named("murulorn-tiny", vocab=512, width=128, pattern=("attention", "channel_delta", "attention"), heads=4,
              kv_heads=2, dim=32, vdim=32, ff=256, experts=8, expert_ff=64, top=2, groups=4, keep=2, side_dim=16,
              buckets=251, loop=(1, 2, 2), window=48, rank=16, max_position=4096)
MID = _named("murulorn-mid", vocab=32768, width=2048, pattern=PATTERN, heads=16, kv_heads=8, dim=128, vdim=128, ff=8192,
             experts=16, expert_ff=2048, top=2, groups=4, keep=2, side_dim=64, buckets=65521, loop=(1, 2, 2))
WIDE = _named("murulorn-wide", vocab=32768, width=4096, pattern=PATTERN, heads=32, kv_heads=8, dim=128, vdim=128,
              ff=14336, experts=16, expert_ff=4096, top=2, groups=4, keep=2, side_dim=64, buckets=65521, loop=(1, 2, 2))

CONFIGS = {c.name: c for c in (TINY, MID, WIDE)}
