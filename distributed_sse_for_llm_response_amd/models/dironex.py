"""Dironex: a decoder-only family on several residual streams whose layer list comes from the checkpoint's
``config.json``.

The model carries ``streams`` copies of the residual (all equal to the scaled embedding at the start).  A sublayer
reads a weighted sum of them, ``u = sum_s in[s] x_s``, RMS-norms it with a gain per channel, adds a short causal
per-channel convolution over time of the normed rows (``h + conv(h)``; the last ``taps - 1`` normed rows are sequence
state), and writes back to every stream at once: ``x_t = sum_s mix[s, t] x_s + m out[t] y`` with one residual
multiplier ``m`` for the whole model.  Mixers:

* ``latent_attention`` -- queries through an RMS-normed rank-``q_rank`` latent, keys and values up-projected from a
  cached RMS-normed rank-``kv_rank`` latent plus one rotated key slice that every head shares; rotate-half rotary on
  the rotated part with YaRN frequency blending and amplitude; causal; the concatenated heads are multiplied by
  ``sigmoid(W_g h)`` before the output projection.
* ``attention`` -- grouped key/value heads, RMS norm per head on queries and keys (one gain vector for all heads), no
  rotation, sliding window.

The feed-forward is dense with the xIELU activation (``a_p z^2 + z / 2`` for ``z > 0``, ``a_n (e^z - 1 - z) + z / 2``
otherwise, ``a_p = softplus(p)``, ``a_n = 1/2 + softplus(q)``) or a routed mixture of squared-ReLU experts: sigmoid
scores, a per-expert correction that enters the choice but not the weights, groups of neighbouring experts of which
only the best ``keep`` (by the sum of their two best choice scores) are eligible, the chosen scores normalised and
scaled.  A span of layers may run several times in a row with the same weights (``loop``); every pass has its own
cache and state.  The head reads the RMS-normed sum of the streams.

This module holds the configuration (parsed from / written to the ``config.json`` dictionary), the checkpoint's tensor
naming, random initialisation for tests and benchmarks, and named configurations.  The forward pass lives in
``engine/layered_runner.py`` on the kernels of ``ops/layers.py``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch

from .muderax import NO_WINDOW, RotarySpec
from .surodra import LayerRun

MAX_STREAMS = 8     # residual copies the stream kernel holds in registers
MAX_EXPERTS = 256   # experts a routing thread ranks


@dataclass(frozen=True)
class GatedLatentSpec:
    heads: int
    dim: int         # unrotated query / key width per head
    rot_dim: int     # rotated width per head (the key's rotated part is shared by the heads)
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotarySpec
    window: int = NO_WINDOW


@dataclass(frozen=True)
class WindowAttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = NO_WINDOW


@dataclass(frozen=True)
class DenseSpec:
    ff: int


@dataclass(frozen=True)
class RoutedSpec:
    experts: int
    top: int
    ff: int
    scale: float
    groups: int = 1     # equal groups of neighbouring experts
    keep: int = 1       # groups whose experts can be chosen


@dataclass(frozen=True)
class LayerSpec:
    kind: str             # "latent_attention" | "attention"
    mixer: object
    mlp: object           # DenseSpec | RoutedSpec | None


@dataclass(frozen=True)
class DironexConfig:
    vocab_size: int
    width: int
    eps: float
    layers: tuple
    residual_mult: float = 1.0
    embed_scale: float = 1.0
    streams: int = 0               # 0 = one plain residual stream without stream weights
    canon_taps: int = 0            # 0 = no convolution on the sublayers' inputs
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0            # 0 = the checkpoint has no loop
    name: str = "dironex"
    max_position: int = 32768
    bos_token_id: int = 1
    eos_token_id: int = 2
    raw: dict = field(default=None, compare=False, hash=False, repr=False)

    family = "dironex"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def num_streams(self) -> int:
        return max(1, self.streams)

    def runs(self) -> list:
        """The layer runs in order: layers before the loop, the looped span `loop_times` times, the rest."""
        n = len(self.layers)
        if self.loop_times <= 0:
            order = list(range(n))
        else:
            order = (list(range(self.loop_start)) + list(range(self.loop_start, self.loop_stop)) * self.loop_times
                     + list(range(self.loop_stop, n)))
        return [LayerRun(layer=i, index=r, pass_no=-1) for r, i in enumerate(order)]

    # ---- config.json <-> dataclasses
    @classmethod
    def from_dict(cls, d: dict, name: str = "dironex") -> "DironexConfig":
        layers = []
        for i, L in enumerate(d["layers"]):
            m = L["mixer"]
            window = int((m.get("mask") or {}).get("size", NO_WINDOW))
            if L["type"] == "latent_attention":
                r = m["rot"]
                sc = r.get("scaling") or {}
                rot = RotarySpec(dims=int(r["dims"]), base=float(r["base"]), factor=float(sc.get("factor", 1.0)),
                                 original=float(sc.get("original", 0.0)), fast=float(sc.get("fast", 0.0)),
                                 slow=float(sc.get("slow", 0.0)))
                mixer = GatedLatentSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]),
                                        vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]),
                                        scale=float(m["scale"]), rot=rot, window=window)
            elif L["type"] == "attention":
                mixer = WindowAttentionSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                                            dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
                                            window=window)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            f = L.get("mlp")
            mlp = None
            if f:
                kind = f.get("kind", "dense")
                if kind == "dense":
                    mlp = DenseSpec(ff=int(f["ff"]))
                elif kind == "moe":
                    r = f["router"]
                    g = r.get("groups") or {}
                    mlp = RoutedSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(f["expert"]["ff"]),
                                     scale=float(r.get("scale", 1.0)), groups=int(g.get("count", 1)),
                                     keep=int(g.get("keep", g.get("count", 1))))
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
            layers.append(LayerSpec(kind=L["type"], mixer=mixer, mlp=mlp))
        loop = d.get("loop") or {}
        cfg = cls(vocab_size=int(d["vocab"]), width=int(d["width"]), eps=float(d["norm"]["eps"]), layers=tuple(layers),
                  residual_mult=float(d.get("residual_mult", 1.0)),
                  embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)), streams=int(d.get("streams", 0)),
                  canon_taps=int((d.get("canon") or {}).get("taps", 0)), loop_start=int(loop.get("start", 0)),
                  loop_stop=int(loop.get("stop", 0)), loop_times=int(loop.get("times", 0)), name=name, raw=d)
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        out = {"architecture": "Dironex", "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.eps},
               "residual_mult": self.residual_mult, "embedding": {"scale": self.embed_scale}, "layers": []}
        if self.streams > 0:
            out["streams"] = self.streams
        if self.canon_taps > 0:
            out["canon"] = {"taps": self.canon_taps}
        if self.loop_times > 0:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        for L in self.layers:
            m = L.mixer
            if L.kind == "latent_attention":
                rot = {"base": m.rot.base, "dims": m.rot.dims}
                if m.rot.scaled:
                    rot["scaling"] = {"factor": m.rot.factor, "original": m.rot.original, "fast": m.rot.fast,
                                      "slow": m.rot.slow}
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                         "q_rank": m.q_rank, "scale": m.scale, "rot": rot}
            else:
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
            if m.window != NO_WINDOW:
                mixer["mask"] = {"size": m.window}
            f = L.mlp
            if f is None:
                mlp = None
            elif isinstance(f, DenseSpec):
                mlp = {"kind": "dense", "ff": f.ff}
            else:
                mlp = {"kind": "moe", "expert": {"ff": f.ff},
                       "router": {"experts": f.experts, "top": f.top, "scale": f.scale,
                                  "groups": {"count": f.groups, "keep": f.keep}}}
            out["layers"].append({"type": L.kind, "mixer": mixer, "mlp": mlp})
        return out

    def validate(self, tp: int = 1) -> None:
        if tp != 1:
            raise ValueError("Dironex runs on one GPU per replica (no tensor-parallel sharding of its layers)")
        n = len(self.layers)
        if self.loop_times > 0 and not 0 <= self.loop_start < self.loop_stop <= n:
            raise ValueError(f"loop span {self.loop_start}..{self.loop_stop} does not fit {n} layers")
        if not 0 <= self.streams <= MAX_STREAMS:
            raise ValueError(f"streams must be 0..{MAX_STREAMS}")
        if self.canon_taps < 0:
            raise ValueError("canon.taps must not be negative")
        for i, L in enumerate(self.layers):
            m = L.mixer
            if m.window < 1:
                raise ValueError(f"layer {i}: window >= 1")
            if L.kind == "latent_attention":
                if m.rot_dim % 2 or m.rot.dims % 2 or not 0 <= m.rot.dims <= m.rot_dim or m.kv_rank > 1024:
                    raise ValueError(f"layer {i}: rot_dim and rot.dims must be even, rot.dims <= rot_dim, "
                                     f"kv_rank <= 1024")
            else:
                if m.heads % m.kv_heads or max(m.dim, m.vdim) > 512:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads, head widths <= 512")
            f = L.mlp
            if isinstance(f, RoutedSpec):
                if (f.experts > MAX_EXPERTS or not 1 <= f.top <= f.experts or f.groups < 1 or f.experts % f.groups
                        or not 1 <= f.keep <= f.groups or f.top > f.keep * (f.experts // f.groups)):
                    raise ValueError(f"layer {i}: router sizes do not fit (experts <= {MAX_EXPERTS}, equal groups, "
                                     f"top <= experts of the kept groups)")

    def num_params(self) -> int:
        return sum(math.prod(s) for s in tensor_shapes(self).values())

    def cache_bytes_per_token(self, elem_bytes: int = 2) -> int:
        """Paged cache bytes per token over all layer runs: a latent row per latent-attention run, keys and values per
        windowed-attention run."""
        n = 0
        for r in self.runs():
            m = self.layers[r.layer].mixer
            if self.layers[r.layer].kind == "latent_attention":
                n += (m.kv_rank + m.rot_dim) * elem_bytes
            else:
                n += m.kv_heads * (m.dim + m.vdim) * elem_bytes
        return n

    def state_bytes_per_sequence(self) -> int:
        """fp32 convolution tails of one sequence: both sublayers of every run."""
        k = max(0, self.canon_taps - 1)
        return 4 * k * self.width * sum(1 + (self.layers[r.layer].mlp is not None) for r in self.runs())


def layer_tensor_shapes(cfg: DironexConfig, i: int) -> dict:
    """{tensor name: shape} of layer i (checkpoint naming, linear weights [out, in])."""
    L, W, p = cfg.layers[i], cfg.width, f"l{i}."
    m = L.mixer
    s = {p + "norm1": (W,)}
    if L.kind == "latent_attention":
        s.update({p + "mix.dq": (m.q_rank, W), p + "mix.dq.norm": (m.q_rank,),
                  p + "mix.uq": (m.heads * (m.dim + m.rot_dim), m.q_rank), p + "mix.dkv": (m.kv_rank + m.rot_dim, W),
                  p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                  p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.g": (m.heads * m.vdim, W),
                  p + "mix.o": (W, m.heads * m.vdim)})
    else:
        s.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.kv_heads * m.dim, W),
                  p + "mix.v": (m.kv_heads * m.vdim, W), p + "mix.q.norm": (m.dim,), p + "mix.k.norm": (m.dim,),
                  p + "mix.o": (W, m.heads * m.vdim)})
    subs = ["1"]
    f = L.mlp
    if f is not None:
        subs.append("2")
        s[p + "norm2"] = (W,)
        if isinstance(f, DenseSpec):
            s.update({p + "mlp.up": (f.ff, W), p + "mlp.down": (W, f.ff), p + "mlp.act": (2,)})
        else:
            for e in range(f.experts):
                s.update({f"{p}mlp.e{e}.up": (f.ff, W), f"{p}mlp.e{e}.down": (W, f.ff)})
            s.update({p + "mlp.router": (f.experts, W), p + "mlp.correction": (f.experts,)})
    for q in subs:
        if cfg.streams > 0:
            S = cfg.streams
            s.update({f"{p}hc{q}.in": (S,), f"{p}hc{q}.out": (S,), f"{p}hc{q}.mix": (S, S)})
        if cfg.canon_taps > 0:
            s[f"{p}canon{q}"] = (W, cfg.canon_taps)
    return s


def tensor_shapes(cfg: DironexConfig) -> dict:
    s = {"embed": (cfg.vocab_size, cfg.width)}
    for i in range(len(cfg.layers)):
        s.update(layer_tensor_shapes(cfg, i))
    s["final.norm"] = (cfg.width,)
    s["head"] = (cfg.vocab_size, cfg.width)
    return s


@torch.no_grad()
def init_weights(cfg: DironexConfig, seed: int = 0, device="cpu", dtype=torch.bfloat16) -> dict:
    """Random weights in the checkpoint's naming: projections ~ N(0, 1 / fan-in), norm gains near 1, stream weights
    near a plain residual, corrections large enough to change the choice of experts."""
    dev = torch.device(device)
    gdev = dev if dev.type == "cuda" else torch.device("cpu")
    g = torch.Generator(device=gdev).manual_seed(seed)
    out = {}

    def randn(shape):
        return torch.randn(tuple(shape), generator=g, device=gdev)

    S = cfg.num_streams
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = randn(shape)
        elif leaf in ("norm1", "norm2", "norm") or name == "final.norm":
            t = 1.0 + 0.2 * randn(shape)
        elif leaf == "in":
            t = 1.0 / S + 0.2 * randn(shape)
        elif leaf == "out":
            t = 1.0 + 0.3 * randn(shape)
        elif leaf == "mix":
            t = torch.eye(S, device=gdev) + 0.15 * randn(shape)
        elif leaf.startswith("canon"):
            t = 0.3 * randn(shape)
        elif leaf == "act":
            t = 0.5 * randn(shape)
        elif leaf == "correction":
            t = 0.3 * randn(shape)
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(dtype).to(dev)
    return out


def _named(name: str, vocab: int, width: int, n_layers: int, heads: int, dim: int, rot_dim: int, kv_rank: int,
           q_rank: int, kv_heads: int, window: int, ff: int, experts: int, top: int, expert_ff: int, groups: int,
           keep: int, loop: tuple = (0, 0, 0), streams: int = 4, max_position: int = 32768) -> DironexConfig:
    rot = RotarySpec(dims=rot_dim, base=500000.0, factor=4.0, original=4096.0, fast=32.0, slow=1.0)
    lat = GatedLatentSpec(heads=heads, dim=dim, rot_dim=rot_dim, vdim=dim, kv_rank=kv_rank, q_rank=q_rank,
                          scale=1.0 / math.sqrt(dim + rot_dim), rot=rot)
    att = WindowAttentionSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=1.0 / math.sqrt(dim),
                              window=window)
    moe = RoutedSpec(experts=experts, top=top, ff=expert_ff, scale=2.0, groups=groups, keep=keep)
    pattern = (("latent_attention", lat, DenseSpec(ff=ff)), ("attention", att, moe), ("latent_attention", lat, moe))
    layers = tuple(LayerSpec(kind=k, mixer=m, mlp=f) for k, m, f in (pattern[i % 3] for i in range(n_layers)))
    cfg = DironexConfig(vocab_size=vocab, width=width, eps=1e-6, layers=layers, residual_mult=0.5, embed_scale=2.0,
                        streams=streams, canon_taps=4, loop_start=loop[0], loop_stop=loop[1], loop_times=loop[2],
                        name=name, max_position=max_position)
    cfg.validate()
    return cfg


# Named configurations (random weights): a toy for smoke runs, and sizes that resemble real models' layers for the
# benchmark -- "mid" has 2048-wide layers, "wide" the 4096-wide layers of a 7B-class model.
TINY = _named("dironex-tiny", vocab=512, width=128, n_layers=3, heads=4, dim=32, rot_dim=16, kv_rank=48, q_rank=40,
              kv_heads=2, window=40, ff=256, experts=8, top=2, expert_ff=64, groups=4, keep=2, loop=(0, 2, 2),
              streams=2, max_position=4096)
MID = _named("dironex-mid", vocab=32768, width=2048, n_layers=6, heads=16, dim=128, rot_dim=64, kv_rank=512,
             q_rank=1024, kv_heads=8, window=1024, ff=8192, experts=16, top=2, expert_ff=2048, groups=4, keep=2)
WIDE = _named("dironex-wide", vocab=32768, width=4096, n_layers=6, heads=32, dim=128, rot_dim=64, kv_rank=512,
              q_rank=1536, kv_heads=8, window=1024, ff=14336, experts=16, top=2, expert_ff=4096, groups=4, keep=2)

CONFIGS = {c.name: c for c in (TINY, MID, WIDE)}
