"""Engine weight layout and tensor-parallel sharding.

The decode kernels want, per rank (t = TP degree, r = rank):

* ``wqkv``  [(Hq/t + 2·Hkv/t)·128, H]  — q heads, then k heads, then v heads of this rank, each
  128-row head unit permuted by :func:`ops.reference.rotary_perm` so the fused RoPE epilogue finds
  the rotary partner 8 lanes away (column-parallel: Megatron split by heads).
* ``wo``    [H, Hq/t·128]              — row-parallel (input features split by heads).
* ``wgu``   [2·F/t, H]                 — gate/up rows interleaved in 8-row blocks (column-parallel),
  so the SiLU·mul epilogue pairs gate and up in one MFMA tile.
* ``wd``    [H, F/t]                   — row-parallel.
* ``lm_head`` [V/t, H]                 — vocab-parallel; the sampler merges per-rank candidates.
* ``embed`` [V, H] replicated (256 MiB; HBM is plentiful, and it avoids an all-reduce per step).

Every GEMM of the engine -- decode (gemm_skinny / gemm_stream / gemm_wide) and prefill (gemm_tiled) --
consumes the tiled layout of :func:`ops.reference.tile_weight` (``*_t`` fields, made by :func:`attach_tiled`):
every weight load instruction reads 1 KiB of contiguous HBM, and a (16-column, 32-deep) block is one MFMA B
fragment.  The row-major [out, in] matrices above are only the conversion input; :func:`attach_tiled` drops
them, so the model is resident once (round 1 kept both layouts for the library prefill GEMMs: 14.5 GB more for
Mistral-7B at TP=1, now KV cache).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from ..models.mistral import MistralConfig
from ..ops.reference import gate_up_perm, rotary_perm, tile_weight


@dataclass
class LayerWeights:
    attn_norm: torch.Tensor
    wqkv: torch.Tensor   # row-major conversion inputs (None once attach_tiled has run)
    wo: torch.Tensor
    ffn_norm: torch.Tensor
    wgu: torch.Tensor
    wd: torch.Tensor
    # the engine's copies, in the tiled layout (attach_tiled)
    wqkv_t: torch.Tensor = None
    wo_t: torch.Tensor = None
    wgu_t: torch.Tensor = None
    wd_t: torch.Tensor = None


@dataclass
class EngineWeights:
    cfg: MistralConfig
    tp_rank: int
    tp_size: int
    embed: torch.Tensor
    layers: list
    final_norm: torch.Tensor
    lm_head: torch.Tensor
    lm_head_t: torch.Tensor = None

    @property
    def nh(self) -> int:
        return self.cfg.num_heads // self.tp_size

    @property
    def nkv(self) -> int:
        return self.cfg.num_kv_heads // self.tp_size

    @property
    def ffn(self) -> int:
        return self.cfg.intermediate_size // self.tp_size

    @property
    def vocab_local(self) -> int:
        return self.cfg.vocab_size // self.tp_size

    @property
    def vocab_offset(self) -> int:
        return self.tp_rank * self.vocab_local

    def nbytes(self) -> int:
        """Bytes of the resident model (what a decode step streams, plus the embedding table)."""
        n = self.embed.numel() + self.final_norm.numel() + self.lm_head_t.numel()
        for L in self.layers:
            n += sum(t.numel() for t in (L.attn_norm, L.wqkv_t, L.wo_t, L.ffn_norm, L.wgu_t, L.wd_t))
        return 2 * n


@torch.no_grad()
def attach_tiled(w: EngineWeights) -> EngineWeights:
    """Convert every GEMM weight to the tiled layout and drop the row-major input (idempotent)."""
    for L in w.layers:
        if L.wqkv_t is None:
            L.wqkv_t, L.wo_t = tile_weight(L.wqkv), tile_weight(L.wo)
            L.wgu_t, L.wd_t = tile_weight(L.wgu), tile_weight(L.wd)
        L.wqkv = L.wo = L.wgu = L.wd = None
    if w.lm_head_t is None:
        w.lm_head_t = tile_weight(w.lm_head)
    w.lm_head = None
    return w


def _permute_units(w: torch.Tensor) -> torch.Tensor:
    """Permute the rows of each 128-row head unit by rotary_perm (works for q, k and v units)."""
    units = w.shape[0] // 128
    perm = rotary_perm().to(w.device)
    return w.view(units, 128, -1)[:, perm, :].reshape(w.shape)


def convert_standard(cfg: MistralConfig, std, tp_rank: int = 0, tp_size: int = 1, device="cpu") -> EngineWeights:
    """Standard (HF-layout) weights -> this rank's engine weights."""
    cfg.validate(tp_size)
    D = cfg.head_dim
    nh, nkv, F = cfg.num_heads // tp_size, cfg.num_kv_heads // tp_size, cfg.intermediate_size // tp_size
    V = cfg.vocab_size // tp_size
    r = tp_rank
    layers = []
    for L in std["layers"]:
        q = L["q"][r * nh * D:(r + 1) * nh * D]
        k = L["k"][r * nkv * D:(r + 1) * nkv * D]
        v = L["v"][r * nkv * D:(r + 1) * nkv * D]
        wqkv = _permute_units(torch.cat([q, k, v]))
        wo = L["o"][:, r * nh * D:(r + 1) * nh * D]
        gate = L["gate"][r * F:(r + 1) * F]
        up = L["up"][r * F:(r + 1) * F]
        wgu = torch.cat([gate, up])[gate_up_perm(F)]
        wd = L["down"][:, r * F:(r + 1) * F]
        layers.append(LayerWeights(
            attn_norm=L["attn_norm"].contiguous().to(device), wqkv=wqkv.contiguous().to(device),
            wo=wo.contiguous().to(device), ffn_norm=L["ffn_norm"].contiguous().to(device),
            wgu=wgu.contiguous().to(device), wd=wd.contiguous().to(device)))
    return attach_tiled(EngineWeights(
        cfg=cfg, tp_rank=tp_rank, tp_size=tp_size, embed=std["embed"].contiguous().to(device), layers=layers,
        final_norm=std["final_norm"].contiguous().to(device), lm_head=std["lm_head"][r * V:(r + 1) * V].contiguous().to(device)))


@torch.no_grad()
def random_engine_weights(cfg: MistralConfig, tp_rank: int = 0, tp_size: int = 1, device="cuda",
                          seed: int = 0, dtype=torch.bfloat16) -> EngineWeights:
    """Random weights generated directly on the device in engine layout (the 7B bench path).

    Generating 14.5 GB through the standard layout on the host would take minutes; the engine layout
    is a fixed row permutation of the standard one, so the distribution is identical.  Each rank
    draws its own shard (seeded by (seed, rank)), i.e. the global model is a valid random model.
    """
    cfg.validate(tp_size)
    D, H = cfg.head_dim, cfg.hidden_size
    nh, nkv, F = cfg.num_heads // tp_size, cfg.num_kv_heads // tp_size, cfg.intermediate_size // tp_size
    V = cfg.vocab_size // tp_size
    gen = torch.Generator(device=device)
    gen.manual_seed(seed * 1000003 + tp_rank)

    def lin(out_f, in_f):
        t = torch.empty(out_f, in_f, device=device, dtype=dtype)
        t.normal_(0.0, 1.0 / math.sqrt(in_f), generator=gen)
        return t

    def norm(n):
        t = torch.empty(n, device=device, dtype=torch.float32).normal_(1.0, 0.1, generator=gen)
        return t.to(dtype)

    embed_gen = torch.Generator(device=device)
    embed_gen.manual_seed(seed * 1000003 + 999)  # replicated: identical on every rank
    embed = torch.empty(cfg.vocab_size, H, device=device, dtype=dtype).normal_(0.0, 1.0, generator=embed_gen)
    layers = []
    for _ in range(cfg.num_layers):
        L = LayerWeights(attn_norm=norm(H), wqkv=lin((nh + 2 * nkv) * D, H), wo=lin(H, nh * D),
                         ffn_norm=norm(H), wgu=lin(2 * F, H), wd=lin(H, F))
        L.wqkv_t, L.wo_t, L.wgu_t, L.wd_t = (tile_weight(t) for t in (L.wqkv, L.wo, L.wgu, L.wd))
        L.wqkv = L.wo = L.wgu = L.wd = None  # one layer's row-major copy at a time
        layers.append(L)
    return attach_tiled(EngineWeights(cfg=cfg, tp_rank=tp_rank, tp_size=tp_size, embed=embed, layers=layers,
                                      final_norm=norm(H), lm_head=lin(V, H)))


def load_safetensors(cfg: MistralConfig, path: str, tp_rank: int = 0, tp_size: int = 1, device="cpu") -> EngineWeights:
    """Load an HF Mistral checkpoint directory (``*.safetensors``) into the engine layout."""
    from pathlib import Path

    from safetensors.torch import load_file

    tensors = {}
    for f in sorted(Path(path).glob("*.safetensors")):
        tensors.update(load_file(str(f)))
    std = {"embed": tensors["model.embed_tokens.weight"], "final_norm": tensors["model.norm.weight"],
           "lm_head": tensors.get("lm_head.weight", tensors["model.embed_tokens.weight"]), "layers": []}
    for i in range(cfg.num_layers):
        p = f"model.layers.{i}."
        std["layers"].append({
            "attn_norm": tensors[p + "input_layernorm.weight"],
            "q": tensors[p + "self_attn.q_proj.weight"], "k": tensors[p + "self_attn.k_proj.weight"],
            "v": tensors[p + "self_attn.v_proj.weight"], "o": tensors[p + "self_attn.o_proj.weight"],
            "ffn_norm": tensors[p + "post_attention_layernorm.weight"],
            "gate": tensors[p + "mlp.gate_proj.weight"], "up": tensors[p + "mlp.up_proj.weight"],
            "down": tensors[p + "mlp.down_proj.weight"],
        })
    return convert_standard(cfg, std, tp_rank, tp_size, device)


# ---------------------------------------------------------------------------------------------------------------------
# Configuration-driven designs (models/muderax.py): row-major weights for the general GEMM (ops.gemm_rm), regrouped so
# that every per-head / per-block / per-expert family is ONE tensor with a batch axis.
@dataclass
class LatentAttentionWeights:
    q: torch.Tensor          # [H (dn + dr), W]
    dkv: torch.Tensor        # [rk + dr, W]
    dkv_norm: torch.Tensor   # [rk]
    uk_t: torch.Tensor       # [H, rk, dn]: the key up-projection transposed per head (folds into the query)
    uv: torch.Tensor         # [H, dv, rk]
    o: torch.Tensor          # [W, H dv]
    q_t: torch.Tensor = None  # q / o in the tiled layout (tile_weight) when their shapes fit the engine's tiled-layout
    o_t: torch.Tensor = None  # GEMMs; the row-major tensor is then dropped (None)


@dataclass
class RglruWeights:
    y: torch.Tensor          # [C, W]
    y_b: torch.Tensor
    x: torch.Tensor          # [C, W]
    x_b: torch.Tensor
    conv: torch.Tensor       # [C, taps]
    conv_b: torch.Tensor
    gates: torch.Tensor      # [blocks, 2 bw, bw]: rows [recurrence gate | input gate] of each block
    gates_b: torch.Tensor    # [blocks, 2 bw]
    lam: torch.Tensor        # [C]
    o: torch.Tensor          # [W, C]
    y_t: torch.Tensor = None  # y / x / o in the tiled layout when their shapes fit (row-major then None)
    x_t: torch.Tensor = None
    o_t: torch.Tensor = None


@dataclass
class MoeWeights:
    router: torch.Tensor     # [E, W]
    router_b: torch.Tensor   # [E]
    gate: torch.Tensor       # [E, F, W]
    up: torch.Tensor         # [E, F, W]
    down: torch.Tensor       # [E, W, F]
    sgate: torch.Tensor = None   # shared expert [Fs, W] (None: the design has none)
    sup: torch.Tensor = None
    sdown: torch.Tensor = None   # [W, Fs]


@dataclass
class LayeredLayer:
    norm1: torch.Tensor      # one number
    mix: object
    norm2: torch.Tensor = None
    mlp: MoeWeights = None


@dataclass
class LayeredWeights:
    cfg: object
    embed: torch.Tensor
    layers: list             # one entry per layer; layers that borrow weights hold the lender's object
    final_norm: torch.Tensor
    head: torch.Tensor
    dtype: torch.dtype = torch.bfloat16
    tp_rank: int = 0
    tp_size: int = 1
    head_t: torch.Tensor = None  # the head in the tiled layout when its shape fits (head then None)
    step: torch.Tensor = None    # [passes, W] fp32: the vector added before each pass of a looped span (or None)
    ones: torch.Tensor = None    # [streams] fp32 ones of a design on several residual streams (or None)
    bigram: torch.Tensor = None  # [buckets + 1, W] hashed (previous token, token) rows added to the embedding (or None)
    side_embed: torch.Tensor = None  # [vocab, layers * dim] per-layer token inputs (or None)
    loop_in: torch.Tensor = None     # [W, 2 W] projection of [stream | embedding output] that opens a loop pass
    loop_in_t: torch.Tensor = None

    @property
    def vocab_local(self) -> int:
        return self.cfg.vocab_size

    @property
    def vocab_offset(self) -> int:
        return 0

    def nbytes(self) -> int:
        seen, n = set(), 0

        def size(obj) -> int:
            if isinstance(obj, torch.Tensor):
                return obj.numel() * obj.element_size()
            if obj is None or id(obj) in seen or not hasattr(obj, "__dataclass_fields__"):
                return 0
            seen.add(id(obj))
            return sum(size(v) for v in vars(obj).values())

        for L in self.layers:
            n += size(L)
        return n + sum(size(t) for t in (self.embed, self.final_norm, self.head, self.head_t, self.step, self.ones,
                                         self.bigram, self.side_embed, self.loop_in, self.loop_in_t))


TILED_MIN = 1024  # smallest N and K that go to the tiled-layout GEMMs


def fits_tiled(w: torch.Tensor) -> bool:
    """A bf16 [N, K] projection that the engine's tiled-layout GEMMs (ops.gemm_out: skinny / stream / wide / tiled /
    pipe kernels, picked per row count) serve at every row count: N % 128 == 0, K % 512 == 0, model-sized."""
    N, K = w.shape
    return (w.dtype == torch.bfloat16 and N % 128 == 0 and K % 512 == 0 and N >= TILED_MIN and K >= TILED_MIN
            and N * K * 2 < 2 ** 31)


def _tile_fields(obj, names) -> None:
    for n in names:
        w = getattr(obj, n)
        if w is not None and w.dim() == 2 and fits_tiled(w):
            setattr(obj, n + "_t", tile_weight(w))
            setattr(obj, n, None)


@torch.no_grad()
def convert_layered(cfg, tensors: dict, device="cpu", dtype=torch.bfloat16) -> LayeredWeights:
    """Checkpoint tensors {name: tensor} (models/muderax.py tensor_shapes) -> the engine's grouped layout in `dtype`
    (bf16 for serving; fp32 is the exact mode -- bf16 checkpoint values convert without loss)."""
    from ..models.muderax import tensor_shapes

    for name, shape in tensor_shapes(cfg).items():
        if name not in tensors:
            raise KeyError(f"checkpoint lacks tensor {name!r}")
        if tuple(tensors[name].shape) != tuple(shape):
            raise ValueError(f"tensor {name!r} has shape {tuple(tensors[name].shape)}, the configuration says {shape}")

    def t(name):
        return tensors[name].to(device=device, dtype=dtype).contiguous()

    def one(name):
        return t(name).reshape(1)

    own = {}
    for i, L in enumerate(cfg.layers):
        if L.weights_of != i:
            continue
        p, m = f"l{i}.", L.mixer
        if L.kind == "latent_attention":
            mix = LatentAttentionWeights(
                q=t(p + "mix.q"), dkv=t(p + "mix.dkv"), dkv_norm=t(p + "mix.dkv.norm"),
                uk_t=t(p + "mix.uk").view(m.heads, m.dim, m.kv_rank).transpose(1, 2).contiguous(),
                uv=t(p + "mix.uv").view(m.heads, m.vdim, m.kv_rank).contiguous(), o=t(p + "mix.o"))
        else:
            mix = RglruWeights(
                y=t(p + "mix.y"), y_b=t(p + "mix.y.b"), x=t(p + "mix.x"), x_b=t(p + "mix.x.b"), conv=t(p + "mix.conv"),
                conv_b=t(p + "mix.conv.b"), gates=torch.cat([t(p + "mix.ra"), t(p + "mix.ri")], dim=1).contiguous(),
                gates_b=torch.cat([t(p + "mix.ra.b"), t(p + "mix.ri.b")], dim=1).contiguous(), lam=t(p + "mix.lam"),
                o=t(p + "mix.o"))
        _tile_fields(mix, ("q", "o") if L.kind == "latent_attention" else ("y", "x", "o"))
        layer = LayeredLayer(norm1=one(p + "norm1"), mix=mix)
        if L.mlp is not None:
            f = L.mlp
            stack = lambda leaf: torch.stack([t(f"{p}mlp.e{e}.{leaf}") for e in range(f.experts)]).contiguous()  # noqa: E731
            layer.norm2 = one(p + "norm2")
            layer.mlp = MoeWeights(router=t(p + "mlp.router"), router_b=t(p + "mlp.router.b"), gate=stack("gate"),
                                   up=stack("up"), down=stack("down"))
            if f.shared_ff:
                layer.mlp.sgate, layer.mlp.sup, layer.mlp.sdown = (t(f"{p}mlp.shared.{leaf}")
                                                                   for leaf in ("gate", "up", "down"))
        own[i] = layer
    out = LayeredWeights(cfg=cfg, embed=t("embed"), layers=[own[L.weights_of] for L in cfg.layers],
                         final_norm=one("final.norm"), head=t("head"), dtype=dtype)
    _tile_fields(out, ("head",))
    return out


def load_layered_dir(cfg, path: str, device="cpu", dtype=torch.bfloat16) -> LayeredWeights:
    """``*.safetensors`` of a checkpoint directory -> LayeredWeights (the loader executes nothing from the files)."""
    from pathlib import Path

    from safetensors.torch import load_file

    tensors = {}
    for f in sorted(Path(path).glob("*.safetensors")):
        tensors.update(load_file(str(f)))
    return convert_layered(cfg, tensors, device=device, dtype=dtype)


# ---------------------------------------------------------------------------------------------------------------------
# Pre-norm designs with matrix-state mixers (models/surodra.py): every projection that reads the same input is ONE
# weight (its outputs are column ranges of one fp32 GEMM output) -- also the few-row ones (gates per head, the decay's
# inner projection), which come last; zero rows pad the fused weight to a multiple of 128 rows when it is large enough
# for the tiled-layout GEMMs.  Norm gains, sinks and decay parameters are fp32 in both element types.
@dataclass
class TanhNormWeights:
    alpha: torch.Tensor      # [1] fp32
    w: torch.Tensor          # [W] fp32
    b: torch.Tensor          # [W] fp32


@dataclass
class DeltaWeights:
    big: torch.Tensor        # rows [q (G D) | k (G D) | v (H V) | g (H V) | a (H) | b (H) | zero rows] x W
    n_big: int               # rows of big (the width of its output)
    conv: torch.Tensor       # [2 G D + H V, taps] fp32: the taps of q | k | v
    a_log: torch.Tensor      # [H] fp32
    dt_bias: torch.Tensor    # [H] fp32
    norm: torch.Tensor       # [V] fp32
    o: torch.Tensor          # [W, H V]
    big_t: torch.Tensor = None
    o_t: torch.Tensor = None


@dataclass
class ParallelWeights:
    big: torch.Tensor        # rows [left q | k | v | right q | k | v | g | left g (H) | right a1 (rank) | zeros] x W
    n_big: int
    q_norm: torch.Tensor     # fp32
    k_norm: torch.Tensor
    sink: torch.Tensor       # [H] fp32
    a2: torch.Tensor         # [Hr Dr, rank] fp32 (its input is the fp32 output of a1)
    a2_b: torch.Tensor       # [Hr Dr] fp32
    rnorm: torch.Tensor      # [Vr] fp32
    lo: torch.Tensor         # [W, H V]
    ro: torch.Tensor         # [W, Hr Vr]
    left_out: torch.Tensor   # [W] fp32
    right_out: torch.Tensor
    big_t: torch.Tensor = None
    lo_t: torch.Tensor = None
    ro_t: torch.Tensor = None


@dataclass
class RetentionWeights:
    big: torch.Tensor        # rows [q | k | v | g] x W
    decay: torch.Tensor      # [H] fp32
    o: torch.Tensor
    big_t: torch.Tensor = None
    o_t: torch.Tensor = None


@dataclass
class DenseFfWeights:
    gu: torch.Tensor         # rows [gate (F) | up (F)] x W
    down: torch.Tensor       # [W, F]
    gu_t: torch.Tensor = None
    down_t: torch.Tensor = None


@dataclass
class PreNormLayer:
    norm1: TanhNormWeights
    mix: object
    norm2: TanhNormWeights = None
    mlp: DenseFfWeights = None


@torch.no_grad()
def convert_surodra(cfg, tensors: dict, device="cpu", dtype=torch.bfloat16) -> LayeredWeights:
    """Checkpoint tensors {name: tensor} (models/surodra.py tensor_shapes) -> the engine's grouped layout in `dtype`."""
    from ..models.surodra import ANY, tensor_shapes

    for name, shape in tensor_shapes(cfg).items():
        if name not in tensors:
            raise KeyError(f"checkpoint lacks tensor {name!r}")
        got = tuple(tensors[name].shape)
        if len(got) != len(shape) or any(s != ANY and s != g for s, g in zip(shape, got)):
            raise ValueError(f"tensor {name!r} has shape {got}, the configuration says {shape}")

    def t(name):
        return tensors[name].to(device=device, dtype=dtype).contiguous()

    def f(name):
        return tensors[name].to(device=device, dtype=torch.float32).contiguous()

    def cat(*names):
        """The named projections as one weight; large ones are padded with zero rows to a multiple of 128 rows."""
        w = torch.cat([t(n) for n in names], dim=0)
        if w.shape[0] >= TILED_MIN and w.shape[0] % 128:
            w = torch.cat([w, w.new_zeros(128 - w.shape[0] % 128, w.shape[1])], dim=0)
        return w.contiguous()

    def norm(name):
        return TanhNormWeights(alpha=f(name + ".alpha").reshape(1), w=f(name), b=f(name + ".b"))

    layers = []
    for i, L in enumerate(cfg.layers):
        p = f"l{i}.mix."
        if L.kind == "delta":
            big = cat(p + "q", p + "k", p + "v", p + "g", p + "a", p + "b")
            mix = DeltaWeights(big=big, n_big=big.shape[0],
                               conv=torch.cat([f(p + "q.conv"), f(p + "k.conv"), f(p + "v.conv")]).contiguous(),
                               a_log=f(p + "A_log"), dt_bias=f(p + "dt_bias"), norm=f(p + "norm"), o=t(p + "o"))
            _tile_fields(mix, ("big", "o"))
        elif L.kind == "parallel":
            l, r = p + "left.", p + "right."
            if tensors[r + "a2"].shape[1] != tensors[r + "a1"].shape[0]:
                raise ValueError(f"layer {i}: the decay's two projections disagree on their inner width")
            big = cat(l + "q", l + "k", l + "v", r + "q", r + "k", r + "v", r + "g", l + "g", r + "a1")
            mix = ParallelWeights(big=big, n_big=big.shape[0], q_norm=f(l + "q.norm"), k_norm=f(l + "k.norm"),
                                  sink=f(l + "sink"), a2=f(r + "a2"), a2_b=f(r + "a2.b"), rnorm=f(r + "norm"),
                                  lo=t(l + "o"), ro=t(r + "o"), left_out=f(l + "out"), right_out=f(r + "out"))
            _tile_fields(mix, ("big", "lo", "ro"))
        else:
            mix = RetentionWeights(big=cat(p + "q", p + "k", p + "v", p + "g"),
                                   decay=torch.tensor(L.mixer.decay, dtype=torch.float32, device=device), o=t(p + "o"))
            _tile_fields(mix, ("big", "o"))
        layer = PreNormLayer(norm1=norm(f"l{i}.norm1"), mix=mix)
        if L.mlp is not None:
            layer.norm2 = norm(f"l{i}.norm2")
            layer.mlp = DenseFfWeights(gu=cat(f"l{i}.mlp.gate", f"l{i}.mlp.up"), down=t(f"l{i}.mlp.down"))
            _tile_fields(layer.mlp, ("gu", "down"))
        layers.append(layer)
    out = LayeredWeights(cfg=cfg, embed=t("embed"), layers=layers, final_norm=norm("final.norm"), head=t("head"),
                         dtype=dtype)
    out.step = f("loop.step") if cfg.loop_times > 0 else None
    _tile_fields(out, ("head",))
    return out


def load_surodra_dir(cfg, path: str, device="cpu", dtype=torch.bfloat16) -> LayeredWeights:
    """``*.safetensors`` of a checkpoint directory -> the engine's layout (the loader executes nothing from them)."""
    from pathlib import Path

    from safetensors.torch import load_file

    tensors = {}
    for f in sorted(Path(path).glob("*.safetensors")):
        tensors.update(load_file(str(f)))
    return convert_surodra(cfg, tensors, device=device, dtype=dtype)


# ---------------------------------------------------------------------------------------------------------------------
# Designs on several residual streams (models/dironex.py).  Projections that read the same input are ONE weight, as for
# the other pre-norm family; stream weights, norm gains, router corrections and activation constants are fp32 in both
# element types.  The latent attention kernels rotate interleaved pairs (2i, 2i + 1); this family pairs coordinate i
# with i + dims / 2, so the rows of the two projections that make the rotated parts (the query up-projection's rotated
# rows of every head, the down-projection's shared key rows) are permuted at load: pair i lands on (2i, 2i + 1) of both
# operands, a scalar product is the same under a common permutation, and nothing else reads those coordinates.
@dataclass
class StreamWeights:
    inw: torch.Tensor        # [S] fp32: the sublayer's input is sum_s inw[s] x_s
    outw: torch.Tensor       # [S] fp32: stream t receives mult * outw[t] * y
    mix: torch.Tensor        # [S, S] fp32, [from, to]
    norm: torch.Tensor       # [W] fp32 gain of the RMS norm on the input
    canon: torch.Tensor      # [W, taps] element type, or None


@dataclass
class GatedLatentWeights:
    big: torch.Tensor        # rows [dq (q_rank) | dkv (rk + dr, rotated rows interleaved) | g (H dv) | zero rows] x W
    n_big: int
    dq_norm: torch.Tensor    # [q_rank] fp32
    uq: torch.Tensor         # [H (dn + dr), q_rank], rotated rows of every head interleaved
    dkv_norm: torch.Tensor   # [rk] element type
    uk_t: torch.Tensor       # [H, rk, dn]
    uv: torch.Tensor         # [H, dv, rk]
    o: torch.Tensor          # [W, H dv]
    big_t: torch.Tensor = None
    uq_t: torch.Tensor = None
    o_t: torch.Tensor = None


@dataclass
class WindowAttentionWeights:
    big: torch.Tensor        # rows [q (H D) | k (G D) | v (G V) | zero rows] x W
    n_big: int
    q_norm: torch.Tensor     # [D] fp32
    k_norm: torch.Tensor     # [D] fp32
    o: torch.Tensor
    big_t: torch.Tensor = None
    o_t: torch.Tensor = None


@dataclass
class ActFfWeights:
    up: torch.Tensor         # [F, W]
    down: torch.Tensor       # [W, F]
    act: torch.Tensor        # [2] fp32: (softplus(p), 1/2 + softplus(q)) of the xIELU activation
    up_t: torch.Tensor = None
    down_t: torch.Tensor = None


@dataclass
class RoutedFfWeights:
    router: torch.Tensor     # [E, W] fp32 in both element types (the router runs in true fp32 on the fp32 row)
    correction: torch.Tensor  # [E] fp32
    up: torch.Tensor         # [E, F, W]
    down: torch.Tensor       # [E, W, F]


@dataclass
class StreamLayer:
    hc1: StreamWeights
    mix: object
    hc2: StreamWeights = None
    mlp: object = None


def interleave_half_pairs(width: int, dims: int) -> torch.Tensor:
    """Index list that moves a rotate-half pair (i, i + dims / 2) of a `width`-wide rotated part to (2i, 2i + 1); the
    coordinates from `dims` on keep their place."""
    idx = torch.arange(width)
    half = dims // 2
    idx[0:dims:2] = torch.arange(half)
    idx[1:dims:2] = torch.arange(half) + half
    return idx


@torch.no_grad()
def convert_dironex(cfg, tensors: dict, device="cpu", dtype=torch.bfloat16) -> LayeredWeights:
    """Checkpoint tensors {name: tensor} (models/dironex.py tensor_shapes) -> the engine's grouped layout in `dtype`."""
    from ..models.dironex import DenseSpec, tensor_shapes

    for name, shape in tensor_shapes(cfg).items():
        if name not in tensors:
            raise KeyError(f"checkpoint lacks tensor {name!r}")
        if tuple(tensors[name].shape) != tuple(shape):
            raise ValueError(f"tensor {name!r} has shape {tuple(tensors[name].shape)}, the configuration says {shape}")

    def t(name):
        return tensors[name].to(device=device, dtype=dtype).contiguous()

    def f(name):
        return tensors[name].to(device=device, dtype=torch.float32).contiguous()

    def cat(*parts):
        w = torch.cat(parts, dim=0)
        if w.shape[0] >= TILED_MIN and w.shape[0] % 128:
            w = torch.cat([w, w.new_zeros(128 - w.shape[0] % 128, w.shape[1])], dim=0)
        return w.contiguous()

    S, W = cfg.num_streams, cfg.width

    def stream(p, q):
        if cfg.streams > 0:
            inw, outw, mix = f(f"{p}hc{q}.in"), f(f"{p}hc{q}.out"), f(f"{p}hc{q}.mix")
        else:
            inw, outw, mix = (torch.ones(n, device=device, dtype=torch.float32) for n in ((1,), (1,), (1, 1)))
        return StreamWeights(inw=inw, outw=outw, mix=mix, norm=f(f"{p}norm{q}"),
                             canon=t(f"{p}canon{q}") if cfg.canon_taps > 0 else None)

    layers = []
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        if L.kind == "latent_attention":
            H, dn, dr, rk = m.heads, m.dim, m.rot_dim, m.kv_rank
            perm = interleave_half_pairs(dr, m.rot.dims).to(device)
            dkv = t(p + "mix.dkv")
            dkv = torch.cat([dkv[:rk], dkv[rk:][perm]], dim=0)
            uq = t(p + "mix.uq").view(H, dn + dr, m.q_rank)
            uq = torch.cat([uq[:, :dn], uq[:, dn:][:, perm]], dim=1).reshape(H * (dn + dr), m.q_rank).contiguous()
            big = cat(t(p + "mix.dq"), dkv, t(p + "mix.g"))
            mix = GatedLatentWeights(
                big=big, n_big=big.shape[0], dq_norm=f(p + "mix.dq.norm"), uq=uq, dkv_norm=t(p + "mix.dkv.norm"),
                uk_t=t(p + "mix.uk").view(H, dn, rk).transpose(1, 2).contiguous(),
                uv=t(p + "mix.uv").view(H, m.vdim, rk).contiguous(), o=t(p + "mix.o"))
            _tile_fields(mix, ("big", "uq", "o"))
        else:
            big = cat(t(p + "mix.q"), t(p + "mix.k"), t(p + "mix.v"))
            mix = WindowAttentionWeights(big=big, n_big=big.shape[0], q_norm=f(p + "mix.q.norm"),
                                         k_norm=f(p + "mix.k.norm"), o=t(p + "mix.o"))
            _tile_fields(mix, ("big", "o"))
        layer = StreamLayer(hc1=stream(p, "1"), mix=mix)
        fs = L.mlp
        if fs is not None:
            layer.hc2 = stream(p, "2")
            if isinstance(fs, DenseSpec):
                pq = tensors[p + "mlp.act"].to(torch.float64)
                sp = torch.nn.functional.softplus(pq)
                act = torch.stack([sp[0], 0.5 + sp[1]]).to(device=device, dtype=torch.float32)
                layer.mlp = ActFfWeights(up=t(p + "mlp.up"), down=t(p + "mlp.down"), act=act)
                _tile_fields(layer.mlp, ("up", "down"))
            else:
                stack = lambda leaf: torch.stack([t(f"{p}mlp.e{e}.{leaf}") for e in range(fs.experts)]).contiguous()  # noqa: E731
                layer.mlp = RoutedFfWeights(router=f(p + "mlp.router"), correction=f(p + "mlp.correction"),
                                            up=stack("up"), down=stack("down"))
        layers.append(layer)
    out = LayeredWeights(cfg=cfg, embed=t("embed"), layers=layers, final_norm=f("final.norm"), head=t("head"),
                         dtype=dtype)
    out.ones = torch.ones(S, device=device, dtype=torch.float32)   # the head reads the plain sum of the streams
    _tile_fields(out, ("head",))
    return out


def load_dironex_dir(cfg, path: str, device="cpu", dtype=torch.bfloat16) -> LayeredWeights:
    """``*.safetensors`` of a checkpoint directory -> the engine's layout (the loader executes nothing from them)."""
    from pathlib import Path

    from safetensors.torch import load_file

    tensors = {}
    for f in sorted(Path(path).glob("*.safetensors")):
        tensors.update(load_file(str(f)))
    return convert_dironex(cfg, tensors, device=device, dtype=dtype)


# ---------------------------------------------------------------------------------------------------------------------
# Designs with bracketing norms, hashed bigram embeddings and per-layer token inputs (models/murulorn.py).  Projections
# that read the same input are ONE weight, as for the other configuration-driven families; norm gains (stored around
# zero in the checkpoint: 1 + w is formed here, in fp32), decay parameters, the decay's and the output gate's second
# projections and the router are fp32 in both element types.  **Rotation layout**: the design rotates neighbouring
# coordinates (2i, 2i + 1); the engine's norm / rotation / attention kernels pair coordinate i with i + dims / 2.  The
# rows of the query and key projections (and their norm gains) are therefore permuted inside every head so that pair
# i lands on (i, i + dims / 2) -- a scalar product is the same under a common permutation of both operands and the
# whole-row RMS norm does not see the order -- and so are the rows of the value projection (whose per-head RMS norm
# does not see the order either) together with the COLUMNS of the output projection, which reads the heads' outputs in
# the values' order.
@dataclass
class RotatedValueAttentionWeights:
    big: torch.Tensor        # rows [q (H D) | k (G D) | v (G V) | g (H) | zero rows] x W, heads in rotate-half order
    n_big: int
    q_norm: torch.Tensor     # [H D] fp32, in the same order
    k_norm: torch.Tensor     # [G D] fp32
    o: torch.Tensor          # [W, H V], columns in the values' order
    big_t: torch.Tensor = None
    o_t: torch.Tensor = None


@dataclass
class ChannelDeltaWeights:
    big: torch.Tensor        # rows [q (G D) | k (G D) | v (H V) | b (H) | a1 (ra) | g1 (rg) | zero rows] x W
    n_big: int
    conv: torch.Tensor       # [2 G D + H V, taps] fp32: the taps of q | k | v
    a_log: torch.Tensor      # [H] fp32
    dt_bias: torch.Tensor    # [H D] fp32
    ag2: torch.Tensor        # [H D + H V, ra + rg] fp32, block-diagonal: the decay's and the gate's second projections
                             # as ONE product on the adjacent fp32 outputs of a1 and g1 (rows [a2 | 0] then [0 | g2])
    ra: int                  # inner widths of the two pairs
    rg: int
    norm: torch.Tensor       # [V] fp32
    o: torch.Tensor          # [W, H V]
    big_t: torch.Tensor = None
    o_t: torch.Tensor = None


@dataclass
class SquaredReluFfWeights:
    up: torch.Tensor         # [F, W]
    down: torch.Tensor       # [W, F]
    up_t: torch.Tensor = None
    down_t: torch.Tensor = None


@dataclass
class SoftmaxRoutedFfWeights:
    router: torch.Tensor     # [E, W] fp32 in both element types (the router runs in true fp32 on the fp32 row)
    up: torch.Tensor         # [E, F, W]
    down: torch.Tensor       # [E, W, F]


@dataclass
class TokenSideWeights:
    gate: torch.Tensor       # [dim, W]
    proj: torch.Tensor       # [W, dim]
    norm: torch.Tensor       # [W] fp32, a plain gain
    col0: int                # the layer's first column of the side table


@dataclass
class BracketLayer:
    norm1: torch.Tensor      # [W] fp32 gains (1 + stored) of the norm before the mixer ...
    norm1b: torch.Tensor     # ... and after it
    mix: object
    norm2: torch.Tensor = None
    norm2b: torch.Tensor = None
    mlp: object = None
    side: TokenSideWeights = None


def half_from_pairs(width: int, dims: int) -> torch.Tensor:
    """Index list that moves a neighbouring pair (2i, 2i + 1) of the first `dims` of `width` coordinates to
    (i, i + dims / 2): new[j] = old[index[j]]; the coordinates from `dims` on keep their place."""
    idx = torch.arange(width)
    half = dims // 2
    if half > 0:
        idx[:half] = torch.arange(0, dims, 2)
        idx[half:dims] = torch.arange(1, dims, 2)
    return idx


@torch.no_grad()
def convert_murulorn(cfg, tensors: dict, device="cpu", dtype=torch.bfloat16) -> LayeredWeights:
    """Checkpoint tensors {name: tensor} (models/murulorn.py tensor_shapes) -> the engine's grouped layout in `dtype`."""
    from ..models.murulorn import ANY, SquaredReluSpec, tensor_shapes

    for name, shape in tensor_shapes(cfg).items():
        if name not in tensors:
            raise KeyError(f"checkpoint lacks tensor {name!r}")
        got = tuple(tensors[name].shape)
        if len(got) != len(shape) or any(s != ANY and s != g for s, g in zip(shape, got)):
            raise ValueError(f"tensor {name!r} has shape {got}, the configuration says {shape}")

    def t(name):
        return tensors[name].to(device=device, dtype=dtype).contiguous()

    def f(name):
        return tensors[name].to(device=device, dtype=torch.float32).contiguous()

    def gain(name):
        return (1.0 + tensors[name].to(device=device, dtype=torch.float32)).contiguous()

    def cat(*parts):
        w = torch.cat(parts, dim=0)
        if w.shape[0] >= TILED_MIN and w.shape[0] % 128:
            w = torch.cat([w, w.new_zeros(128 - w.shape[0] % 128, w.shape[1])], dim=0)
        return w.contiguous()

    def heads_perm(n_heads: int, width: int, dims: int) -> torch.Tensor:
        one = half_from_pairs(width, dims)
        return (torch.arange(n_heads)[:, None] * width + one[None, :]).reshape(-1).to(device)

    W = cfg.width
    layers = []
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        if L.kind == "attention":
            pq, pk = heads_perm(m.heads, m.dim, m.rot_dims), heads_perm(m.kv_heads, m.dim, m.rot_dims)
            pv, po = heads_perm(m.kv_heads, m.vdim, m.vdim), heads_perm(m.heads, m.vdim, m.vdim)
            big = cat(t(p + "mix.q")[pq], t(p + "mix.k")[pk], t(p + "mix.v")[pv], t(p + "mix.g"))
            mix = RotatedValueAttentionWeights(big=big, n_big=big.shape[0], q_norm=f(p + "mix.q.norm")[pq].contiguous(),
                                               k_norm=f(p + "mix.k.norm")[pk].contiguous(),
                                               o=t(p + "mix.o")[:, po].contiguous())
        else:
            if tensors[p + "mix.a2"].shape[1] != tensors[p + "mix.a1"].shape[0] or \
                    tensors[p + "mix.g2"].shape[1] != tensors[p + "mix.g1"].shape[0]:
                raise ValueError(f"layer {i}: a low-rank pair disagrees on its inner width")
            big = cat(t(p + "mix.q"), t(p + "mix.k"), t(p + "mix.v"), t(p + "mix.b"), t(p + "mix.a1"), t(p + "mix.g1"))
            mix = ChannelDeltaWeights(big=big, n_big=big.shape[0],
                                      conv=torch.cat([f(p + "mix.q.conv"), f(p + "mix.k.conv"),
                                                      f(p + "mix.v.conv")]).contiguous(),
                                      a_log=f(p + "mix.A_log"), dt_bias=f(p + "mix.dt_bias"),
                                      ag2=torch.block_diag(f(p + "mix.a2"), f(p + "mix.g2")).contiguous(),
                                      ra=tensors[p + "mix.a2"].shape[1], rg=tensors[p + "mix.g2"].shape[1],
                                      norm=f(p + "mix.norm"), o=t(p + "mix.o"))
        _tile_fields(mix, ("big", "o"))
        layer = BracketLayer(norm1=gain(p + "norm1"), norm1b=gain(p + "norm1b"), mix=mix)
        fs = L.mlp
        if fs is not None:
            layer.norm2, layer.norm2b = gain(p + "norm2"), gain(p + "norm2b")
            if isinstance(fs, SquaredReluSpec):
                layer.mlp = SquaredReluFfWeights(up=t(p + "mlp.up"), down=t(p + "mlp.down"))
                _tile_fields(layer.mlp, ("up", "down"))
            else:
                stack = lambda leaf: torch.stack([t(f"{p}mlp.e{e}.{leaf}") for e in range(fs.experts)]).contiguous()  # noqa: E731
                layer.mlp = SoftmaxRoutedFfWeights(router=f(p + "mlp.router"), up=stack("up"), down=stack("down"))
        if cfg.side_dim:
            layer.side = TokenSideWeights(gate=t(p + "side.gate"), proj=t(p + "side.proj"), norm=f(p + "side.norm"),
                                          col0=i * cfg.side_dim)
        layers.append(layer)
    embed = t("embed")
    out = LayeredWeights(cfg=cfg, embed=embed, layers=layers, final_norm=gain("final.norm"), head=embed, dtype=dtype)
    if fits_tiled(embed):    # the head is the embedding table: the gather keeps the row-major copy
        out.head_t, out.head = tile_weight(embed), None
    out.bigram = t("bigram") if cfg.bigram else None
    out.side_embed = t("side.embed") if cfg.side_dim else None
    if cfg.loop_times > 0:
        out.loop_in = t("loop.in")
        _tile_fields(out, ("loop_in",))
    return out


def load_murulorn_dir(cfg, path: str, device="cpu", dtype=torch.bfloat16) -> LayeredWeights:
    """``*.safetensors`` of a checkpoint directory -> the engine's layout (the loader executes nothing from them)."""
    from pathlib import Path

    from safetensors.torch import load_file

    tensors = {}
    for f in sorted(Path(path).glob("*.safetensors")):
        tensors.update(load_file(str(f)))
    return convert_murulorn(cfg, tensors, device=device, dtype=dtype)
