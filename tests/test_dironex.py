"""Dironex on the engine against the plain oracle (tests/dironex_oracle.py).

Every test builds its own small configuration and random weights, drives the engine through its own entry points
(LLMEngine.force_step for given tokens, add_request + step for generation) and compares the logits with the oracle's
whole-sequence forward in float64.  The same tests run on the CPU (PyTorch reference ops: scheduler, cache and state
plumbing) and, marked ``gpu``, on the HIP kernels in fp32 (every row, tight tolerance) and bf16 (the bulk of the rows:
a close router call flips under bf16 rounding in these tiny random models and moves single rows).
"""
from __future__ import annotations

import copy
import json

import pytest
import torch

import dironex_oracle as oracle
from distributed_sse_for_llm_response_amd.engine.engine import LLMEngine, SamplingParams
from distributed_sse_for_llm_response_amd.engine.model_runner import PrefillSeq
from distributed_sse_for_llm_response_amd.engine.weights import convert_dironex, interleave_half_pairs
from distributed_sse_for_llm_response_amd.models import registry
from distributed_sse_for_llm_response_amd.models.dironex import DironexConfig, init_weights, tensor_shapes

GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVICES = ["cpu", GPU]
VOCAB = 53


def rot(dims, base=400.0, yarn=True):
    r = {"base": base, "dims": dims}
    if yarn:
        r["scaling"] = {"factor": 3.0, "original": 24, "fast": 4.0, "slow": 0.5}
    return r


def lat(heads=3, dim=10, rot_dim=6, vdim=7, kv_rank=12, q_rank=9, scale=0.25, dims=None, yarn=True, mlp=None):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "scale": scale, "rot": rot(rot_dim if dims is None else dims, yarn=yarn)}}


def att(heads=4, kv_heads=2, dim=10, vdim=6, window=9, scale=0.3, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    return {"type": "attention", "mlp": mlp, "mixer": m}


def dense(n=20):
    return {"kind": "dense", "ff": n}


def moe(experts=6, top=2, ff=9, groups=3, keep=2, scale=1.7):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def config(layers, width=26, vocab=VOCAB, eps=3e-6, loop=None, mult=0.4, streams=2, taps=3, embed_scale=1.5):
    d = {"architecture": "Dironex", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "layers": copy.deepcopy(layers), "residual_mult": mult, "embedding": {"scale": embed_scale}}
    if streams:
        d["streams"] = streams
    if taps:
        d["canon"] = {"taps": taps}
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


HYBRID = config([lat(mlp=dense()), att(mlp=moe()), lat(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=8, q_rank=8, mlp=moe(top=3)),
                 att(heads=2, kv_heads=2, window=33, mlp=dense(11))], loop=(1, 3, 2))


class Model:
    """Configuration + random weights + an engine on `device` in `dtype`."""

    def __init__(self, cfg_dict, device, dtype=torch.float32, seed=0, max_tokens=256, max_seqs=4, tweak=None):
        self.cfg_dict = cfg_dict
        self.cfg = DironexConfig.from_dict(cfg_dict)
        self.weights = init_weights(self.cfg, seed=seed)
        if tweak:
            tweak(self.weights)
        self.device, self.dtype = torch.device(device), dtype
        w = convert_dironex(self.cfg, self.weights, device=self.device, dtype=dtype)
        fam = registry.family_of(self.cfg)
        assert fam.name == "dironex"
        self.runner = registry.make_runner(fam, w, num_blocks=-(-max_tokens // 32), max_batch=max_seqs,
                                           max_model_len=max_tokens, max_prefill_tokens=max_tokens, device=self.device,
                                           use_graphs=False)
        self.engine = LLMEngine(self.runner, eos_id=-1)
        self.engine.watermark = 0

    def expect(self, tokens, cfg_dict=None, weights=None):
        return oracle.forward(cfg_dict or self.cfg_dict, weights or self.weights, tokens)[0].float()

    def check(self, got, want, what=""):
        """Row-wise: rms of the difference (mean taken off) over the rms of the expected logits.  fp32 judges every
        row; bf16 judges nine rows in ten and the median."""
        got, want = got.detach().float().cpu(), want.float()
        assert got.shape == want.shape, (got.shape, want.shape)
        assert torch.isfinite(got).all(), what
        d = got - want
        d = d - d.mean(-1, keepdim=True)
        err = d.pow(2).mean(-1).sqrt() / (want - want.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt().clamp_min(1e-6)
        if self.dtype == torch.float32:
            assert float(err.max()) < 2e-4, f"{what}: worst row {int(err.argmax())} error {float(err.max()):.3g}"
        else:
            assert float((err < 6e-2).float().mean()) >= 0.9 and float(err.median()) < 3e-2, \
                f"{what}: median {float(err.median()):.3g}, {int((err >= 6e-2).sum())} of {err.numel()} rows off"

    def run_cut(self, cid, tokens, cuts, end=True):
        """Feed `tokens` in portions of the given sizes (the last size repeats), all logits wanted."""
        out, at, k = [], 0, 0
        while at < len(tokens):
            n = min(cuts[min(k, len(cuts) - 1)], len(tokens) - at)
            last = at + n == len(tokens)
            out.append(self.engine.force_step([(cid, tokens[at:at + n], list(range(n)))], [cid] if last and end else []))
            at, k = at + n, k + 1
        return torch.cat(out)


def toks(n, vocab=VOCAB, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def modes(device):
    return [torch.float32] if device == "cpu" else [torch.float32, torch.bfloat16]


def gap(a, b, rows=slice(None)):
    """Median over rows of |a - b| rms relative to b's rms: how far a variant of the design is from the design."""
    a, b = a[rows], b[rows]
    return float(((a - b).pow(2).mean(-1).sqrt() / b.pow(2).mean(-1).sqrt().clamp_min(1e-6)).median())


def gap_max(a, b, rows=slice(None)):
    """The largest such difference over the rows: whether a variant changes ANY of them."""
    a, b = a[rows], b[rows]
    return float(((a - b).pow(2).mean(-1).sqrt() / b.pow(2).mean(-1).sqrt().clamp_min(1e-6)).max())


def scaled(names_and_factors):
    """A weight tweak: tensors whose name ends with a given suffix are multiplied by a factor."""
    def tweak(w):
        for k in w:
            for suffix, f in names_and_factors:
                if k.endswith(suffix):
                    w[k] = (w[k].float() * f).to(w[k].dtype)
    return tweak


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,cfgd", [
    ("latent attention, YaRN rotation", config([lat()], streams=0, taps=0)),
    ("latent attention, plain rotation of part of the rotated slice", config([lat(dims=4, yarn=False)], streams=0, taps=0)),
    ("latent attention, one head, no unrotated part", config([lat(heads=1, dim=0, rot_dim=8)], streams=0, taps=0)),
    ("windowed attention, grouped heads", config([att()], streams=0, taps=0)),
    ("windowed attention, a key head per head, no window", config([att(heads=3, kv_heads=3, window=None)], streams=0, taps=0)),
    ("windowed attention, one key head, window of one", config([att(heads=3, kv_heads=1, window=1)], streams=0, taps=0)),
    ("dense feed-forward", config([att(heads=1, kv_heads=1, mlp=dense())], streams=0, taps=0)),
    ("routed experts in groups", config([att(heads=1, kv_heads=1, mlp=moe())], streams=0, taps=0)),
    ("routed experts, no groups, one expert per token", config([att(mlp=moe(experts=5, top=1, groups=None))], streams=0, taps=0)),
    ("routed experts, groups of one, all kept", config([att(mlp=moe(experts=4, top=4, groups=4, keep=4))], streams=0, taps=0)),
    ("input convolution alone", config([att(mlp=dense())], streams=0, taps=4)),
    ("one tap", config([lat(mlp=dense())], streams=0, taps=1)),
    ("several streams alone", config([att(mlp=dense())], streams=3, taps=0)),
    ("one stream with its own weights", config([lat(mlp=moe())], streams=1, taps=2)),
    ("five streams", config([lat(mlp=dense()), att()], streams=5, taps=5)),
    ("unit multiplier and embedding scale", config([lat(mlp=dense())], mult=1.0, embed_scale=1.0)),
    ("a loop of one layer, three passes", config([att(), lat(mlp=moe()), att(mlp=dense())], loop=(1, 2, 3))),
    ("a loop of everything, one pass", config([lat(), att(mlp=dense())], loop=(0, 2, 1))),
])
def test_mechanism_alone(device, name, cfgd):
    for dtype in modes(device):
        m = Model(cfgd, device, dtype)
        t = toks(37, seed=1)
        m.check(m.run_cut("a", t, [len(t)]), m.expect(t), name + ", whole")
        m.check(m.run_cut("b", t, [9, 1]), m.expect(t), name + ", decoding")


def test_each_op_against_its_oracle_function():
    """The reference ops the CPU engine runs on, one mechanism at a time, against the oracle's functions."""
    from distributed_sse_for_llm_response_amd import ops
    g = torch.Generator().manual_seed(5)
    # routing: groups, correction in the choice only, normalised weights
    z = torch.randn(40, 12, generator=g)
    corr = torch.randn(12, generator=g) * 0.4
    r = {"experts": 12, "top": 3, "scale": 1.3, "groups": {"count": 4, "keep": 2}}
    idx, w = oracle.route(z.double(), corr.double(), r)
    ti, tw = torch.zeros(40, 3, dtype=torch.int32), torch.zeros(40, 3)
    ops.moe_route(z, corr, ti, tw, 4, 2, 1.3)
    assert torch.equal(ti.long().sort(-1).values, idx.sort(-1).values)
    assert torch.allclose(tw.gather(1, ti.long().argsort(-1)), w.float().gather(1, idx.argsort(-1)), atol=1e-6)
    assert not torch.equal(idx.sort(-1).values, oracle.route(z.double(), corr.double() * 0, r)[0].sort(-1).values)
    assert not torch.equal(idx.sort(-1).values,
                           oracle.route(z.double(), corr.double(), {**r, "groups": None})[0].sort(-1).values)
    # activation rows
    x = torch.randn(9, 14, generator=g) * 2
    pq = torch.tensor([0.3, -0.2], dtype=torch.float64)
    sp = torch.nn.functional.softplus(pq)
    out = torch.zeros(9, 14)
    ops.act_rows(x, out, 1, torch.stack([sp[0], 0.5 + sp[1]]).float())
    assert torch.allclose(out, oracle.xielu(x.double(), pq[0], pq[1]).float(), atol=1e-5)
    # streams: mix indexed [from, to]
    S, W = 3, 8
    streams = torch.randn(5, S, W, generator=g)
    y = torch.randn(5, W, generator=g)
    hc = (torch.randn(S, generator=g), torch.randn(S, generator=g), torch.randn(S, S, generator=g))
    nw = torch.randn(W, generator=g)
    want = oracle.sublayer(streams.permute(1, 0, 2).double(), tuple(t.double() for t in hc), nw.double(), None,
                           lambda h: y.double(), 0.7, 1e-5)
    got, h = streams.clone(), torch.zeros(5, W)
    ops.stream_mix(y, 1, 0.7, got, out_w=hc[1], mix=hc[2], in_w=hc[0], norm_w=nw, eps=1e-5, h=h)
    assert torch.allclose(got.permute(1, 0, 2), want.float(), atol=1e-5)
    u = torch.einsum("s,msw->mw", hc[0], got)
    assert torch.allclose(h, (oracle.rms(u.double(), 1e-5) * nw.double()).float(), atol=1e-5)


def test_rotation_layout_and_table():
    """The rotate-half pairs (i, i + dims / 2) land on interleaved pairs (2i, 2i + 1) of the kernels' rotated part, and
    the engine's (cos, sin) table holds the oracle's YaRN frequencies and amplitude."""
    idx = interleave_half_pairs(10, 6)
    assert idx.tolist() == [0, 3, 1, 4, 2, 5, 6, 7, 8, 9]
    cfg = DironexConfig.from_dict(config([lat(rot_dim=8, dims=6)]))
    spec = cfg.layers[0].mixer.rot
    table = spec.table(50, 8)
    f, amp = oracle.yarn_frequencies(config([lat(rot_dim=8, dims=6)])["layers"][0]["mixer"]["rot"])
    ang = torch.arange(50, dtype=torch.float64)[:, None] * f[None, :]
    assert torch.allclose(table[:, :3, 0].double(), ang.cos() * amp, atol=1e-6)
    assert torch.allclose(table[:, :3, 1].double(), ang.sin() * amp, atol=1e-6)
    assert torch.equal(table[:, 3], torch.tensor([1.0, 0.0]).expand(50, 2)) and amp > 1.0
    assert float((f - oracle.yarn_frequencies(rot(6, yarn=False))[0]).abs().max()) > 1e-3


@pytest.mark.parametrize("device", DEVICES)
def test_layer_trace(device):
    """The engine's layer trace (sum of the streams after every layer run) against the oracle's."""
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype)
        t = toks(21, seed=2)
        got = []
        m.runner.prefill([PrefillSeq(slot=0, tokens=t, start_pos=0, block_table=[0], last_chunk=False)], 0, trace=got)
        want = oracle.forward(HYBRID, m.weights, t)[1]
        assert len(got) == len(want) == 6
        tol = 1e-4 if dtype == torch.float32 else 3e-2
        for i, (a, b) in enumerate(zip(got, want)):
            assert float((a.cpu().double() - b).abs().max() / b.abs().max()) < tol, f"layer run {i}"


# ---------------------------------------------------------------------------------------------- cuts, batches, pools
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_against_token_by_token(device):
    t = toks(45, seed=3)
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype)
        want = m.expect(t)
        whole = m.run_cut("w", t, [len(t)])
        single = m.run_cut("s", t, [1])
        m.check(whole, want, "whole prompt")
        m.check(single, want, "token by token")
        if dtype == torch.float32:
            m.check(single, whole.cpu(), "token by token against the whole prompt")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[2], [3, 2, 7], [5, 1, 1, 2, 11], [31, 2, 1], [33, 1], [64, 2]])
def test_portions(device, cuts):
    """Portions cut inside pages, windows and the convolution's reach, down to two tokens."""
    t = toks(70, seed=4)
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype)
        m.check(m.run_cut("p", t, cuts), m.expect(t), f"portions {cuts}")


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_against_each_alone(device):
    """Four requests of unequal length in one batch: portions of some beside single tokens of others, one sits out
    steps, one ends early and its slot and pages go to a newcomer."""
    seqs = {"a": toks(50, seed=5), "b": toks(9, seed=6), "c": toks(34, seed=7), "d": toks(1, seed=8), "e": toks(40, seed=9)}
    plan = [{"a": 7, "b": 2, "c": 20}, {"a": 1, "b": 1, "d": 1}, {"a": 1, "c": 2, "b": 1}, {"a": 30, "b": 1, "e": 3},
            {"a": 1, "b": 1, "c": 1, "e": 33}, {"a": 1, "b": 1, "c": 11, "e": 1}, {"a": 9, "b": 2, "e": 3}]
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype, max_tokens=256)
        at = {k: 0 for k in seqs}
        got = {k: [] for k in seqs}
        for step in plan:
            entries, end = [], []
            for k, n in step.items():
                n = min(n, len(seqs[k]) - at[k])
                entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
                at[k] += n
                if at[k] == len(seqs[k]):
                    end.append(k)
            out = m.engine.force_step(entries, end)
            o = 0
            for k, tk, _ in entries:
                got[k].append(out[o:o + len(tk)])
                o += len(tk)
        for k, t in seqs.items():
            assert at[k] == len(t), k
            m.check(torch.cat(got[k]), m.expect(t), f"request {k} in the batch")
        assert m.engine.alloc.num_free == m.engine.alloc.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_pages_and_slots_used_again(device):
    """A pool of three pages and two slots: every later request runs in pages and slots that held another one (its
    keys, its convolution tails), in prompts and in decoding."""
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype, max_tokens=96, max_seqs=2)
        for i, (n, cuts) in enumerate([(60, [60]), (64, [33, 1]), (40, [2, 30, 1]), (64, [64]), (5, [1])]):
            t = toks(n, seed=30 + i)
            keep = toks(20, seed=40 + i)
            first = m.engine.force_step([(f"k{i}", keep[:10], list(range(10)))])
            got = m.run_cut(f"r{i}", t, cuts)
            rest = m.engine.force_step([(f"k{i}", keep[10:], list(range(10)))], [f"k{i}"])
            m.check(got, m.expect(t), f"request {i}")
            m.check(torch.cat([first, rest]), m.expect(keep), f"neighbour of request {i}")
        assert m.engine.alloc.num_free == m.engine.alloc.num_blocks
    m.engine.force_step([("held", toks(64, seed=1), [])])
    with pytest.raises(MemoryError):
        m.engine.force_step([("late", toks(64, seed=2), [])])


# ---------------------------------------------------------------------------------------------- far keys and edges
@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds(device):
    """Latent attention made sharp (queries scaled up): single far keys carry the weight.  Changing the second token
    moves logits 250 tokens later in the oracle, and the engine agrees with it in prompts cut at page borders and in
    decoding."""
    cfgd = config([lat(heads=2, dim=8, rot_dim=4, vdim=6, kv_rank=10, q_rank=7, scale=0.5)], streams=2, taps=2)
    sharp = scaled([("mix.uq", 3.0)])
    t = toks(300, seed=10)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, max_tokens=320, tweak=sharp)
        want = m.expect(t)
        moved = list(t)
        moved[1] = (moved[1] + 11) % VOCAB
        assert gap_max(m.expect(moved), want, slice(250, None)) > 5e-2, "early tokens do not matter in this construction"
        m.check(m.run_cut("a", t, [256, 1]), want, "prompt to a page border, then decoding")
        m.check(m.run_cut("b", t, [32, 64, 33, 2, 97, 1]), want, "portions on and off page borders")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window", [1, 2, 31, 32, 33, 40, 70])
def test_window_edges(device, window):
    """Sharp windowed attention: the key just inside the window counts and the one just outside does not, in prompts
    and in decoding.  The oracle with a window one token larger or smaller is far from the design in the rows whose
    strongest key sits at the edge (every row is judged against the design)."""
    def cfg_w(w):
        return config([att(heads=2, kv_heads=1, dim=8, vdim=6, window=w, scale=1.0)], streams=2, taps=0)

    sharp = scaled([("q.norm", 2.0), ("k.norm", 2.0)])
    t = toks(110, seed=11)
    for dtype in modes(device):
        m = Model(cfg_w(window), device, dtype, tweak=sharp)
        want = m.expect(t)
        for other in (window + 1, window - 1):
            if other >= 1:
                assert gap_max(m.expect(t, cfg_w(other)), want, slice(window + 1, None)) > 1e-2, other
        m.check(m.run_cut("p", t, [len(t)]), want, "prompt")
        m.check(m.run_cut("d", t, [max(1, window - 1), 1]), want, "decoding over the edge")
        m.check(m.run_cut("c", t, [window + 1, 2, 31, 1]), want, "portions over the edge")


@pytest.mark.parametrize("device", DEVICES)
def test_convolution_reaches_over_cuts(device):
    """The input convolution with large taps: a portion's first rows read the tail that the step before left, also
    when that step was shorter than the tail; the oracle without the convolution is far away."""
    cfgd = config([att(mlp=dense()), lat(mlp=moe())], streams=2, taps=5)
    big = scaled([("canon1", 3.0), ("canon2", 3.0)])
    t = toks(40, seed=12)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, tweak=big)
        want = m.expect(t)
        none = {k: (v * 0 if "canon" in k else v) for k, v in m.weights.items()}
        assert gap(m.expect(t, weights=none), want) > 5e-2
        for cuts in ([2], [1], [3, 1, 1, 2, 6, 1], [4, 5, 1]):
            m.check(m.run_cut("c", t, cuts), want, f"portions {cuts}")


@pytest.mark.parametrize("device", DEVICES)
def test_router_correction_and_groups_matter(device):
    """Large corrections decide which experts run (but not their weights) and the group limit removes experts: the
    oracle without either is far away, the engine follows the design."""
    cfgd = config([att(mlp=moe(experts=8, top=2, groups=4, keep=1, scale=2.5))], streams=2, taps=2)
    t = toks(40, seed=13)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, tweak=scaled([("correction", 3.0)]))
        want = m.expect(t)
        flat = copy.deepcopy(cfgd)
        del flat["layers"][0]["mlp"]["router"]["groups"]
        assert gap(m.expect(t, flat), want) > 1e-2
        assert gap(m.expect(t, weights={k: (v * 0 if k.endswith("correction") else v) for k, v in m.weights.items()}),
                   want) > 1e-2
        m.check(m.run_cut("r", t, [17, 2, 1]), want, "routing")


@pytest.mark.parametrize("device", DEVICES)
def test_stream_weights_matter(device):
    """The mix matrix is indexed [from, to]: the oracle with it transposed is far away."""
    cfgd = config([lat(mlp=dense()), att(mlp=dense())], streams=3, taps=0)
    t = toks(30, seed=14)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, tweak=scaled([(".mix", 1.0)]))
        want = m.expect(t)
        flipped = {k: (v.t().contiguous() if k.endswith(".mix") and "hc" in k else v) for k, v in m.weights.items()}
        assert gap(m.expect(t, weights=flipped), want) > 1e-2
        m.check(m.run_cut("s", t, [11, 1]), want, "streams")


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(device):
    """Positions 0, 1, 2: the convolution's empty history and one-key attention; as a one-token request, as single
    tokens from the start, and in a slot that held another sequence."""
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype, max_seqs=1)
        m.run_cut("warm", toks(40, seed=15), [40])
        for n in (1, 2, 3):
            t = toks(n, seed=16 + n)
            m.check(m.run_cut(f"n{n}", t, [1]), m.expect(t), f"{n} first tokens, one by one")
            m.check(m.run_cut(f"w{n}", t, [n]), m.expect(t), f"{n} first tokens, at once")


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(device):
    """Decoding runs over several pages and past the windows."""
    t = toks(150, seed=20)
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype)
        m.check(m.run_cut("l", t, [5, 1]), m.expect(t), "long decoding")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,cfgd", [
    ("all ones", config([lat(heads=1, dim=1, rot_dim=2, vdim=1, kv_rank=1, q_rank=1, mlp=dense(1)),
                         att(heads=1, kv_heads=1, dim=1, vdim=1, window=1, mlp=moe(experts=1, top=1, ff=1, groups=1, keep=1))],
                        width=2, vocab=7, streams=1, taps=1, loop=(0, 2, 1))),
    ("odd sizes", config([lat(heads=5, dim=7, rot_dim=10, vdim=9, kv_rank=13, q_rank=11, dims=6, mlp=moe(experts=9, top=4, ff=7, groups=3, keep=2)),
                          att(heads=6, kv_heads=3, dim=14, vdim=5, window=13, mlp=dense(17))], width=19, vocab=23,
                         streams=4, taps=2, loop=(0, 2, 2))),
    ("sizes that vector loads like", config([lat(heads=4, dim=32, rot_dim=32, vdim=32, kv_rank=64, q_rank=48, mlp=dense(128)),
                                             att(heads=8, kv_heads=2, dim=64, vdim=32, window=48,
                                                 mlp=moe(experts=8, top=2, ff=64, groups=2, keep=1))], width=64, vocab=96, taps=4)),
    ("wide ranks and heads", config([lat(heads=2, dim=72, rot_dim=40, vdim=136, kv_rank=264, q_rank=520),
                                     att(heads=2, kv_heads=1, dim=136, vdim=72, window=20)], width=48, vocab=50)),
    ("projections on the tiled-layout GEMMs", config([lat(heads=8, dim=128, rot_dim=64, vdim=128, kv_rank=128, q_rank=1024, mlp=dense(2048)),
                                                      att(heads=8, kv_heads=4, dim=128, vdim=128, window=40,
                                                          mlp=moe(experts=4, top=2, ff=256, groups=2, keep=2))],
                                                     width=1024, vocab=1024)),
])
def test_other_sizes(device, name, cfgd):
    vocab = cfgd["vocab"]
    t = toks(41, vocab=vocab, seed=21)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype)
        m.check(m.run_cut("x", t, [len(t)]), m.expect(t), name + ", whole")
        m.check(m.run_cut("y", t, [7, 2, 1]), m.expect(t), name + ", portions and decoding")


@pytest.mark.gpu
def test_long_prompt_of_many_tiles():
    """Six hundred tokens on the GPU: prompt-sized expert tiles, attention tiles over many pages, windows inside."""
    cfgd = config([lat(heads=4, dim=32, rot_dim=32, vdim=32, kv_rank=64, q_rank=48, mlp=moe(experts=8, top=2, ff=64, groups=4, keep=2)),
                   att(heads=4, kv_heads=2, dim=32, vdim=32, window=100, mlp=dense(128))], width=64, vocab=200, taps=4,
                  streams=3, loop=(0, 2, 2))
    t = toks(600, vocab=200, seed=22)
    for dtype in (torch.float32, torch.bfloat16):
        m = Model(cfgd, "cuda", dtype, max_tokens=640)
        want = m.expect(t)
        m.check(m.run_cut("a", t, [560, 1]), want, "prompt, then decoding")
        m.check(m.run_cut("b", t, [300, 3, 257, 1]), want, "portions")


# ---------------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(device):
    """add_request + step: admission, chunked prompt passes (a 16-token budget), mixed steps, decode with sampling at
    temperature 0, slot release.  Each generated token is the oracle's argmax given the tokens before it (a step
    whose two best logits are closer than the tolerance is not judged)."""
    m = Model(HYBRID, device, torch.float32, max_tokens=512, max_seqs=3)
    eng = LLMEngine(m.runner, eos_id=-1, prefill_budget=16, idle_prefill_budget=16)
    prompts = {"g0": toks(19, seed=23), "g1": toks(40, seed=24), "g2": toks(3, seed=25), "g3": toks(33, seed=26)}
    for cid, p in prompts.items():
        eng.add_request(cid, p, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    out = {cid: [] for cid in prompts}
    for ev in eng.run_until_idle():
        if not ev.done:
            out[ev.conversation_id].append(ev.token_id)
    for cid, p in prompts.items():
        assert len(out[cid]) == 12, (cid, out[cid])
        logits = m.expect(p + out[cid])
        for i, tok in enumerate(out[cid]):
            row = logits[len(p) + i - 1]
            top = torch.topk(row, 2).values
            if float(top[0] - top[1]) > 1e-3 * float(row.abs().max()):
                assert tok == int(row.argmax()), f"{cid}: token {i} is {tok}, the oracle says {int(row.argmax())}"
    assert eng.alloc.num_free == eng.alloc.num_blocks


@pytest.mark.gpu
def test_decode_graphs_match_eager():
    """The captured decode step replayed over several steps (with eager work between the replays) gives the eager
    step's logits."""
    m = Model(HYBRID, "cuda", torch.bfloat16)
    t = toks(60, seed=27)
    eager = m.run_cut("e", t, [20, 1])
    m.runner.use_graphs = True
    m.runner.capture()
    assert m.runner.graphs
    graphed = m.run_cut("g", t, [20, 1])
    assert torch.allclose(eager, graphed, atol=1e-5, rtol=1e-5)
    m.check(graphed, m.expect(t), "graph replays")


def test_config_round_trip_and_registry(tmp_path):
    cfg = DironexConfig.from_dict(HYBRID)
    again = DironexConfig.from_dict(cfg.to_dict())
    assert again.layers == cfg.layers and again == cfg
    assert [r.layer for r in cfg.runs()] == [0, 1, 2, 1, 2, 3]
    bare = DironexConfig.from_dict(config([att()], streams=0, taps=0))
    assert bare.num_streams == 1 and bare.canon_taps == 0 and DironexConfig.from_dict(bare.to_dict()) == bare
    from safetensors.torch import save_file

    (tmp_path / "config.json").write_text(json.dumps(HYBRID))
    weights = init_weights(cfg, seed=3)
    save_file({k: v.contiguous() for k, v in weights.items()}, str(tmp_path / "model.safetensors"))
    fam, cfg2, path = registry.resolve(str(tmp_path))
    assert fam.name == "dironex" and cfg2.layers == cfg.layers and cfg2.width == cfg.width and path == str(tmp_path)
    w = registry.load_weights(fam, cfg2, path, device="cpu", dtype=torch.float32)
    assert w.layers[1].mlp.up.shape == (6, 9, 26) and w.layers[0].hc1.mix.shape == (2, 2) and w.head.dtype == torch.float32
    assert set(tensor_shapes(cfg)) == set(weights)
    assert registry.resolve("dironex-tiny")[0].name == "dironex"
    assert cfg.cache_bytes_per_token() > 0 and cfg.state_bytes_per_sequence() > 0
    bad = dict(weights)
    bad["l0.mix.uq"] = bad["l0.mix.uq"][:-1]
    with pytest.raises(ValueError):
        convert_dironex(cfg, bad)
    with pytest.raises(ValueError):
        DironexConfig.from_dict(config([att(mlp=moe(experts=6, top=5, groups=3, keep=2))]))


def test_serving_builds_the_family_by_name():
    """The serving launcher's engine builder resolves the family through the registry and generates with it."""
    from distributed_sse_for_llm_response_amd.serving.app import build_engine
    from distributed_sse_for_llm_response_amd.serving.config import ServeConfig

    eng, _ = build_engine(ServeConfig(model="dironex-tiny", engine="cpu"))
    eng.add_request("c1", [5, 6, 7, 8, 9, 10], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
    eng.add_request("c2", [11, 12], SamplingParams(temperature=0.8, max_tokens=3, ignore_eos=True))
    ev = eng.run_until_idle()
    assert sum(1 for e in ev if e.conversation_id == "c1" and not e.done) == 4
    assert sum(1 for e in ev if e.conversation_id == "c2" and not e.done) == 3
