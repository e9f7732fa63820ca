"""HIP kernels of the multi-stream / routed squared-ReLU mechanisms against their plain PyTorch references
(ops/layers_reference.py), op by op, on shapes that hit the kernels' edges: widths that are no multiple of the
workgroup, one to eight streams, strided column views, experts per tile from none to hundreds of rows, groups of one."""
import pytest
import torch

from distributed_sse_for_llm_response_amd import ops
from distributed_sse_for_llm_response_amd.ops import layers_reference as lref

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda")


def i32(x):
    return torch.tensor(x, dtype=torch.int32)


def close(a, b, tol):
    a, b = a.float().cpu(), b.float().cpu()
    err = (a - b).abs().max().item()
    ref = b.abs().max().item() + 1e-6
    assert err <= tol * ref, f"max abs err {err} vs scale {ref}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,W,nsum", [(1, 5, 1), (2, 333, 3), (3, 256, 1), (5, 1030, 2), (8, 64, 4)])
def test_stream_mix(dtype, S, W, nsum):
    g = torch.Generator().manual_seed(S * W)
    M, V = 6, 40
    streams = torch.randn(M, S, W, generator=g)
    y = torch.randn(M * nsum, W, generator=g)
    embed = torch.randn(V, W, generator=g).to(dtype)
    ids = i32([3, 39, 0, 7, 7, 100])  # the last id is out of range: row 0 of the table
    inw, outw, mix = torch.randn(S, generator=g), torch.randn(S, generator=g), torch.randn(S, S, generator=g)
    nw = torch.randn(W, generator=g)
    c = lambda t: None if t is None else t.to(dev())  # noqa: E731
    # (y, embed, norm, h in fp32, total)
    for use in ((1, 0, 1, 0, 0), (0, 1, 1, 1, 0), (1, 0, 0, 0, 1), (0, 0, 1, 0, 1), (1, 1, 1, 1, 1), (1, 0, 1, 1, 0)):
        hdt = torch.float32 if use[3] else dtype
        s_ref, h_ref, t_ref = streams.clone(), torch.zeros(M, W, dtype=hdt), torch.zeros(M, W)
        args = (y if use[0] else None, nsum, 0.6, None, ids if use[1] else None, embed if use[1] else None, 1.7,
                outw if use[0] else None, mix if use[0] else None, inw if use[2] else None, nw if use[2] else None, 1e-5)
        lref.stream_mix(*args[:3], s_ref, *args[4:], h_ref if use[2] else None, t_ref if use[4] else None)
        s_gpu, h_gpu, t_gpu = c(streams.clone()), torch.zeros(M, W, dtype=hdt, device=dev()), torch.zeros(M, W, device=dev())
        ops.stream_mix(c(args[0]), nsum, 0.6, s_gpu, c(args[4]), c(args[5]), 1.7, c(args[7]), c(args[8]), c(args[9]),
                       c(args[10]), 1e-5, h_gpu if use[2] else None, t_gpu if use[4] else None)
        close(s_gpu, s_ref, 1e-5)
        if use[2]:
            close(h_gpu, h_ref, 1e-5 if hdt == torch.float32 else 1e-2)
        if use[4]:
            close(t_gpu, t_ref, 1e-5)


def test_stream_mix_reads_a_column_slice():
    """One stream with weight 1 read in place from a wider buffer: the RMS norm of a fused projection's column range."""
    g = torch.Generator().manual_seed(3)
    wide = torch.randn(9, 700, generator=g)
    nw, one = torch.randn(520, generator=g), torch.ones(1)
    ref = torch.zeros(9, 520, dtype=torch.bfloat16)
    lref.stream_mix(None, 1, 0.0, wide[:, 100:620].unsqueeze(1), None, None, 1.0, None, None, one, nw, 1e-6, ref, None)
    out = torch.zeros(9, 520, dtype=torch.bfloat16, device=dev())
    wg = wide.to(dev())
    ops.stream_mix(None, 1, 0.0, wg[:, 100:620].unsqueeze(1), in_w=one.to(dev()), norm_w=nw.to(dev()), eps=1e-6, h=out)
    close(out, ref, 1e-2)
    assert torch.equal(wg.cpu(), wide)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", [0, 1, 2])
def test_act_rows(dtype, kind):
    g = torch.Generator().manual_seed(kind)
    M, F = 7, 77
    wide = torch.randn(M, F + 9, generator=g) * 3
    gates = torch.randn(M, 2 * F, generator=g)
    params = torch.tensor([0.8, 1.3])
    for gate in (None, gates[:, 5:5 + F]):
        ref = torch.zeros(M, F, dtype=dtype)
        lref.act_rows(wide[:, 4:4 + F], ref, kind, params, gate)
        out = torch.zeros(M, F, dtype=dtype, device=dev())
        gg = None if gate is None else gates.to(dev())[:, 5:5 + F]
        ops.act_rows(wide.to(dev())[:, 4:4 + F], out, kind, params.to(dev()), gg)
        close(out, ref, 1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("E,top,groups,keep", [(12, 3, 4, 2), (8, 2, 8, 3), (6, 6, 1, 1), (256, 8, 8, 4), (5, 1, 1, 1),
                                               (16, 4, 4, 1), (1, 1, 1, 1)])
def test_moe_route(E, top, groups, keep):
    g = torch.Generator().manual_seed(E + top)
    M = 300
    z = torch.randn(M, E, generator=g) * 2
    z[0, 0] = float("nan")
    corr = torch.randn(E, generator=g) * 0.5
    ri, rw = torch.zeros(M, top, dtype=torch.int32), torch.zeros(M, top)
    lref.moe_route(z, corr, ri, rw, groups, keep, 1.9)
    gi, gw = torch.zeros(M, top, dtype=torch.int32, device=dev()), torch.zeros(M, top, device=dev())
    ops.moe_route(z.to(dev()), corr.to(dev()), gi, gw, groups, keep, 1.9)
    assert torch.equal(gi.cpu(), ri)
    close(gw, rw, 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,W,F,E,top", [(1, 64, 32, 4, 2), (5, 100, 36, 7, 3), (70, 128, 64, 8, 2), (400, 192, 72, 6, 4),
                                         (700, 256, 136, 3, 1)])
def test_grouped_experts_without_a_gate(dtype, M, W, F, E, top):
    """down(relu(up x)^2) per (row, slot): the register-direct kernels (few rows, fp32) and the LDS-staged tiles (bf16,
    hundreds of rows), experts that get no row included."""
    g = torch.Generator().manual_seed(M + F)
    x = torch.randn(M, W, generator=g).to(dtype)
    up = (torch.randn(E, F, W, generator=g) / W ** 0.5).to(dtype)
    down = (torch.randn(E, W, F, generator=g) / F ** 0.5).to(dtype)
    tki = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(M)]).to(torch.int32)
    if E > 2:
        tki[tki == E - 1] = 0  # the last expert gets nothing (a row may then name expert 0 twice: two slots, same expert)
    tkw = torch.rand(M, top, generator=g)
    ref = torch.zeros(M * top, W)
    lref.moe_grouped(x, tki, tkw, None, up, down, None, None, None, ref)
    tiles = -(-M * top // 64) + E + 2
    o = torch.zeros(M * top, W, device=dev())
    c = lambda t: t.to(dev())  # noqa: E731
    ops.moe_grouped(c(x), c(tki), c(tkw), None, c(up), c(down), None, None, None,
                    torch.zeros(tiles * 64, dtype=torch.int32, device=dev()),
                    torch.zeros(tiles, dtype=torch.int32, device=dev()), torch.zeros(1, dtype=torch.int32, device=dev()),
                    torch.zeros(M * top, -(-F // 8) * 8, dtype=dtype, device=dev()), o)
    close(o, ref, 1e-4 if dtype == torch.float32 else 3e-2)


def test_norm_rows_per_head_gain():
    g = torch.Generator().manual_seed(9)
    T, H, D = 11, 5, 72
    wide = torch.randn(T, H * D + 13, generator=g)
    x = wide[:, 6:6 + H * D].unflatten(1, (H, D))
    nw = torch.randn(D, generator=g)
    pos = torch.zeros(T, dtype=torch.int32)
    ref = torch.zeros(T, H, D)
    lref.norm_rope_rows(x, nw, pos, None, ref, None, 3, 1e-5, 1.0)
    out = torch.zeros(T, H, D, device=dev())
    ops.norm_rope_rows(wide.to(dev())[:, 6:6 + H * D].unflatten(1, (H, D)), nw.to(dev()), pos.to(dev()), None, out, None, 3,
                       1e-5, 1.0)
    close(out, ref, 1e-5)
    one = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * nw
    close(ref, one, 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_plus_input(dtype):
    """out = in + conv(in) continued from the slot tails, sequences that start here and sequences that go on."""
    g = torch.Generator().manual_seed(4)
    C, K, slots = 70, 4, 3
    qs, ql, ctx, ss = i32([0, 5, 6]), i32([5, 1, 9]), i32([5, 8, 20]), i32([2, 0, 1])
    inp = torch.randn(15, C, generator=g)
    taps = torch.randn(C, K, generator=g).to(dtype)
    tail = torch.randn(slots, K - 1, C, generator=g)
    t_ref, o_ref, b_ref = tail.clone(), torch.zeros(15, C), torch.zeros(15, C, dtype=dtype)
    lref.conv_state(inp, taps, None, t_ref, qs, ql, ctx, ss, o_ref, b_ref, None, 2)
    c = lambda t: t.to(dev())  # noqa: E731
    t_gpu, o_gpu, b_gpu = c(tail.clone()), torch.zeros(15, C, device=dev()), torch.zeros(15, C, dtype=dtype, device=dev())
    ops.conv_state(c(inp), c(taps), None, t_gpu, c(qs), c(ql), c(ctx), c(ss), o_gpu, b_gpu, None, 2)
    close(o_gpu, o_ref, 1e-5)
    close(b_gpu, b_ref, 1e-5 if dtype == torch.float32 else 1e-2)
    close(t_gpu, t_ref, 1e-6)
    plain = torch.zeros(15, C)
    lref.conv_state(inp, taps, None, tail.clone(), qs, ql, ctx, ss, plain, None, None, 0)
    close(o_ref, plain + inp, 1e-6)


def test_latent_cache_write_from_a_column_slice():
    g = torch.Generator().manual_seed(6)
    T, rk, dr, pages = 9, 24, 8, 2
    wide = torch.randn(T, 50, generator=g)
    nw = torch.randn(rk, generator=g)
    pos = torch.arange(T, dtype=torch.int32)
    slots = i32([0, 1, 2, 40, 41, -1, 63, 5, 6])
    ang = torch.arange(16, dtype=torch.float32)[:, None] * torch.tensor([1.0, 0.3, 0.1, 0.03])[None, :]
    rope = torch.stack([ang.cos(), ang.sin()], dim=-1)
    ref = torch.zeros(pages, 32, rk + dr)
    lref.latent_kv_write(wide[:, 7:7 + rk + dr], nw, pos, slots, rope, ref, 1e-5)
    out = torch.zeros(pages, 32, rk + dr, device=dev())
    ops.latent_kv_write(wide.to(dev())[:, 7:7 + rk + dr], nw.to(dev()), pos.to(dev()), slots.to(dev()), rope.to(dev()), out,
                        1e-5)
    close(out, ref, 1e-5)
