"""HIP kernels of the bracketing-norm mechanisms against their plain PyTorch references (ops/layers_reference.py), op by
op: the pair embedding's rows, the add + norm rows, the token gate, capped scores and turned-back outputs in the
attention kernels (row form, MFMA form, key split), softmax routing with group maxima, the sigmoid head gate, decay
parameters that serve runs of columns, the per-head norm without a gain, and the delta rule under a per-channel decay."""
import math

import pytest
import torch

from distributed_sse_for_llm_response_amd import ops
from distributed_sse_for_llm_response_amd.models.surodra import HalfRotarySpec
from distributed_sse_for_llm_response_amd.ops import layers_reference as lref

pytestmark = pytest.mark.gpu

PAGE = 32


def dev():
    return torch.device("cuda")


def i32(x):
    return torch.tensor(x, dtype=torch.int32)


def c(t):
    return None if t is None else t.to(dev())


def close(a, b, tol):
    a, b = a.float().cpu(), b.float().cpu()
    err = (a - b).abs().max().item()
    ref = b.abs().max().item() + 1e-6
    assert err <= tol * ref, f"max abs err {err} vs scale {ref}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [1, 333, 1024])
def test_embed_pair_rows(dtype, W):
    g = torch.Generator().manual_seed(0)
    M, V, n = 9, 50, 23
    embed, pair = torch.randn(V, W, generator=g).to(dtype), torch.randn(n + 1, W, generator=g).to(dtype)
    ids = i32([3, 49, 0, 7, 7, 12, 100, 5, 6])  # one id out of range: row 0 of the table
    prev = i32([-1, 3, 49, 0, 7, 7, 12, 44, 5])
    pos = i32([0, 1, 2, 3, 0, 5, 6, 7, 0])
    keep = i32([1, 0, 1, 1])
    for with_pair in (True, False):
        wide_ref = torch.zeros(M, 2 * W + 3, dtype=dtype)
        r_ref, p_ref = torch.zeros(M, W), prev.clone()
        lref.embed_pair_rows(ids, prev, pos, embed, pair if with_pair else None, 2 ** 20 + 7, 31, n, r_ref,
                             wide_ref[:, W:2 * W], p_ref[:4], keep)
        wide = torch.zeros(M, 2 * W + 3, dtype=dtype, device=dev())
        r, p = torch.zeros(M, W, device=dev()), c(prev.clone())
        ops.embed_pair_rows(c(ids), p, c(pos), c(embed), c(pair) if with_pair else None, 2 ** 20 + 7, 31, n, r,
                            wide[:, W:2 * W], p[:4], c(keep))   # prev_out is prev itself, as in a decode step
        close(r, r_ref, 1e-6)
        assert torch.equal(wide.cpu(), wide_ref) and torch.equal(p.cpu(), p_ref)
    assert p_ref.tolist()[:4] == [3, 3, 0, 7]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,nsum", [(1, 1), (19, 3), (256, 2), (2052, 1), (4096, 2), (9000, 1), (16388, 2)])
def test_add_norm_rows(dtype, W, nsum):
    """Widths on the register path with and without 16-byte accesses and on the path that reads the row again."""
    g = torch.Generator().manual_seed(1)
    M = 5
    y, resid = torch.randn(M * nsum, W, generator=g), torch.randn(M, W, generator=g)
    ga, go = torch.randn(W, generator=g), torch.randn(W, generator=g)
    for use_y, use_go, use_out, use_32, strided in ((1, 1, 1, 1, 0), (1, 0, 1, 0, 1), (0, 1, 1, 0, 0), (1, 1, 0, 0, 0),
                                                    (0, 0, 1, 1, 1), (1, 1, 1, 0, 1)):
        r_ref = resid.clone()
        wide_ref, o32_ref = torch.zeros(M, 2 * W + 8, dtype=dtype), torch.zeros(M, W)
        out_ref = wide_ref[:, :W] if strided else torch.zeros(M, W, dtype=dtype)
        lref.add_norm_rows(y if use_y else None, nsum, ga if use_y else None, r_ref, go if use_go else None, 1e-5,
                           out_ref if use_out else None, o32_ref if use_32 else None)
        r = c(resid.clone())
        wide, o32 = torch.zeros(M, 2 * W + 8, dtype=dtype, device=dev()), torch.zeros(M, W, device=dev())
        out = wide[:, :W] if strided else torch.zeros(M, W, dtype=dtype, device=dev())
        ops.add_norm_rows(c(y) if use_y else None, nsum, c(ga) if use_y else None, r, c(go) if use_go else None, 1e-5,
                          out if use_out else None, o32 if use_32 else None)
        close(r, r_ref, 2e-6)
        if use_out:
            close(out, out_ref, 1e-5 if dtype == torch.float32 else 1e-2)
            assert float(wide[:, W:].abs().max()) == 0.0
        if use_32:
            close(o32, o32_ref, 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_gate_rows(dtype):
    g = torch.Generator().manual_seed(2)
    M, F, V = 11, 24, 40
    wide = torch.randn(M, F + 5, generator=g) * 2
    table = torch.randn(V, 3 * F + 1, generator=g).to(dtype)
    ids = i32(torch.randint(0, V, (M,), generator=g).tolist())
    ref = torch.zeros(M, F, dtype=dtype)
    lref.token_gate_rows(wide[:, 2:2 + F], ids, table, F + 1, ref)
    out = torch.zeros(M, F, dtype=dtype, device=dev())
    ops.token_gate_rows(c(wide)[:, 2:2 + F], c(ids), c(table), F + 1, out)
    close(out, ref, 1e-6 if dtype == torch.float32 else 1e-2)


def _pages(n_seq, lens, g):
    need = [math.ceil(n / PAGE) for n in lens]
    perm = torch.randperm(sum(need) + 3, generator=g).tolist()
    bt = torch.zeros(n_seq, max(need) + 1, dtype=torch.int32)
    k = 0
    for s, n in enumerate(need):
        bt[s, :n] = torch.tensor(perm[k:k + n], dtype=torch.int32)
        k += n
    return bt, sum(need) + 3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V,window", [(4, 2, 64, 64, 10 ** 9), (6, 1, 40, 24, 37), (3, 3, 128, 130, 10 ** 9),
                                            (2, 1, 16, 2, 5)])
def test_attention_row_form_with_cap_and_output_rotation(dtype, H, G, D, V, window):
    g = torch.Generator().manual_seed(4)
    ctx, ql = [300, 1, 70, 33], [40, 1, 70, 1]        # a late portion, a first token, a whole prompt, a decode row
    bt, pages = _pages(4, ctx, g)
    T = sum(ql)
    q = torch.randn(T, H, D, generator=g)
    kc = torch.randn(pages, PAGE, G, D, generator=g).to(dtype)
    vc = torch.randn(pages, PAGE, G, V, generator=g).to(dtype)
    gate = torch.randn(T, H + 2, generator=g)
    rope = HalfRotarySpec(dims=V, base=50.0).table(310)
    qs = i32([0, 40, 41, 111])
    qt = 4
    ws = [s for s, n in enumerate(ql) for _ in range(math.ceil(n / qt))]
    wt = [t for n in ql for t in range(math.ceil(n / qt))]
    for cap, turn in ((3.0, True), (0.0, True), (2.0, False)):
        o_ref = torch.zeros(T, H, V, dtype=dtype)
        lref.sink_attention(q, kc, vc, bt, qs, i32(ql), i32(ctx), None, gate[:, 1:1 + H], o_ref, window, 0.5, None, cap,
                            rope if turn else None)
        o = torch.zeros(T, H, V, dtype=dtype, device=dev())
        ops.sink_attention(c(q), c(kc), c(vc), c(bt), c(qs), c(i32(ql)), c(i32(ctx)), c(i32(ws)), c(i32(wt)), None,
                           c(gate)[:, 1:1 + H], o, window, 0.5, qt, None, False, cap, c(rope) if turn else None)
        close(o, o_ref, 1e-5 if dtype == torch.float32 else 1e-2)
    plain = torch.zeros(T, H, V, dtype=dtype)
    lref.sink_attention(q, kc, vc, bt, qs, i32(ql), i32(ctx), None, gate[:, 1:1 + H], plain, window, 0.5)
    assert float((plain.float() - o_ref.float()).abs().max()) > 1e-2, "the cap changes nothing at these scores"


@pytest.mark.parametrize("H,G,D,V,window", [(4, 2, 64, 64, 10 ** 9), (6, 1, 32, 32, 37), (5, 5, 128, 96, 10 ** 9),
                                            (8, 2, 96, 320, 100)])
def test_attention_mfma_form_with_cap_and_output_rotation(H, G, D, V, window):
    """Prompt tiles and the key split of the MFMA form against the reference (which reads the same transposed pages)."""
    g = torch.Generator().manual_seed(8)
    ctx, ql = [300, 1, 70, 45], [40, 1, 70, 2]
    bt, pages = _pages(4, ctx, g)
    T = sum(ql)
    q = torch.randn(T, H, D, generator=g)
    kc = torch.randn(pages, PAGE, G, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(pages, PAGE, G, V, generator=g).to(torch.bfloat16)
    off = torch.arange(PAGE)
    vt = torch.zeros(pages, G, V, PAGE, dtype=torch.bfloat16)
    vt[:, :, :, lref.vt_position(off)] = vc.permute(0, 2, 3, 1)
    gate = torch.randn(T, H, generator=g)
    rope = HalfRotarySpec(dims=V, base=50.0).table(310)
    qs = i32([0, 40, 41, 111])
    hs = [s for s, n in enumerate(ql) for _ in range(math.ceil(n / 16))]
    ht = [t for n in ql for t in range(math.ceil(n / 16))]
    for cap, turn in ((3.0, True), (0.0, True), (2.0, False)):
        o_ref = torch.zeros(T, H, V, dtype=torch.bfloat16)
        lref.sink_attention(q, kc, torch.zeros_like(vc), bt, qs, i32(ql), i32(ctx), None, gate, o_ref, window, 0.2, vt, cap,
                            rope if turn else None)
        o = torch.zeros(T, H, V, dtype=torch.bfloat16, device=dev())
        ops.sink_attention(c(q), c(kc), c(vc), c(bt), c(qs), c(i32(ql)), c(i32(ctx)), c(i32(hs)), c(i32(ht)), None, c(gate),
                           o, window, 0.2, 16, c(vt), False, cap, c(rope) if turn else None)
        close(o, o_ref, 2e-2)
        if V <= 128:
            o2 = torch.zeros_like(o)
            ops.sink_attention(c(q), c(kc), c(vc), c(bt), c(qs), c(i32(ql)), c(i32(ctx)), c(i32(hs)), c(i32(ht)), None,
                               c(gate), o2, window, 0.2, 16, c(vt), True, cap, c(rope) if turn else None)
            close(o2, o_ref, 2e-2)


def test_value_pages_normed_and_rotated():
    """Values into their pages: RMS norm per head without a gain, rotated over the whole width, also transposed."""
    g = torch.Generator().manual_seed(9)
    T, G, V = 40, 2, 48
    x = torch.randn(T, G, V, generator=g)
    pos = i32(torch.randint(0, 200, (T,), generator=g).tolist())
    rows = torch.randperm(3 * PAGE, generator=g)[:T].to(torch.int32)
    rows[5] = -1
    rope = HalfRotarySpec(dims=V, base=100.0).table(200)
    ref, ref_t = torch.zeros(3, PAGE, G, V), torch.zeros(3, G, V, PAGE)
    lref.norm_rope_rows(x, None, pos, rope, ref, rows, 3, 1e-5, 1.0, ref_t)
    out, out_t = c(torch.zeros_like(ref)), c(torch.zeros_like(ref_t))
    ops.norm_rope_rows(c(x), None, c(pos), c(rope), out, c(rows), 3, 1e-5, 1.0, out_t)
    close(out, ref, 1e-6)
    close(out_t, ref_t, 1e-6)
    want = x[0] / x[0].pow(2).mean(-1, keepdim=True).add(1e-5).sqrt()
    assert torch.allclose(ref.view(-1, G, V)[int(rows[0])].pow(2).sum(-1), want.pow(2).sum(-1), atol=1e-4)


def test_gate_math_with_parameters_per_run_of_columns():
    g = torch.Generator().manual_seed(10)
    M, H, D = 9, 5, 12
    wide = torch.randn(M, H * D + 6, generator=g)
    a_log, dt = torch.randn(H, generator=g), torch.randn(H * D, generator=g)
    ref = wide.clone()
    lref.gate_math(ref[:, 3:3 + H * D], 0, a_log, dt, 1.0)
    want = torch.exp(-torch.exp(a_log)[None, :, None] * torch.nn.functional.softplus(wide[:, 3:3 + H * D].view(M, H, D) + dt.view(H, D)))
    assert torch.allclose(ref[:, 3:3 + H * D].view(M, H, D), want, atol=1e-6)
    x = c(wide.clone())
    ops.gate_math(x[:, 3:3 + H * D], 0, c(a_log), c(dt))
    close(x, ref, 1e-6)
    with pytest.raises(RuntimeError):
        ops.gate_math(x[:, 3:3 + H * D], 0, c(torch.randn(7)), c(dt))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_norm_with_sigmoid_gate(dtype):
    g = torch.Generator().manual_seed(11)
    M, H, V = 7, 3, 40
    o, w = torch.randn(M, H, V, generator=g), torch.randn(V, generator=g)
    wide = torch.randn(M, H * V + 4, generator=g) * 2
    for kind in (0, 1):
        ref = torch.zeros(M, H * V, dtype=dtype)
        lref.gated_head_norm(o, w, wide[:, 1:1 + H * V], 1e-5, ref, kind)
        out = torch.zeros(M, H * V, dtype=dtype, device=dev())
        ops.gated_head_norm(c(o), c(w), c(wide)[:, 1:1 + H * V], 1e-5, out, kind)
        close(out, ref, 1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("E,top,groups,keep", [(1, 1, 1, 1), (16, 4, 4, 3), (12, 3, 4, 2), (10, 2, 1, 1), (8, 8, 8, 8),
                                               (256, 8, 8, 4), (96, 5, 32, 2)])
def test_softmax_routing(E, top, groups, keep):
    g = torch.Generator().manual_seed(12)
    M = 50
    z = torch.randn(M, E, generator=g) * 3
    ri, rw = torch.zeros(M, top, dtype=torch.int32), torch.zeros(M, top)
    lref.moe_route(z, None, ri, rw, groups, keep, 1.0, 1)
    ti, tw = torch.zeros(M, top, dtype=torch.int32, device=dev()), torch.zeros(M, top, device=dev())
    ops.moe_route(c(z), None, ti, tw, groups, keep, 1.0, 1)
    assert torch.equal(ti.cpu(), ri)
    close(tw, rw, 1e-5)
    s = torch.softmax(z, -1)
    assert torch.allclose(rw, s.gather(1, ri.long()), atol=1e-6)


@pytest.mark.parametrize("H,G,D,V", [(4, 2, 32, 32), (6, 6, 64, 64), (3, 1, 128, 64), (2, 1, 8, 5)])
def test_delta_rule_under_a_per_channel_decay(H, G, D, V):
    """The recurrence with the delta rule AND one decay per (token, head, key channel): prompt portions (the wave-local
    kernel) and decode rows (the state-traffic kernel), continued from slot states."""
    from distributed_sse_for_llm_response_amd.ops.layers import scan_state_from_plain, scan_state_plain

    g = torch.Generator().manual_seed(13)
    for ql, ctx, slot in (([37, 1, 0, 5], [37, 9, 4, 25], [2, 0, 3, 1]), ([1, 1, 0, 1], [9, 1, 4, 300], [3, 0, 2, 1])):
        T = sum(ql) + 1
        qs = i32([0, ql[0], ql[0] + ql[1], ql[0] + ql[1] + ql[2]])
        q = torch.randn(T, G, D, generator=g) * 0.3
        k = torch.randn(T, G, D, generator=g)
        k = k / k.norm(dim=-1, keepdim=True)
        v = torch.randn(T, H, V, generator=g)
        decay = torch.rand(T, H, D, generator=g) * 0.5 + 0.5
        beta = torch.rand(T, H, generator=g)
        state0 = torch.randn(4, H, D, V, generator=g)
        st_ref, o_ref = state0.clone(), torch.zeros(T, H, V)
        lref.matrix_scan(q, k, v, decay, beta, st_ref, qs, i32(ql), i32(ctx), i32(slot), o_ref, 1.0)
        st, o = scan_state_from_plain(c(state0.clone())), torch.zeros(T, H, V, device=dev())
        ops.matrix_scan(c(q), c(k), c(v), c(decay), c(beta), st, c(qs), c(i32(ql)), c(i32(ctx)), c(i32(slot)), o, 1.0)
        close(o, o_ref, 2e-5)
        close(scan_state_plain(st), st_ref, 2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,F,nsum", [(1, 1, 1), (19, 3, 2), (256, 24, 1), (2048, 64, 3), (1000, 20, 1)])
def test_token_side_rows(dtype, W, F, nsum):
    """The one-launch token input against its reference: with and without a pending add, a following norm, a strided
    output and the unrounded copy."""
    g = torch.Generator().manual_seed(14)
    M, V = 6, 30
    y, resid = torch.randn(M * nsum, W, generator=g), torch.randn(M, W, generator=g)
    ga, go, sn = (torch.randn(W, generator=g) for _ in range(3))
    gate_w = (torch.randn(F, W, generator=g) / math.sqrt(W)).to(dtype)
    proj_w = (torch.randn(W, F, generator=g) / math.sqrt(F)).to(dtype)
    table = torch.randn(V, 2 * F + 3, generator=g).to(dtype)
    ids = i32(torch.randint(0, V, (M,), generator=g).tolist())
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for use_y, use_go, use_out, use_32 in ((1, 1, 1, 1), (0, 0, 1, 0), (1, 0, 0, 0), (1, 1, 1, 0)):
        r_ref = resid.clone()
        wide_ref, o32_ref = torch.zeros(M, 2 * W + 8, dtype=dtype), torch.zeros(M, W)
        lref.token_side_rows(y if use_y else None, nsum, ga if use_y else None, r_ref, ids, table, F + 1, gate_w, proj_w, sn,
                             go if use_go else None, 1e-5, wide_ref[:, :W] if use_out else None, o32_ref if use_32 else None)
        r = c(resid.clone())
        wide, o32 = torch.zeros(M, 2 * W + 8, dtype=dtype, device=dev()), torch.zeros(M, W, device=dev())
        ops.token_side_rows(c(y) if use_y else None, nsum, c(ga) if use_y else None, r, c(ids), c(table), F + 1, c(gate_w),
                            c(proj_w), c(sn), c(go) if use_go else None, 1e-5, wide[:, :W] if use_out else None,
                            o32 if use_32 else None)
        close(r, r_ref, tol)
        if use_out:
            close(wide, wide_ref, tol)
        if use_32:
            close(o32, o32_ref, tol)
    assert ops.token_side_fits(64, 8192, 256) and not ops.token_side_fits(65, 64, 8) and not ops.token_side_fits(4, 16384, 64)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1000, 16, 2048), (333, 64, 300), (40, 5, 256), (17, 1, 4100)])
def test_many_rows_of_a_narrow_output(dtype, M, N, K):
    """A router's logits or a few-column gate for a prompt: 16 x 16 output tiles with the K axis split over the waves."""
    g = torch.Generator().manual_seed(15)
    x = torch.randn(M, K + 3, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    ref = x[:, :K].float() @ w.float().t()
    out = torch.zeros(M, N, device=dev())
    ops.gemm_rm(c(x)[:, :K], c(w), out)
    close(out, ref, 1e-5 if dtype == torch.float32 else 1e-2)
