"""Forward passes of configuration-driven designs (models/muderax.py, models/surodra.py, models/dironex.py,
models/murulorn.py) on the layer-mechanism kernels (ops/layers.py).  Four block styles share the runner: sandwich
norms on a sublayer's output (Muderax, described first), pre-norm blocks around matrix-state mixers (Surodra,
described after it), pre-norm blocks on several residual streams (Dironex) and blocks with a norm before and after
each sublayer plus a per-layer token input (Murulorn, described last).

A step is a set of packed rows -- the B decode slots first (one row each, state on the device as in ModelRunner), then
the rows of prompt portions -- that walk the layer list once:

    embed_rows              stream (fp32) = embedding; xb = its rounding (what the projections read)
    latent_attention layer  q and down-projection GEMMs -> latent_kv_write (norm + rotation + paged cache row) -> per-head
                            fold of the unrotated query through the key up-projection -> latent_attention over the
                            window (decode slots: one-row items; portions: tiled items) -> per-head value up-projection
                            -> output GEMM (fp32)
    rglru layer             gelu-branch and input GEMMs (fp32 out) -> conv_state (+ input bias; slot tail) -> block-
                            diagonal gate GEMM -> lru_scan (coefficients for all rows at once, then the walk over each
                            sequence's rows with the branch's bias + gelu; slot state) -> output GEMM (fp32)
    feed-forward            router GEMM (fp32 logits) -> moe_topk -> moe_grouped (rows sorted by expert, 16-row MFMA tiles; the shared expert is one
                            more slot of every row) -> per-slot outputs, summed inside the norm
    after each sublayer     scalar_norm: stream += out / rms(out) * g; xb = rounding
    head                    scalar_norm (final) on the rows that need logits -> GEMM (fp32 logits)

The pre-norm walk (`_prenorm_layers`) goes over layer RUNS -- a looped span of layers runs several times with the
same weights and its own pages and state slots per pass:

    stream_step             resid += m * (finished sublayer) (+ embedding again + the pass's vector at a pass's start);
                            xb = tanh(alpha resid) w + b -- the add, the pass additions and the next norm in one kernel
    delta layer             ONE fused GEMM [q | k | v | g | a | b] (fp32 out) -> conv_state over q | k | v (SiLU; slot
                            tail) -> unit q, k per head -> gate_math (decay, write strength) -> matrix_scan (delta rule;
                            slot state) -> gated_head_norm -> output GEMM
    parallel layer          ONE fused GEMM for both halves -> left: norm_rope_rows (whole-row RMS norm + rotation: q to
                            a buffer, k and v into this run's pages) -> sink_attention (MFMA form over transposed value
                            pages for prompt portions and decode rows, row form otherwise) -> output GEMM; right: decay
                            GEMM (fp32) -> gate_math -> matrix_scan (per-channel decay) -> gated_head_norm -> output
                            GEMM; rms_mix of the two
    retention layer         fused GEMM -> rotation of q, k -> matrix_scan (fixed decay) -> gated_head_norm -> output GEMM
    feed-forward            fused [gate | up] GEMM -> gated_act (gelu) -> down GEMM
    head                    stream_step (last add + final norm) -> head GEMM -> logit_cap (scale, tanh cap)

Long prompt groups walk the recurrences without the delta rule in two levels (matrix_scan_chunked).

The multi-stream walk (`_stream_layers`) also goes over layer runs; a row carries S residual copies:

    stream_mix              (first step) every stream = embedding * scale; x_t = sum_s mix[s][t] x_s + m out[t] y for the
                            finished sublayer; u = sum_s in[s] x_s; RMS norm with a gain per channel -- one kernel
    conv_state (act 2)      h + conv(h) over time per channel, continued from the slot's tail of normed rows (one launch
                            for decode rows, rows in parallel + a tail kernel for prompt portions)
    latent attention        ONE fused GEMM [dq | dkv | g] (fp32 out) -> stream_mix as the query latent's RMS norm -> query
                            up-projection -> latent_kv_write from the dkv columns -> per-head fold -> latent_attention
                            (causal, this run's latent pages) -> per-head value up-projection (fp32) -> act_rows (times
                            sigmoid(g)) -> output GEMM
    windowed attention      fused GEMM [q | k | v] -> norm_rope_rows kind 3 (RMS per head; k and v into this run's pages)
                            -> sink_attention without sink and gate over the window -> output GEMM
    feed-forward            up GEMM -> act_rows (xIELU) -> down GEMM; or router GEMM in fp32 on the fp32 row -> moe_route
                            (group-limited sigmoid routing) -> moe_grouped without a gate (squared ReLU), per-slot outputs
                            summed inside the next stream_mix
    head                    stream_mix (last write-back, sum of the streams) -> RMS norm -> head GEMM

The bracket-norm walk (`_bracket_layers`) also goes over layer runs:

    embed_pair_rows         stream = embed[token] + pair[hash(previous token, token)] (the table's last row at position
                            0); the embedding output once more, rounded, beside the stream's place in [stream | x0]
    add_norm_rows           between sublayers: stream += rms-norm(finished sublayer) * gain; xb = rms-norm(stream) * gain
                            of the next one (also fp32 for a router), or the rounded stream
    loop pass               stream <- W_in [stream | x0] (one GEMM on the rounded pair) before the pass's first layer
    attention layer         ONE fused GEMM [q | k | v | g] -> norm_rope_rows (whole-row RMS + rotation: q to a buffer, k
                            into the run's pages; v: RMS per head + rotation over its whole width into the pages) ->
                            sink_attention with capped scores, the head's sum turned back by the row's position, sigmoid
                            gate -> output GEMM
    channel-delta layer     ONE fused GEMM [q | k | v | b | a1 | g1] -> conv_state (SiLU; slot tail) -> unit q | k ->
                            block-diagonal fp32 GEMM [a2 0; 0 g2] -> gate_math (rate per head, bias per head and channel)
                            -> matrix_scan (delta rule, per-channel decay; slot state) -> gated_head_norm (sigmoid) ->
                            output GEMM
    feed-forward            up GEMM -> act_rows (squared ReLU) -> down GEMM; or router GEMM in fp32 on the fp32 row ->
                            moe_route (softmax scores, group maxima) -> moe_grouped without a gate
    token input             steps of up to 64 rows: token_side_rows, one launch that also writes the next sublayer's
                            input; larger steps: rounding, gate GEMM, token_gate_rows, back-projection GEMM
    head                    add_norm_rows (final norm) -> GEMM on the embedding table

A decode row's token becomes its slot's previous token inside embed_pair_rows (the captured graph carries it); prompt
portions bring each row's predecessor with them (PrefillSeq.prev_token for the first row).

The residual stream, norms, scores, router and recurrence are fp32 in both element types; ``dtype=torch.float32`` runs
the projections in true fp32 as well (the exact mode).  The cache is paged with the engine's block tables and
allocator (LatentKVCache, PagedKVCache, both at once in MixedKVCache); recurrent layers and input convolutions keep
their state in the sequence's decode slot (RecurrentStateCache, MatrixStateCache, ConvTailCache), so
slots and pages are handed from one sequence to the next with no clearing pass.  The decode step of each batch bucket
is captured into a graph like ModelRunner's; prompt portions and mixed steps run eagerly.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from .. import ops
from ..models.muderax import LRU_DECAY_SCALE
from ..models.surodra import UNIT_EPS, HalfRotarySpec
from ..parallel.comm import TPComm
from .kv_cache import (PAGE, ConvTailCache, LatentKVCache, MatrixStateCache, MixedKVCache, PagedKVCache,
                       RecurrentStateCache)
from .model_runner import RunnerBase, _capture, batch_buckets
from .weights import LayeredWeights

ATTN_ROWS_TILE = 4    # query rows per work item of the row-wise attention kernel (prompt portions)
FLASH_DECODE_WAVES = 512  # waves a decode attention launch aims for (two per CU)
SINK_ROWS_TILE = 16   # query rows per work item of the sink attention's MFMA form (one head per wave)
FLASH_ROWS_TILE = 4   # query rows per work item of the MFMA attention form, x 4 heads = 16 columns: a page of keys is
                      # read once for four heads (16 rows x 1 head re-read it per head: 2-3x the time at 16 heads)


class LayeredRunner(RunnerBase):
    def __init__(self, w: LayeredWeights, num_blocks: int, max_batch: int = 64, max_model_len: int = 4096,
                 max_prefill_tokens: int = 8192, device="cuda", comm: TPComm | None = None, use_graphs=None):
        self.w, self.cfg = w, w.cfg
        self.device = torch.device(device)
        self.comm = comm or TPComm()
        if self.comm.size != 1:
            raise ValueError(f"{self.cfg.name}: tensor parallelism is not implemented for this family")
        self.dtype = w.dtype
        self.max_batch = max_batch
        self.max_model_len = max_model_len
        self.max_blocks = math.ceil(max_model_len / PAGE) + 1
        self.max_prefill_tokens = max_prefill_tokens
        self.use_graphs = (self.device.type == "cuda") if use_graphs is None else use_graphs
        cfg, dev = self.cfg, self.device
        self._init_slots(max_batch, self.max_blocks, cfg.vocab_size, dev, self.comm)
        self.num_blocks = num_blocks
        self.prenorm = getattr(cfg, "family", "") == "surodra"   # pre-norm blocks with matrix-state mixers
        self.multistream = getattr(cfg, "family", "") == "dironex"  # pre-norm blocks on several residual streams
        self.bracket = getattr(cfg, "family", "") == "murulorn"    # a norm before and after each sublayer, token inputs
        if self.bracket:
            self._setup_bracket()
        elif self.multistream:
            self._setup_streams()
        elif self.prenorm:
            self._setup_prenorm()
        else:
            self._setup_sandwich()
        self._dec = self._buffers(max_batch)  # static decode activations (captured graphs read and write them)

    def _setup_sandwich(self) -> None:
        cfg, dev, max_batch = self.cfg, self.device, self.max_batch
        att = {i: L.mixer for i, L in enumerate(cfg.layers) if L.kind == "latent_attention"}
        rec = {i: L.mixer for i, L in enumerate(cfg.layers) if L.kind == "rglru"}
        flash = {i: m.kv_rank for i, m in att.items() if ops.latent_flash_ok(self.dtype, m.kv_rank, m.rot_dim)}
        self.kv = LatentKVCache({i: m.kv_rank + m.rot_dim for i, m in att.items()}, self.num_blocks, dev, self.dtype,
                                transposed=flash)
        self.state = RecurrentStateCache({i: (m.width, m.conv) for i, m in rec.items()}, max_batch, dev)
        # one rotation table per distinct (rotation, rotated width)
        self._rope = {}
        for m in att.values():
            key = (m.rot, m.rot_dim)
            if key not in self._rope:
                self._rope[key] = m.rot.table(self.max_model_len + 1, m.rot_dim, dev)
        words = max((ops.latent_flash_part_floats(max_batch, m.heads, 16, 16, m.kv_rank) for i, m in att.items()
                     if i in flash), default=0)
        self._flash_part = torch.zeros(max(1, words), device=dev, dtype=torch.float32)

    def _setup_prenorm(self) -> None:
        """Caches and state of a pre-norm design, keyed by layer RUN: a layer inside a looped span runs several times
        with the same weights and has its own pages and state slots each time."""
        cfg, dev = self.cfg, self.device
        self.runs = cfg.runs()
        kv, st, self._rope = {}, {}, {}
        for r in self.runs:
            L, m = cfg.layers[r.layer], cfg.layers[r.layer].mixer
            if L.kind == "delta":
                st[r.index] = ((m.heads, m.dim, m.vdim), 2 * m.kv_heads * m.dim + m.heads * m.vdim, m.conv)
            elif L.kind == "parallel":
                kv[r.index] = (m.left.kv_heads, m.left.dim, m.left.vdim)
                st[r.index] = ((m.right.heads, m.right.dim, m.right.vdim), 0, 1)
            else:
                st[r.index] = ((m.heads, m.dim, m.vdim), 0, 1)
            rot = m.left.rot if L.kind == "parallel" else getattr(m, "rot", None)
            if rot is not None and rot.dims > 0 and rot not in self._rope:
                self._rope[rot] = rot.table(self.max_model_len + 1, dev)
        flash = [r for r, (_, d, v) in kv.items() if ops.sink_flash_ok(self.dtype, d, v)]
        self.kv = PagedKVCache(kv, self.num_blocks, dev, self.dtype, transposed=flash)
        self.state = MatrixStateCache(st, self.max_batch, dev)

    # ------------------------------------------------------------------ buffers
    def _buffers(self, M: int) -> dict:
        cfg, dev = self.cfg, self.device
        f32 = dict(device=dev, dtype=torch.float32)
        el = dict(device=dev, dtype=self.dtype)
        W = cfg.width
        d = {"resid": torch.zeros(M, W, **f32), "xb": torch.zeros(M, W, **el), "y": torch.zeros(M, W, **f32)}
        if self.bracket:
            d.update(self._bracket_buffers(M))
            return d
        if self.multistream:
            d.update(self._stream_buffers(M))
            return d
        if self.prenorm:
            d.update(self._prenorm_buffers(M))
            return d
        att = [L.mixer for L in cfg.layers if L.kind == "latent_attention"]
        rec = [L.mixer for L in cfg.layers if L.kind == "rglru"]
        moe = [L.mlp for L in cfg.layers if L.mlp is not None]
        if att:
            d["q"] = torch.zeros(M * max(m.heads * (m.dim + m.rot_dim) for m in att), **el)
            d["ckr"] = torch.zeros(M * max(m.kv_rank + m.rot_dim for m in att), **f32)
            d["qabs"] = torch.zeros(M * max(m.heads * m.kv_rank for m in att), **f32)
            d["lat"] = torch.zeros(M * max(m.heads * m.kv_rank for m in att), **el)
            d["attn"] = torch.zeros(M * max(m.heads * m.vdim for m in att), **el)
        if rec:
            C = max(m.width for m in rec)
            d["ub"], d["hs"] = (torch.zeros(M * C, **el) for _ in range(2))
            d["yr"], d["ux"], d["u"] = (torch.zeros(M * C, **f32) for _ in range(3))
            d["gates"] = torch.zeros(M * 2 * C, **f32)
            # chunked walk of the recurrence over prompt portions: (A, B) per 32-row chunk
            d["scan"] = torch.zeros(2 * (M // 32 + max(M, self.max_batch) + 2) * C, **f32) if M >= 128 else None
        if moe:
            top = max(f.top for f in moe)
            d["tki"] = torch.zeros(M * top, device=dev, dtype=torch.int32)
            d["tkw"] = torch.zeros(M * top, **f32)
            # grouped experts: ids = (row, slot), slots = top (+ 1: the shared expert)
            slots = max(f.top + (1 if f.shared_ff else 0) for f in moe)
            tiles = -(-M * slots // 64) + max(f.experts for f in moe) + 2
            d["mo_z"] = torch.zeros(M * max(f.experts for f in moe), **f32)
            ldh = -(-max(max(f.ff, f.shared_ff) for f in moe) // 8) * 8
            d["mo_sorted"] = torch.zeros(tiles * 64, device=dev, dtype=torch.int32)
            d["mo_tile"] = torch.zeros(tiles, device=dev, dtype=torch.int32)
            d["mo_n"] = torch.zeros(1, device=dev, dtype=torch.int32)
            d["mo_h"] = torch.zeros(M * slots, ldh, **el)
            d["mo_o"] = torch.zeros(M * slots * W, **f32)
        return d

    # ------------------------------------------------------------------ layers
    @staticmethod
    def _lin(x, w, wt, out) -> None:
        """out = x · Wᵀ: the engine's tiled-layout GEMMs when the projection was tiled at load (model-sized, aligned
        shapes: weights.fits_tiled), else the general row-major GEMM."""
        if wt is not None:
            ops.gemm_out(x, wt, out)
        else:
            ops.gemm_rm(x, w, out)

    def _attention(self, li: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        H, dn, dr, rk, dv = m.heads, m.dim, m.rot_dim, m.kv_rank, m.vdim
        rope = self._rope[(m.rot, m.rot_dim)]
        cache = self.kv[li]
        q = d["q"][:M * H * (dn + dr)].view(M, H, dn + dr)
        ckr = d["ckr"][:M * (rk + dr)].view(M, rk + dr)
        qabs = d["qabs"][:M * H * rk].view(M, H, rk)
        lat = d["lat"][:M * H * rk].view(M, H, rk)
        attn = d["attn"][:M * H * dv].view(M, H, dv)
        self._lin(d["xb"], Lw.q, Lw.q_t, q.view(M, H * (dn + dr)))
        ops.gemm_rm(d["xb"], Lw.dkv, ckr)
        vt = self.kv.vt.get(li)
        ops.latent_kv_write(ckr, Lw.dkv_norm, pos, slots, rope, cache, self.cfg.eps, vt)
        ops.gemm_rm(q[:, :, :dn].permute(1, 0, 2), Lw.uk_t, qabs.permute(1, 0, 2))
        for g in groups:
            if vt is not None:  # MFMA form: a decode row's heads side by side, a portion's rows in tiles of 16
                dec = g["qt"] == 1
                if dec:  # few items: their keys are split over partitions so that the chip is filled
                    B = g["ws"].numel()
                    np_ = self._decode_parts(B, H, m.window)
                    ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], rope,
                                         lat, m.window, m.scale, 1, vt, 16, self._flash_part if np_ > 1 else None, np_)
                else:
                    ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["fs"], g["ft"], rope,
                                         lat, m.window, m.scale, FLASH_ROWS_TILE, vt, 16 // FLASH_ROWS_TILE)
            else:
                ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], rope, lat,
                                     m.window, m.scale, g["qt"])
        ops.gemm_rm(lat.permute(1, 0, 2), Lw.uv, attn.permute(1, 0, 2))
        self._lin(attn.view(M, H * dv), Lw.o, Lw.o_t, d["y"])

    def _decode_parts(self, B: int, heads: int, window: int) -> int:
        """Key partitions of the decode attention: enough (item, head tile, partition) waves for the chip, at most one
        per page that a sequence can hold inside the window, at most 16."""
        pages = -(-min(window, self.max_model_len) // PAGE) + 1
        want = -(-FLASH_DECODE_WAVES // max(1, B * (-(-heads // 16))))
        return max(1, min(16, pages, want))

    def _recurrent(self, li: int, m, Lw, M: int, d: dict, groups: list) -> None:
        C, nb = m.width, m.blocks
        bw = C // nb
        ub, hs = (d[k][:M * C].view(M, C) for k in ("ub", "hs"))
        yr, ux, u = (d[k][:M * C].view(M, C) for k in ("yr", "ux", "u"))
        gates = d["gates"][:M * 2 * C].view(M, nb, 2 * bw)
        # both input projections leave fp32 without bias: the convolution adds its input's bias, the scan applies
        # the branch's bias and gelu
        self._lin(d["xb"], Lw.y, Lw.y_t, yr)
        self._lin(d["xb"], Lw.x, Lw.x_t, ux)
        for g in groups:
            ops.conv_state(ux, Lw.conv, Lw.conv_b, self.state.tail[li], g["qs"], g["ql"], g["ctx"], g["ss"], u, ub,
                           Lw.x_b)
        ops.gemm_rm(ub.view(M, nb, bw).permute(1, 0, 2), Lw.gates, gates.permute(1, 0, 2), bias=Lw.gates_b)
        for i, g in enumerate(groups):
            scr = d.get("scan")
            if scr is not None:
                slots = M // 32 + g["ql"].numel() + 1
                scr = scr[:2 * slots * C].view(2, slots, C)
            ops.lru_scan(u, gates, yr, Lw.lam, self.state.state[li], g["qs"], g["ql"], g["ctx"], g["ss"], hs,
                         LRU_DECAY_SCALE, Lw.y_b, i == 0, scr)
        self._lin(hs, Lw.o, Lw.o_t, d["y"])

    def _moe(self, f, Fw, M: int, d: dict):
        """Router + grouped experts; returns (per-slot outputs [M * S, W] fp32, S): the norm that follows sums them."""
        tki = d["tki"][:M * f.top].view(M, f.top)
        tkw = d["tkw"][:M * f.top].view(M, f.top)
        S = f.top + (1 if f.shared_ff else 0)
        o = d["mo_o"][:M * S * self.cfg.width].view(M * S, self.cfg.width)
        z = d["mo_z"][:M * f.experts].view(M, f.experts)
        ops.gemm_rm(d["xb"], Fw.router, z, bias=Fw.router_b)  # fp32 logits
        ops.moe_topk(z, tki, tkw)
        ops.moe_grouped(d["xb"], tki, tkw, Fw.gate, Fw.up, Fw.down, Fw.sgate, Fw.sup, Fw.sdown, d["mo_sorted"],
                        d["mo_tile"], d["mo_n"], d["mo_h"], o)
        return o, S

    def _layers(self, M: int, d: dict, ids, pos, slots, groups: list, trace: list | None = None, prev=None) -> None:
        """Embedding + every layer over M packed rows.  `groups`: sequence groups of the step (decode slots, prompt
        portions), each with its own metadata (block tables bt, q_start qs, q_len ql, ctx_len ctx, state slots ss,
        attention work items ws / wt of qt rows).  trace (a list) receives a copy of the stream after every layer.
        prev: (previous token per row, where decode rows store their own token, which of them do) for designs whose
        embedding reads the previous token."""
        cfg, eps = self.cfg, self.cfg.eps
        if self.bracket:
            self._bracket_layers(M, d, ids, prev, pos, slots, groups, trace)
            return
        if self.multistream:
            self._stream_layers(M, d, ids, pos, slots, groups, trace)
            return
        ops.embed_rows(ids, self.w.embed, d["resid"], d["xb"])
        if self.prenorm:
            self._prenorm_layers(M, d, ids, pos, slots, groups, trace)
            return
        for li, (L, Lw) in enumerate(zip(cfg.layers, self.w.layers)):
            if L.kind == "latent_attention":
                self._attention(li, L.mixer, Lw.mix, M, d, pos, slots, groups)
            else:
                self._recurrent(li, L.mixer, Lw.mix, M, d, groups)
            ops.scalar_norm(d["y"], Lw.norm1, d["resid"], d["xb"], eps)
            if L.mlp is not None:
                o, S = self._moe(L.mlp, Lw.mlp, M, d)
                ops.scalar_norm(o, Lw.norm2, d["resid"], d["xb"], eps, S)
            if trace is not None:
                trace.append(d["resid"].clone())

    def _lm_head(self, rows, logits) -> None:
        """rows: fp32 stream rows (not normed yet) -> final norm -> head GEMM (-> logit scale and cap)."""
        rows = rows.contiguous()
        xn = torch.empty(rows.shape, device=rows.device, dtype=self.dtype)
        self._head(rows, xn, logits)

    def _head(self, resid, xn, logits) -> None:
        if self.bracket:
            ops.add_norm_rows(None, 1, None, resid, self.w.final_norm, self.cfg.eps, xn)
            self._lin(xn, self.w.head, self.w.head_t, logits)
        elif self.multistream:  # resid holds the sum of the streams: one stream with weight 1 through the RMS norm
            ops.stream_mix(None, 1, 0.0, resid.unsqueeze(1), in_w=self.w.ones[:1], norm_w=self.w.final_norm,
                           eps=self.cfg.eps, h=xn)
            self._lin(xn, self.w.head, self.w.head_t, logits)
        elif self.prenorm:
            n, cfg = self.w.final_norm, self.cfg
            ops.stream_step(None, 0.0, resid, None, None, None, n.alpha, n.w, n.b, xn)
            self._lin(xn, self.w.head, self.w.head_t, logits)
            if cfg.logit_scale != 1.0 or cfg.logit_softcap > 0:
                ops.logit_cap(logits, cfg.logit_scale, cfg.logit_softcap)
        else:
            ops.scalar_norm(None, self.w.final_norm, resid, xn, self.cfg.eps)
            self._lin(xn, self.w.head, self.w.head_t, logits)

    # ------------------------------------------------------------------ pre-norm designs, matrix-state mixers
    def _prenorm_buffers(self, M: int) -> dict:
        """Scratch of a step of M rows, each sized for the widest layer: `big` takes the fused projection's fp32 output
        (its column ranges are the mixer's q, k, v and gates), `cv` the convolution's, `z` the per-channel
        decays, `qa` the attention's normed and rotated queries, `o` the recurrences' outputs, `ao` a mixer's gated
        output in the element type (the output projection's input), `y2` the second mixer of a parallel pair."""
        cfg, dev = self.cfg, self.device
        f32 = dict(device=dev, dtype=torch.float32)
        el = dict(device=dev, dtype=self.dtype)
        big = cv = z = qa = o = ff = 1
        for i, L in enumerate(cfg.layers):
            m = L.mixer
            if L.kind == "delta":
                big, cv = max(big, self.w.layers[i].mix.n_big), max(cv, 2 * m.kv_heads * m.dim + m.heads * m.vdim)
                o = max(o, m.heads * m.vdim)
            elif L.kind == "parallel":
                a, r = m.left, m.right
                big = max(big, self.w.layers[i].mix.n_big)
                z, qa = max(z, r.heads * r.dim), max(qa, a.heads * a.dim)
                o = max(o, a.heads * a.vdim, r.heads * r.vdim)
            else:
                big, o = max(big, 2 * m.heads * (m.dim + m.vdim)), max(o, m.heads * m.vdim)
            if L.mlp is not None:
                ff = max(ff, L.mlp.ff)
        return {"y2": torch.zeros(M, cfg.width, **f32), "big": torch.zeros(M * big, **f32),
                "cv": torch.zeros(M * cv, **f32), "z": torch.zeros(M * z, **f32),
                "qa": torch.zeros(M * qa, **f32), "o": torch.zeros(M * o, **f32), "ao": torch.zeros(M * o, **el),
                "gu": torch.zeros(M * 2 * ff, **f32), "h": torch.zeros(M * ff, **el)}

    def _prenorm_layers(self, M: int, d: dict, ids, pos, slots, groups: list, trace: list | None) -> None:
        """Every layer run over M packed rows.  Between sublayers ONE stream_step adds the finished sublayer's output
        (times the residual multiplier), what a new pass of the looped span adds (the embedding again, the pass's
        vector) and applies the next sublayer's norm; the last output is added before the head's norm."""
        cfg, w = self.cfg, self.w
        mult = cfg.residual_mult
        pending = None
        for run in self.runs:
            L, Lw = cfg.layers[run.layer], w.layers[run.layer]
            t = run.pass_no
            n = Lw.norm1
            ops.stream_step(pending, mult, d["resid"], ids if t > 0 else None, w.embed if t > 0 else None,
                            w.step[t] if t >= 0 else None, n.alpha, n.w, n.b, d["xb"])
            getattr(self, "_" + L.kind)(run.index, L.mixer, Lw.mix, M, d, pos, slots, groups)
            if L.mlp is not None:
                n = Lw.norm2
                ops.stream_step(d["y"], mult, d["resid"], None, None, None, n.alpha, n.w, n.b, d["xb"])
                self._dense_ff(L.mlp, Lw.mlp, M, d)
            pending = d["y"]
            if trace is not None:
                ops.stream_step(pending, mult, d["resid"], None, None, None, None, None, None, None)
                pending = None
                trace.append(d["resid"].clone())
        if pending is not None:
            ops.stream_step(pending, mult, d["resid"], None, None, None, None, None, None, None)

    def _dense_ff(self, f, Fw, M: int, d: dict) -> None:
        gu = d["gu"][:M * 2 * f.ff].view(M, 2 * f.ff)
        h = d["h"][:M * f.ff].view(M, f.ff)
        self._lin(d["xb"], Fw.gu, Fw.gu_t, gu)
        ops.gated_act(gu, h, 1)
        self._lin(h, Fw.down, Fw.down_t, d["y"])

    def _scratch(self, d: dict, name: str, numel: int):
        """An fp32 work area of the step, grown on demand and shared by its layers."""
        t = d.get(name)
        if t is None or t.numel() < numel:
            t = d[name] = torch.empty(numel, device=self.device, dtype=torch.float32)
        return t

    @staticmethod
    def _cols(buf, c0: int, heads: int, width: int):
        """Columns [c0, c0 + heads * width) of a row-major fp32 buffer as [rows, heads, width] (a view)."""
        return buf[:, c0:c0 + heads * width].unflatten(1, (heads, width))

    def _scan_out(self, ri: int, Lw_norm, gate, H: int, V: int, M: int, d: dict, q, k, v, decay, beta, groups, q_scale,
                  o_w, o_t, y) -> None:
        """Recurrence over every sequence group, per-head output norm times the SiLU gate, output projection."""
        o = d["o"][:M * H * V].view(M, H, V)
        for g in groups:
            if beta is None and "ck" in g:
                s_first, s_count, cm = g["ck"]
                D = k.shape[2]
                scr = self._scratch(d, "scan_s", cm.shape[1] * H * D * V)
                chan = decay is not None and decay.dim() == 3
                ascr = self._scratch(d, "scan_a", cm.shape[1] * H * D) if chan else None
                ops.matrix_scan_chunked(q, k, v, decay, self.state.state[ri], g["qs"], g["ql"], g["ctx"], g["ss"],
                                        s_first, s_count, cm, scr, ascr, o, q_scale)
            else:
                ops.matrix_scan(q, k, v, decay, beta, self.state.state[ri], g["qs"], g["ql"], g["ctx"], g["ss"], o,
                                q_scale)
        ao = d["ao"][:M * H * V].view(M, H * V)
        ops.gated_head_norm(o, Lw_norm, gate, self.cfg.eps, ao)
        self._lin(ao, o_w, o_t, y)

    def _delta(self, ri: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        H, G, D, V = m.heads, m.kv_heads, m.dim, m.vdim
        C = 2 * G * D + H * V
        big = d["big"][:M * Lw.n_big].view(M, Lw.n_big)
        small = big[:, C + H * V:C + H * V + 2 * H]   # per-head decay and write-strength pre-activations
        cv = d["cv"][:M * C].view(M, C)
        self._lin(d["xb"], Lw.big, Lw.big_t, big)
        for g in groups:
            ops.conv_state(big[:, :C], Lw.conv, None, self.state.tail.get(ri), g["qs"], g["ql"], g["ctx"], g["ss"], cv,
                           None, None, 1)
        q, k, v = self._cols(cv, 0, G, D), self._cols(cv, G * D, G, D), self._cols(cv, 2 * G * D, H, V)
        ops.norm_rope_rows(q, None, pos, None, q, None, 2, UNIT_EPS, D ** -0.5)
        ops.norm_rope_rows(k, None, pos, None, k, None, 2, UNIT_EPS, 1.0)
        ops.gate_math(small[:, :H], 0, Lw.a_log, Lw.dt_bias)
        ops.gate_math(small[:, H:], 1)
        self._scan_out(ri, Lw.norm, big[:, C:C + H * V], H, V, M, d, q, k, v, small[:, :H], small[:, H:], groups, 1.0,
                       Lw.o, Lw.o_t, d["y"])

    def _parallel(self, ri: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        a, r = m.left, m.right
        H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
        Hr, Dr, Vr = r.heads, r.dim, r.vdim
        NL, NR = (H + G) * D + G * V, 2 * Hr * (Dr + Vr)
        rank = Lw.a2.shape[1]
        big = d["big"][:M * Lw.n_big].view(M, Lw.n_big)
        small = big[:, NL + NR:NL + NR + H + rank]    # the attention's per-head gates | the decay's inner projection
        self._lin(d["xb"], Lw.big, Lw.big_t, big)
        # left: softmax attention with a sink over this run's pages
        rope = self._rope.get(a.rot)
        qa = d["qa"][:M * H * D].view(M, H, D)
        ops.norm_rope_rows(self._cols(big, 0, H, D), Lw.q_norm, pos, rope, qa, None, 1, self.cfg.eps, 1.0)
        ops.norm_rope_rows(self._cols(big, H * D, G, D), Lw.k_norm, pos, rope, self.kv.k[ri], slots, 1, self.cfg.eps,
                           1.0)
        vt = self.kv.vt.get(ri)
        ops.norm_rope_rows(self._cols(big, (H + G) * D, G, V), None, pos, None, self.kv.v[ri], slots, 0, 0.0, 1.0, vt)
        ao = d["ao"][:M * H * V].view(M, H, V)
        for g in groups:
            if vt is not None and g["qt"] > 1:  # prompt portions on the MFMA form: tiles of 16 rows
                ops.sink_attention(qa, self.kv.k[ri], self.kv.v[ri], g["bt"], g["qs"], g["ql"], g["ctx"], g["hs"],
                                   g["ht"], Lw.sink, small[:, :H], ao, a.window, a.scale, SINK_ROWS_TILE, vt)
            elif vt is not None and V <= ops.layers.SINK_SPLIT_MAX_V:  # decode rows: tile 0, keys split over the waves
                ops.sink_attention(qa, self.kv.k[ri], self.kv.v[ri], g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"],
                                   g["wt"], Lw.sink, small[:, :H], ao, a.window, a.scale, SINK_ROWS_TILE, vt, True)
            else:
                ops.sink_attention(qa, self.kv.k[ri], self.kv.v[ri], g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"],
                                   g["wt"], Lw.sink, small[:, :H], ao, a.window, a.scale, g["qt"])
        self._lin(ao.view(M, H * V), Lw.lo, Lw.lo_t, d["y"])
        # right: gated linear attention, decay per key channel from the low-rank projection (fp32 throughout)
        z = d["z"][:M * Hr * Dr].view(M, Hr * Dr)
        ops.gemm_rm(small[:, H:], Lw.a2, z, bias=Lw.a2_b)
        ops.gate_math(z, 2, None, None, r.tau)
        c0 = NL
        q, k = self._cols(big, c0, Hr, Dr), self._cols(big, c0 + Hr * Dr, Hr, Dr)
        v = self._cols(big, c0 + 2 * Hr * Dr, Hr, Vr)
        gate = big[:, c0 + 2 * Hr * Dr + Hr * Vr:NL + NR]
        self._scan_out(ri, Lw.rnorm, gate, Hr, Vr, M, d, q, k, v, z.view(M, Hr, Dr), None, groups, Dr ** -0.5, Lw.ro,
                       Lw.ro_t, d["y2"])
        ops.rms_mix(d["y"], Lw.left_out, d["y2"], Lw.right_out, self.cfg.eps, 0.5, d["y"])

    def _retention(self, ri: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        H, D, V = m.heads, m.dim, m.vdim
        N = 2 * H * (D + V)
        big = d["big"][:M * N].view(M, N)
        self._lin(d["xb"], Lw.big, Lw.big_t, big)
        rope = self._rope.get(m.rot)
        q, k, v = self._cols(big, 0, H, D), self._cols(big, H * D, H, D), self._cols(big, 2 * H * D, H, V)
        ops.norm_rope_rows(q, None, pos, rope, q, None, 0, 0.0, 1.0)
        ops.norm_rope_rows(k, None, pos, rope, k, None, 0, 0.0, D ** -0.5)
        self._scan_out(ri, None, big[:, 2 * H * D + H * V:], H, V, M, d, q, k, v, Lw.decay, None, groups, 1.0, Lw.o,
                       Lw.o_t, d["y"])

    # ------------------------------------------------------------------ pre-norm designs on several residual streams
    def _setup_streams(self) -> None:
        """Caches and state of a design on several residual streams, keyed by layer RUN: latent rows for the
        latent-attention runs, keys and values for the windowed-attention runs (same pages and block tables), and the
        tails of the input convolutions of both sublayers of every run."""
        cfg, dev = self.cfg, self.device
        self.runs = cfg.runs()
        lat, kv, tails, self._rope = {}, {}, {}, {}
        for r in self.runs:
            L, m = cfg.layers[r.layer], cfg.layers[r.layer].mixer
            if L.kind == "latent_attention":
                lat[r.index] = m
                key = (m.rot, m.rot_dim)
                if key not in self._rope:
                    self._rope[key] = m.rot.table(self.max_model_len + 1, m.rot_dim, dev)
            else:
                kv[r.index] = (m.kv_heads, m.dim, m.vdim)
            tails[(r.index, 1)] = (cfg.width, cfg.canon_taps)
            if L.mlp is not None:
                tails[(r.index, 2)] = (cfg.width, cfg.canon_taps)
        lflash = {r: m.kv_rank for r, m in lat.items() if ops.latent_flash_ok(self.dtype, m.kv_rank, m.rot_dim)}
        kflash = [r for r, (_, dm, v) in kv.items() if ops.sink_flash_ok(self.dtype, dm, v)]
        self.kv = MixedKVCache({r: m.kv_rank + m.rot_dim for r, m in lat.items()}, kv, self.num_blocks, dev, self.dtype,
                               latent_transposed=lflash, kv_transposed=kflash)
        self.state = ConvTailCache(tails, self.max_batch, dev)
        words = max((ops.latent_flash_part_floats(self.max_batch, m.heads, 16, 16, m.kv_rank) for r, m in lat.items()
                     if r in lflash), default=0)
        self._flash_part = torch.zeros(max(1, words), device=dev, dtype=torch.float32)

    def _stream_buffers(self, M: int) -> dict:
        """Scratch of a step of M rows, each sized for the widest layer: `streams` the residual copies, `hn` a
        sublayer's normed input before the input convolution and `hc` after it (fp32; the latter only where a router
        reads it), `big` the fused projection's fp32
        output, `cq` the normed query latent, `q` / `qabs` / `lat` the latent attention's operands, `o` a mixer's
        heads in fp32, `ao` them in the element type (the output projection's input), `up` / `h` the dense
        feed-forward's hidden row, and the routed experts' lists."""
        cfg, dev = self.cfg, self.device
        f32 = dict(device=dev, dtype=torch.float32)
        el = dict(device=dev, dtype=self.dtype)
        W = cfg.width
        big = cq = q = qabs = o = ff = qa = 1
        moe = []
        for i, L in enumerate(cfg.layers):
            m = L.mixer
            big = max(big, self.w.layers[i].mix.n_big)
            if L.kind == "latent_attention":
                cq, q = max(cq, m.q_rank), max(q, m.heads * (m.dim + m.rot_dim))
                qabs, o = max(qabs, m.heads * m.kv_rank), max(o, m.heads * m.vdim)
            else:
                qa, o = max(qa, m.heads * m.dim), max(o, m.heads * m.vdim)
            if L.mlp is not None:
                if hasattr(L.mlp, "experts"):
                    moe.append(L.mlp)
                else:
                    ff = max(ff, L.mlp.ff)
        d = {"streams": torch.zeros(M, cfg.num_streams, W, **f32), "hn": torch.zeros(M, W, **f32),
             "hc": torch.zeros(M, W, **f32) if moe else None, "big": torch.zeros(M * big, **f32), "cq": torch.zeros(M * cq, **el),
             "q": torch.zeros(M * q, **el), "qabs": torch.zeros(M * qabs, **f32), "lat": torch.zeros(M * qabs, **el),
             "qa": torch.zeros(M * qa, **f32), "o": torch.zeros(M * o, **f32), "ao": torch.zeros(M * o, **el),
             "up": torch.zeros(M * ff, **f32), "h": torch.zeros(M * ff, **el)}
        if moe:
            top = max(f.top for f in moe)
            tiles = -(-M * top // 64) + max(f.experts for f in moe) + 2
            ldh = -(-max(f.ff for f in moe) // 8) * 8
            d.update({"tki": torch.zeros(M * top, device=dev, dtype=torch.int32), "tkw": torch.zeros(M * top, **f32),
                      "mo_z": torch.zeros(M * max(f.experts for f in moe), **f32),
                      "mo_sorted": torch.zeros(tiles * 64, device=dev, dtype=torch.int32),
                      "mo_tile": torch.zeros(tiles, device=dev, dtype=torch.int32),
                      "mo_n": torch.zeros(1, device=dev, dtype=torch.int32), "mo_h": torch.zeros(M * top, ldh, **el),
                      "mo_o": torch.zeros(M * top * W, **f32)})
        return d

    def _stream_layers(self, M: int, d: dict, ids, pos, slots, groups: list, trace: list | None) -> None:
        """Every layer run over M packed rows.  Between sublayers ONE stream_mix writes the finished sublayer's output
        into all streams (through its mix matrix and output weights, times the residual multiplier), forms the next
        sublayer's input from them and RMS-norms it; the first one also fills the streams with the scaled embedding.
        The input convolution then continues each sequence's tail.  At the end d["resid"] holds the sum of the streams
        (what the head's norm reads)."""
        cfg, w = self.cfg, self.w
        mult, eps, x = cfg.residual_mult, cfg.eps, d["streams"]
        prev = None  # (output rows, parts per row, stream weights) of the sublayer that is not written back yet
        first = True
        for run in self.runs:
            L, Lw = cfg.layers[run.layer], w.layers[run.layer]
            for sub, hc in ((1, Lw.hc1), (2, Lw.hc2)):
                if hc is None:
                    continue
                y, nsum, pw = prev if prev else (None, 1, None)
                conv = hc.canon is not None and hc.canon.shape[1] > 0
                routed = sub == 2 and hasattr(L.mlp, "experts")  # the router reads the fp32 row, not its rounding
                ops.stream_mix(y, nsum, mult, x, ids if first else None, w.embed if first else None, cfg.embed_scale,
                               pw.outw if pw else None, pw.mix if pw else None, hc.inw, hc.norm, eps,
                               d["hn"] if conv or routed else d["xb"])
                first = False
                if conv:
                    for g in groups:
                        ops.conv_state(d["hn"], hc.canon, None, self.state.tail.get((run.index, sub)), g["qs"], g["ql"],
                                       g["ctx"], g["ss"], d["hc"] if routed else None, d["xb"], None, 2, g["qt"] == 1)
                elif routed:
                    ops.act_rows(d["hn"], d["xb"], 0)
                if sub == 1:
                    getattr(self, "_" + L.kind + "_streams")(run.index, L.mixer, Lw.mix, M, d, pos, slots, groups)
                    prev = (d["y"], 1, hc)
                elif routed:
                    prev = self._routed_ff(L.mlp, Lw.mlp, M, d, d["hc"] if conv else d["hn"]) + (hc,)
                else:
                    self._act_ff(L.mlp, Lw.mlp, M, d)
                    prev = (d["y"], 1, hc)
            if trace is not None:
                y, nsum, pw = prev
                ops.stream_mix(y, nsum, mult, x, out_w=pw.outw, mix=pw.mix, total=d["resid"])
                prev = None
                trace.append(d["resid"].clone())
        y, nsum, pw = prev if prev else (None, 1, None)
        ops.stream_mix(y, nsum, mult, x, ids if first else None, w.embed if first else None, cfg.embed_scale,
                       pw.outw if pw else None, pw.mix if pw else None, total=d["resid"])

    def _latent_attention_streams(self, ri: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        """Latent attention with a query latent and a sigmoid output gate: ONE fused GEMM [dq | dkv | g] (fp32 out) ->
        RMS norm of the query latent -> query up-projection; latent_kv_write (norm + rotation + cache row) from the
        dkv columns; folded attention over this run's latent pages; per-head value up-projection (fp32) times
        sigmoid(g) -> output GEMM."""
        H, dn, dr, rk, dv, qr = m.heads, m.dim, m.rot_dim, m.kv_rank, m.vdim, m.q_rank
        rope = self._rope[(m.rot, m.rot_dim)]
        cache, vt = self.kv.latent[ri], self.kv.latent.vt.get(ri)
        big = d["big"][:M * Lw.n_big].view(M, Lw.n_big)
        cq = d["cq"][:M * qr].view(M, qr)
        q = d["q"][:M * H * (dn + dr)].view(M, H, dn + dr)
        qabs = d["qabs"][:M * H * rk].view(M, H, rk)
        lat = d["lat"][:M * H * rk].view(M, H, rk)
        o = d["o"][:M * H * dv].view(M, H, dv)
        ao = d["ao"][:M * H * dv].view(M, H * dv)
        self._lin(d["xb"], Lw.big, Lw.big_t, big)
        # the query latent's RMS norm: one "stream" with weight 1 (any width, read in place from the fused output)
        ops.stream_mix(None, 1, 0.0, big[:, :qr].unsqueeze(1), in_w=self.w.ones[:1], norm_w=Lw.dq_norm, eps=self.cfg.eps,
                       h=cq)
        self._lin(cq, Lw.uq, Lw.uq_t, q.view(M, H * (dn + dr)))
        ops.latent_kv_write(big[:, qr:qr + rk + dr], Lw.dkv_norm, pos, slots, rope, cache, self.cfg.eps, vt)
        if dn > 0:
            ops.gemm_rm(q[:, :, :dn].permute(1, 0, 2), Lw.uk_t, qabs.permute(1, 0, 2))
        else:  # heads without an unrotated part: nothing folds into the latent
            qabs.zero_()
        for g in groups:
            if vt is not None:
                if g["qt"] == 1:
                    np_ = self._decode_parts(g["ws"].numel(), H, m.window)
                    ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], rope,
                                         lat, m.window, m.scale, 1, vt, 16, self._flash_part if np_ > 1 else None, np_)
                else:
                    ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["fs"], g["ft"], rope,
                                         lat, m.window, m.scale, FLASH_ROWS_TILE, vt, 16 // FLASH_ROWS_TILE)
            else:
                ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], rope, lat,
                                     m.window, m.scale, g["qt"])
        ops.gemm_rm(lat.permute(1, 0, 2), Lw.uv, o.permute(1, 0, 2))
        ops.act_rows(o.view(M, H * dv), ao, 0, None, big[:, qr + rk + dr:qr + rk + dr + H * dv])
        self._lin(ao, Lw.o, Lw.o_t, d["y"])

    def _attention_streams(self, ri: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        """Sliding-window attention with grouped key/value heads and per-head RMS norms on q and k, no rotation: ONE
        fused GEMM [q | k | v] -> norm rows (q to a buffer, k and v straight into this run's pages) -> attention over
        the window (MFMA form where the head widths allow it) -> output GEMM."""
        H, G, D, V = m.heads, m.kv_heads, m.dim, m.vdim
        big = d["big"][:M * Lw.n_big].view(M, Lw.n_big)
        self._lin(d["xb"], Lw.big, Lw.big_t, big)
        kc, vc, vt = self.kv.paged.k[ri], self.kv.paged.v[ri], self.kv.paged.vt.get(ri)
        qa = d["qa"][:M * H * D].view(M, H, D)
        eps = self.cfg.eps
        ops.norm_rope_rows(self._cols(big, 0, H, D), Lw.q_norm, pos, None, qa, None, 3, eps, 1.0)
        ops.norm_rope_rows(self._cols(big, H * D, G, D), Lw.k_norm, pos, None, kc, slots, 3, eps, 1.0)
        ops.norm_rope_rows(self._cols(big, (H + G) * D, G, V), None, pos, None, vc, slots, 0, 0.0, 1.0, vt)
        ao = d["ao"][:M * H * V].view(M, H, V)
        for g in groups:
            if vt is not None and g["qt"] > 1:
                ops.sink_attention(qa, kc, vc, g["bt"], g["qs"], g["ql"], g["ctx"], g["hs"], g["ht"], None, None, ao,
                                   m.window, m.scale, SINK_ROWS_TILE, vt)
            elif vt is not None and V <= ops.layers.SINK_SPLIT_MAX_V:
                ops.sink_attention(qa, kc, vc, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], None, None, ao,
                                   m.window, m.scale, SINK_ROWS_TILE, vt, True)
            else:
                ops.sink_attention(qa, kc, vc, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], None, None, ao,
                                   m.window, m.scale, g["qt"])
        self._lin(ao.view(M, H * V), Lw.o, Lw.o_t, d["y"])

    def _act_ff(self, f, Fw, M: int, d: dict) -> None:
        """Dense feed-forward: up GEMM (fp32) -> xIELU -> down GEMM."""
        up = d["up"][:M * f.ff].view(M, f.ff)
        h = d["h"][:M * f.ff].view(M, f.ff)
        self._lin(d["xb"], Fw.up, Fw.up_t, up)
        ops.act_rows(up, h, 1, Fw.act)
        self._lin(h, Fw.down, Fw.down_t, d["y"])

    def _routed_ff(self, f, Fw, M: int, d: dict, h32):
        """Router GEMM in true fp32 on the sublayer's fp32 input `h32` (a close call is decided by the row itself, not by
        its rounding) -> group-limited sigmoid routing -> grouped squared-ReLU experts on the element-type row; returns
        (per-slot outputs [M * top, W] fp32, top): the stream step that follows sums them."""
        tki = d["tki"][:M * f.top].view(M, f.top)
        tkw = d["tkw"][:M * f.top].view(M, f.top)
        o = d["mo_o"][:M * f.top * self.cfg.width].view(M * f.top, self.cfg.width)
        z = d["mo_z"][:M * f.experts].view(M, f.experts)
        ops.gemm_rm(h32, Fw.router, z)
        ops.moe_route(z, Fw.correction, tki, tkw, f.groups, f.keep, f.scale)
        ops.moe_grouped(d["xb"], tki, tkw, None, Fw.up, Fw.down, None, None, None, d["mo_sorted"], d["mo_tile"],
                        d["mo_n"], d["mo_h"], o)
        return o, f.top


    # ------------------------------------------------------------------ bracketing norms, token inputs, rotated values
    def _setup_bracket(self) -> None:
        """Caches and state of a design with bracketing norms, keyed by layer RUN: keys and values (the values rotated
        by their positions) for the attention runs, matrix state and convolution tail for the channel-delta runs, and
        every slot's previous token (the hashed bigram embedding reads it)."""
        cfg, dev = self.cfg, self.device
        self.runs = cfg.runs()
        kv, st, self._rope = {}, {}, {}
        for r in self.runs:
            L, m = cfg.layers[r.layer], cfg.layers[r.layer].mixer
            if L.kind == "attention":
                kv[r.index] = (m.kv_heads, m.dim, m.vdim)
                for dims in (m.rot_dims, m.vdim):
                    rot = HalfRotarySpec(dims=dims, base=m.rot_base)
                    if dims > 0 and rot not in self._rope:
                        self._rope[rot] = rot.table(self.max_model_len + 1, dev)
            else:
                st[r.index] = ((m.heads, m.dim, m.vdim), 2 * m.kv_heads * m.dim + m.heads * m.vdim, m.conv)
        # the MFMA form turns a head's output back inside its registers: both halves of a pair must be whole tiles
        flash = [r for r, (_, dm, v) in kv.items() if ops.sink_flash_ok(self.dtype, dm, v) and v % 32 == 0]
        self.kv = PagedKVCache(kv, self.num_blocks, dev, self.dtype, transposed=flash)
        self.state = MatrixStateCache(st, self.max_batch, dev)
        self.prev_ids = torch.zeros(self.max_batch, device=dev, dtype=torch.int32)
        self._host_prev = {}  # slot -> last token of the latest prompt portion (when the caller names no predecessor)

    def _bracket_buffers(self, M: int) -> dict:
        """Scratch of a step of M rows, each sized for the widest layer: `big` the fused projection's fp32 output, `cv`
        the convolution's, `z` the per-channel decays beside the output gate's pre-activations, `qa` the attention's
        normed and rotated queries, `o` the recurrence's heads, `ao` a mixer's gated output in the element type, `up` /
        `h` the dense feed-forward's hidden row, `hn` the fp32 normed row a router reads, `cat` [stream | embedding
        output] for the projection that opens a loop pass, `sg` / `sh` the token input's gate, and the experts' lists."""
        from ..models.murulorn import SoftmaxRoutedSpec

        cfg, dev = self.cfg, self.device
        f32 = dict(device=dev, dtype=torch.float32)
        el = dict(device=dev, dtype=self.dtype)
        W = cfg.width
        big = cv = z = qa = o = ff = 1
        moe = []
        for i, L in enumerate(cfg.layers):
            m = L.mixer
            big = max(big, self.w.layers[i].mix.n_big)
            o = max(o, m.heads * m.vdim)
            if L.kind == "attention":
                qa = max(qa, m.heads * m.dim)
            else:
                cv, z = max(cv, 2 * m.kv_heads * m.dim + m.heads * m.vdim), max(z, m.heads * (m.dim + m.vdim))
            if isinstance(L.mlp, SoftmaxRoutedSpec):
                moe.append(L.mlp)
            elif L.mlp is not None:
                ff = max(ff, L.mlp.ff)
        d = {"big": torch.zeros(M * big, **f32), "cv": torch.zeros(M * cv, **f32), "z": torch.zeros(M * z, **f32),
             "qa": torch.zeros(M * qa, **f32), "o": torch.zeros(M * o, **f32),
             "ao": torch.zeros(M * o, **el), "up": torch.zeros(M * ff, **f32), "h": torch.zeros(M * ff, **el),
             "hn": torch.zeros(M, W, **f32) if moe else None,
             "cat": torch.zeros(M, 2 * W, **el) if cfg.loop_times > 0 else None,
             "sg": torch.zeros(M * max(1, cfg.side_dim), **f32), "sh": torch.zeros(M * max(1, cfg.side_dim), **el)}
        if moe:
            top = max(f.top for f in moe)
            tiles = -(-M * top // 64) + max(f.experts for f in moe) + 2
            ldh = -(-max(f.ff for f in moe) // 8) * 8
            d.update({"tki": torch.zeros(M * top, device=dev, dtype=torch.int32), "tkw": torch.zeros(M * top, **f32),
                      "mo_z": torch.zeros(M * max(f.experts for f in moe), **f32),
                      "mo_sorted": torch.zeros(tiles * 64, device=dev, dtype=torch.int32),
                      "mo_tile": torch.zeros(tiles, device=dev, dtype=torch.int32),
                      "mo_n": torch.zeros(1, device=dev, dtype=torch.int32), "mo_h": torch.zeros(M * top, ldh, **el),
                      "mo_o": torch.zeros(M * top * W, **f32)})
        return d

    def _bracket_layers(self, M: int, d: dict, ids, prev, pos, slots, groups: list, trace: list | None) -> None:
        """Every layer run over M packed rows.  Between sublayers ONE add_norm_rows adds the finished sublayer's normed
        output to the stream and norms the stream for the next one (or rounds it, for the token input's gate and for
        the projection that opens a loop pass); the last output is added before the head's norm.  `pending` is the
        sublayer output that is not in the stream yet: (rows, parts per row, gain of its norm).  Decode-sized steps
        run a layer's token input as ONE launch (token_side_rows) that also writes the next sublayer's input."""
        from ..models.murulorn import SoftmaxRoutedSpec

        cfg, w, eps = self.cfg, self.w, self.cfg.eps
        W = cfg.width
        bg = cfg.bigram
        prev_rows, prev_out, keep = prev if prev is not None else (None, None, None)
        if bg is not None and prev_rows is None:
            raise ValueError(f"{cfg.name}: the embedding reads each row's previous token")
        cat = d["cat"]
        ops.embed_pair_rows(ids, prev_rows, pos, w.embed, w.bigram, bg.mul_prev if bg else 0, bg.mul_cur if bg else 0,
                            bg.buckets if bg else 1, d["resid"], cat[:, W:] if cat is not None else None, prev_out, keep)
        pending = (None, 1, None)
        ready = False  # the next sublayer's input (xb, or the stream's half of cat) is already written
        fused_side = cfg.side_dim > 0 and ops.token_side_fits(M, W, cfg.side_dim)
        for n, run in enumerate(self.runs):
            L, Lw = cfg.layers[run.layer], w.layers[run.layer]
            if run.pass_no >= 0:  # a pass of the looped span opens: stream <- W_in [stream | embedding output]
                if not ready:
                    ops.add_norm_rows(*pending, d["resid"], None, eps, cat[:, :W])
                self._lin(cat, w.loop_in, w.loop_in_t, d["resid"])
                pending, ready = (None, 1, None), False
            if not ready:
                ops.add_norm_rows(*pending, d["resid"], Lw.norm1, eps, d["xb"])
            ready = False
            getattr(self, "_" + L.kind + "_bracket")(run.index, L.mixer, Lw.mix, M, d, pos, slots, groups)
            pending = (d["y"], 1, Lw.norm1b)
            if L.mlp is not None:
                routed = isinstance(L.mlp, SoftmaxRoutedSpec)
                ops.add_norm_rows(*pending, d["resid"], Lw.norm2, eps, d["xb"], d["hn"] if routed else None)
                if routed:
                    pending = self._softmax_routed_ff(L.mlp, Lw.mlp, M, d) + (Lw.norm2b,)
                else:
                    self._relu2_ff(L.mlp, Lw.mlp, M, d)
                    pending = (d["y"], 1, Lw.norm2b)
            if Lw.side is not None:  # the layer's token input reads the stream after the feed-forward
                sd = Lw.side
                if fused_side:  # decode-sized steps: one launch, which also makes the next sublayer's input
                    nxt = self.runs[n + 1] if n + 1 < len(self.runs) else None
                    g_out, out = None, None
                    if trace is None and nxt is not None:
                        g_out, out = (None, cat[:, :W]) if nxt.pass_no >= 0 else (w.layers[nxt.layer].norm1, d["xb"])
                    ops.token_side_rows(*pending, d["resid"], ids, w.side_embed, sd.col0, sd.gate, sd.proj, sd.norm, g_out,
                                        eps, out)
                    pending, ready = (None, 1, None), out is not None
                else:
                    F = sd.gate.shape[0]
                    sg, sh = d["sg"][:M * F].view(M, F), d["sh"][:M * F].view(M, F)
                    ops.add_norm_rows(*pending, d["resid"], None, eps, d["xb"])
                    ops.gemm_rm(d["xb"], sd.gate, sg)
                    ops.token_gate_rows(sg, ids, w.side_embed, sd.col0, sh)
                    ops.gemm_rm(sh, sd.proj, d["y"])
                    pending = (d["y"], 1, sd.norm)
            if trace is not None:
                if pending[0] is not None:
                    ops.add_norm_rows(*pending, d["resid"], None, eps)
                pending = (None, 1, None)
                trace.append(d["resid"].clone())
        if pending[0] is not None:
            ops.add_norm_rows(*pending, d["resid"], None, eps)

    def _attention_bracket(self, ri: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        """Softmax attention whose values are rotated by their positions: ONE fused GEMM [q | k | v | g] (fp32 out) ->
        norm rows (q: whole-row RMS norm + rotation into a buffer; k the same into this run's pages; v: RMS norm per
        head + rotation over the whole value width into the pages, also transposed) -> attention over the window with
        capped scores, each head's sum turned back by the row's position and gated -> output GEMM."""
        H, G, D, V = m.heads, m.kv_heads, m.dim, m.vdim
        big = d["big"][:M * Lw.n_big].view(M, Lw.n_big)
        self._lin(d["xb"], Lw.big, Lw.big_t, big)
        kc, vc, vt = self.kv.k[ri], self.kv.v[ri], self.kv.vt.get(ri)
        rope = self._rope.get(HalfRotarySpec(dims=m.rot_dims, base=m.rot_base))
        vrope = self._rope[HalfRotarySpec(dims=V, base=m.rot_base)]
        qa = d["qa"][:M * H * D].view(M, H, D)
        eps = self.cfg.eps
        ops.norm_rope_rows(self._cols(big, 0, H, D), Lw.q_norm, pos, rope, qa, None, 1, eps, 1.0)
        ops.norm_rope_rows(self._cols(big, H * D, G, D), Lw.k_norm, pos, rope, kc, slots, 1, eps, 1.0)
        ops.norm_rope_rows(self._cols(big, (H + G) * D, G, V), None, pos, vrope, vc, slots, 3, eps, 1.0, vt)
        gate = big[:, (H + G) * D + G * V:(H + G) * D + G * V + H]
        ao = d["ao"][:M * H * V].view(M, H, V)
        for g in groups:
            if vt is not None and g["qt"] > 1:
                ops.sink_attention(qa, kc, vc, g["bt"], g["qs"], g["ql"], g["ctx"], g["hs"], g["ht"], None, gate, ao,
                                   m.window, m.scale, SINK_ROWS_TILE, vt, False, m.softcap, vrope)
            elif vt is not None and V <= ops.layers.SINK_SPLIT_MAX_V:
                ops.sink_attention(qa, kc, vc, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], None, gate, ao,
                                   m.window, m.scale, SINK_ROWS_TILE, vt, True, m.softcap, vrope)
            else:
                ops.sink_attention(qa, kc, vc, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], None, gate, ao,
                                   m.window, m.scale, g["qt"], None, False, m.softcap, vrope)
        self._lin(ao.view(M, H * V), Lw.o, Lw.o_t, d["y"])

    def _channel_delta_bracket(self, ri: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        """Gated delta rule with a decay per head and key channel: ONE fused GEMM [q | k | v | b | a1 | g1] (fp32 out)
        -> conv_state over q | k | v (SiLU; slot tail) -> unit q, k per head in one launch (the query's dim^-1/2
        rides in the scan) -> the decay's and the gate's second projections in fp32 as one block-diagonal product
        -> gate_math (one rate per head, one bias per head and channel) -> matrix_scan (delta rule
        with per-channel decay; slot state) -> per-head RMS norm times the sigmoid gate -> output GEMM."""
        H, G, D, V = m.heads, m.kv_heads, m.dim, m.vdim
        C = 2 * G * D + H * V
        big = d["big"][:M * Lw.n_big].view(M, Lw.n_big)
        cv = d["cv"][:M * C].view(M, C)
        self._lin(d["xb"], Lw.big, Lw.big_t, big)
        for g in groups:
            ops.conv_state(big[:, :C], Lw.conv, None, self.state.tail.get(ri), g["qs"], g["ql"], g["ctx"], g["ss"], cv,
                           None, None, 1, g["qt"] == 1)
        q, k, v = self._cols(cv, 0, G, D), self._cols(cv, G * D, G, D), self._cols(cv, 2 * G * D, H, V)
        qk = self._cols(cv, 0, 2 * G, D)   # q and k heads side by side: one launch makes them unit vectors
        ops.norm_rope_rows(qk, None, pos, None, qk, None, 2, UNIT_EPS, 1.0)
        beta = big[:, C:C + H]
        ops.gate_math(beta, 1)
        zz = d["z"][:M * H * (D + V)].view(M, H * (D + V))
        z, gz = zz[:, :H * D], zz[:, H * D:]
        ops.gemm_rm(big[:, C + H:C + H + Lw.ra + Lw.rg], Lw.ag2, zz)
        ops.gate_math(z, 0, Lw.a_log, Lw.dt_bias)
        o = d["o"][:M * H * V].view(M, H, V)
        for g in groups:
            ops.matrix_scan(q, k, v, z.unflatten(1, (H, D)), beta, self.state.state[ri], g["qs"], g["ql"], g["ctx"],
                            g["ss"], o, D ** -0.5)
        ao = d["ao"][:M * H * V].view(M, H * V)
        ops.gated_head_norm(o, Lw.norm, gz, self.cfg.eps, ao, 1)
        self._lin(ao, Lw.o, Lw.o_t, d["y"])

    def _relu2_ff(self, f, Fw, M: int, d: dict) -> None:
        """Dense feed-forward: up GEMM (fp32) -> squared ReLU -> down GEMM."""
        up = d["up"][:M * f.ff].view(M, f.ff)
        h = d["h"][:M * f.ff].view(M, f.ff)
        self._lin(d["xb"], Fw.up, Fw.up_t, up)
        ops.act_rows(up, h, 2)
        self._lin(h, Fw.down, Fw.down_t, d["y"])

    def _softmax_routed_ff(self, f, Fw, M: int, d: dict):
        """Router GEMM in true fp32 on the fp32 normed row -> softmax scores, group-limited choice, unnormalised weights
        -> grouped squared-ReLU experts on the element-type row; returns (per-slot outputs [M * top, W] fp32, top): the
        add_norm_rows that follows sums them."""
        tki = d["tki"][:M * f.top].view(M, f.top)
        tkw = d["tkw"][:M * f.top].view(M, f.top)
        o = d["mo_o"][:M * f.top * self.cfg.width].view(M * f.top, self.cfg.width)
        z = d["mo_z"][:M * f.experts].view(M, f.experts)
        ops.gemm_rm(d["hn"], Fw.router, z)
        ops.moe_route(z, None, tki, tkw, f.groups, f.keep, 1.0, 1)
        ops.moe_grouped(d["xb"], tki, tkw, None, Fw.up, Fw.down, None, None, None, d["mo_sorted"], d["mo_tile"],
                        d["mo_n"], d["mo_h"], o)
        return o, f.top

    def _remember_last(self, seqs: list, g: dict) -> None:
        """After prompt portions: every portion's last token becomes its slot's previous token."""
        if not self.bracket:
            return
        self.prev_ids.index_copy_(0, g["ss"].long(), g["last"])
        for s in seqs:
            self._host_prev[s.slot] = int(s.tokens[-1])

    # ------------------------------------------------------------------ decode
    def _decode_group(self, B: int) -> dict:
        r = slice(0, B)
        return {"bt": self.block_tables[r], "qs": self.q_start[r], "ql": self.q_len[r], "ctx": self.ctx_len[r],
                "ss": self.q_start[r], "ws": self.work_seq[r], "wt": self.work_tile[r], "qt": 1}

    def decode_forward(self, B: int) -> None:
        """One decode step over slots [0, B) (graph-capturable: fixed shapes, no host sync).  Inactive slots
        (q_len 0) write no cache row and touch no state."""
        r = slice(0, B)
        ops.decode_prep(self.active[r], self.positions[r], self.block_tables[r], self.slots[r], self.ctx_len[r],
                        self.q_len[r], self.kv.num_blocks)
        rows = ("resid", "xb", "y", "y2", "streams", "hn", "hc", "cat")
        d = {k: (v[:B] if k in rows and v is not None else v) for k, v in self._dec.items()}
        prev = (self.prev_ids[r], self.prev_ids[r], self.q_len[r]) if self.bracket else None
        self._layers(B, d, self.ids[r], self.positions[r], self.slots[r], [self._decode_group(B)], prev=prev)
        self._head(d["resid"], self._dec["xb"][:B], self.logits[r])
        self._sample_commit(B)
        ops.ring_advance(self.ring_counter)

    def capture(self, buckets=None) -> None:
        """Capture the decode step of each batch bucket into its own graph (shared memory pool)."""
        if not self.use_graphs:
            return
        buckets = buckets or batch_buckets(self.max_batch)
        s = torch.cuda.Stream(self.device)
        s.wait_stream(torch.cuda.current_stream(self.device))
        saved = self._snapshot_state()
        act = self.active.clone()
        self.active.zero_()  # every slot inactive: the warm-up and capture runs touch no cache row and no state
        with torch.cuda.stream(s):
            for B in buckets:
                self.decode_forward(B)
        torch.cuda.current_stream(self.device).wait_stream(s)
        torch.cuda.synchronize(self.device)
        for B in sorted(buckets, reverse=True):
            g = torch.cuda.CUDAGraph()
            with _capture(g, pool=self.graph_pool):
                self.decode_forward(B)
            if self.graph_pool is None:
                self.graph_pool = g.pool()
            self.graphs[B] = g
        torch.cuda.synchronize(self.device)
        self.active.copy_(act)
        self._restore_state(saved)

    def move_slots(self, src: list, dst: list) -> None:
        """Slot compaction: last token and position (RunnerBase) and the recurrent state of each moved slot."""
        super().move_slots(src, dst)
        idx = torch.tensor([src, dst], dtype=torch.long)
        if self.device.type == "cuda":
            idx = idx.pin_memory().to(self.device, non_blocking=True)
        self.state.move(idx[0], idx[1])
        if self.bracket:
            self.prev_ids.index_copy_(0, idx[1], self.prev_ids.index_select(0, idx[0]))
            moved = {b: self._host_prev.get(a) for a, b in zip(src, dst)}
            self._host_prev.update({b: t for b, t in moved.items() if t is not None})

    def close(self) -> None:
        pass

    # ------------------------------------------------------------------ prompt portions
    def _pack(self, seqs: list, row0: int = 0):
        """Packed metadata of prompt portions whose rows start at `row0`: one pinned upload.  Returns (T, q_start
        list, device dict: ids / pos / slots per row, qs / ql / ctx / ss per sequence, ws / wt work items, bt)."""
        n = len(seqs)
        ids_l, pos_l, slots_l, qs, ql, ctx, ss = [], [], [], [], [], [], []
        ws, wt, fs, ft, hs, ht = [], [], [], [], [], []
        prev_l, last = [], []
        bt = torch.zeros(n, self.max_blocks, dtype=torch.int32)
        row = 0
        for i, s in enumerate(seqs):
            m = len(s.tokens)
            p = s.start_pos + np.arange(m, dtype=np.int64)
            table = np.asarray(s.block_table, dtype=np.int64)
            ids_l.append(np.asarray(s.tokens, dtype=np.int64))
            if self.bracket:  # each row's previous token: the caller's (or the slot's remembered one), then the portion's own
                first = -1
                if s.start_pos > 0:
                    first = s.prev_token if s.prev_token >= 0 else self._host_prev.get(s.slot, -1)
                    if first < 0:
                        raise ValueError(f"slot {s.slot}: a portion that starts at position {s.start_pos} needs the token "
                                         "before it (PrefillSeq.prev_token)")
                prev_l.append(np.concatenate([[first], ids_l[-1][:-1]]).astype(np.int64))
                last.append(int(s.tokens[-1]))
            pos_l.append(p)
            slots_l.append(table[p // PAGE] * PAGE + p % PAGE)
            qs.append(row0 + row)
            ql.append(m)
            ctx.append(s.start_pos + m)
            ss.append(s.slot)
            bt[i, : len(s.block_table)] = torch.from_numpy(table.astype(np.int32))
            nt = math.ceil(m / ATTN_ROWS_TILE)
            ws += [i] * nt
            wt += list(range(nt))
            nf = math.ceil(m / FLASH_ROWS_TILE)
            fs += [i] * nf
            ft += list(range(nf))
            nh = math.ceil(m / SINK_ROWS_TILE)
            hs += [i] * nh
            ht += list(range(nh))
            row += m
        T = row
        lists = np.asarray(qs + ql + ctx + ss + ws + wt + fs + ft + hs + ht + last, dtype=np.int64)
        meta = torch.from_numpy(np.concatenate(ids_l + pos_l + slots_l + prev_l + [lists]).astype(np.int32))
        if self.device.type == "cuda":
            meta = meta.pin_memory().to(self.device, non_blocking=True)
            bt = bt.pin_memory().to(self.device, non_blocking=True)
        d, o = {}, 0
        for name, k in (("ids", T), ("pos", T), ("slots", T), ("prev", T if self.bracket else 0), ("qs", n), ("ql", n),
                        ("ctx", n), ("ss", n), ("ws", len(ws)), ("wt", len(ws)), ("fs", len(fs)), ("ft", len(fs)),
                        ("hs", len(hs)), ("ht", len(hs)), ("last", len(last))):
            d[name], o = meta[o:o + k], o + k
        d["bt"] = bt
        d["qt"] = ATTN_ROWS_TILE
        if self.prenorm and T >= ops.layers.SCAN_CHUNKED_FROM:  # long portions: the recurrences' two-level walk
            s_first, s_count, rows = ops.layers.scan_chunks(qs, ql, ss)
            ck = torch.tensor([s_first, s_count], dtype=torch.int32)
            cm = torch.tensor(rows, dtype=torch.int32)
            if self.device.type == "cuda":
                ck = ck.pin_memory().to(self.device, non_blocking=True)
                cm = cm.pin_memory().to(self.device, non_blocking=True)
            d["ck"] = (ck[0], ck[1], cm)
        return T, qs, ql, d

    def prefill(self, seqs: list, ring_row: int, trace: list | None = None) -> None:
        """One packed batch of prompt portions.  Sequences whose last portion this is sample their first token into
        ids[slot] and ring[ring_row, slot]; portions that ask for logits (PrefillSeq.want) leave them in kept_logits."""
        if not seqs:
            return
        T, qs, ql, g = self._pack(seqs)
        d = self._buffers(T)
        self._layers(T, d, g["ids"], g["pos"], g["slots"], [g], trace, prev=(g["prev"], None, None))
        self._remember_last(seqs, g)
        self._prefill_sample(seqs, d["resid"], qs, ql, ring_row)
        self._keep_logits(seqs, d["resid"], qs)

    def mixed(self, B: int, seqs: list, ring_row: int) -> None:
        """ONE forward over the decode slots [0, B) and the prompt portions `seqs` (rows B .. B + T - 1): the weights
        stream once for both.  The decode rows sample and commit as the decode step does, finishing portions sample
        their first token as prefill() does."""
        T, qs, ql, g = self._pack(seqs, row0=B)
        M = B + T
        r = slice(0, B)
        ops.decode_prep(self.active[r], self.positions[r], self.block_tables[r], self.slots[r], self.ctx_len[r],
                        self.q_len[r], self.kv.num_blocks)
        ids = torch.cat([self.ids[r], g["ids"]])
        pos = torch.cat([self.positions[r], g["pos"]])
        slots = torch.cat([self.slots[r], g["slots"]])
        d = self._buffers(M)
        prev = (torch.cat([self.prev_ids[r], g["prev"]]), self.prev_ids[r], self.q_len[r]) if self.bracket else None
        self._layers(M, d, ids, pos, slots, [self._decode_group(B), g], prev=prev)
        self._remember_last(seqs, g)
        self._lm_head(d["resid"][r], self.logits[r])
        self._sample_commit(B)
        ops.ring_advance(self.ring_counter)
        self._prefill_sample(seqs, d["resid"], qs, ql, ring_row)
        self._keep_logits(seqs, d["resid"], qs)
