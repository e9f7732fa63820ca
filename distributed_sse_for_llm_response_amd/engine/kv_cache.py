"""Paged KV cache (HBM) and its host-side block allocator.

Layout (one tensor per K and V for all layers, so a layer's cache is a contiguous view):

* K: [L, blocks, Hkv_local, 32, 128] bf16 — one key row = 256 contiguous bytes
* V: [L, blocks, Hkv_local, 128, 32] bf16 — transposed pages, tokens permuted by ``vperm``

Pages are 32 tokens.  At TP=1 Mistral-7B needs 128 KiB per token, so 100 GB of the 288 GB HBM holds
~780k tokens (about 190 sequences of 4k context per GPU).  The cache is zero-initialised so keys
past a sequence's end inside its last page are finite (they are masked, but 0·NaN would poison PV).
"""
from __future__ import annotations

import torch

PAGE = 32


class KVCache:
    def __init__(self, num_layers: int, num_blocks: int, nkv: int, device, dtype=torch.bfloat16):
        self.num_layers, self.num_blocks, self.nkv = num_layers, num_blocks, nkv
        self.k = torch.zeros(num_layers, num_blocks, nkv, PAGE, 128, device=device, dtype=dtype)
        self.v = torch.zeros(num_layers, num_blocks, nkv, 128, PAGE, device=device, dtype=dtype)

    @staticmethod
    def bytes_per_block(num_layers: int, nkv: int) -> int:
        return 2 * num_layers * nkv * PAGE * 128 * 2

    @classmethod
    def blocks_for_budget(cls, budget_bytes: int, num_layers: int, nkv: int) -> int:
        return max(1, budget_bytes // cls.bytes_per_block(num_layers, nkv))


class BlockAllocator:
    """Free-list allocator of KV pages (host side; the device only sees block tables)."""

    def __init__(self, num_blocks: int):
        self.num_blocks = num_blocks
        self._free = list(range(num_blocks - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def can_allocate(self, n: int) -> bool:
        return n <= len(self._free)

    def allocate(self, n: int) -> list:
        if n > len(self._free):
            raise MemoryError(f"KV cache exhausted: need {n} blocks, {len(self._free)} free")
        out = [self._free.pop() for _ in range(n)]
        return out

    def free(self, blocks) -> None:
        self._free.extend(reversed(list(blocks)))


def blocks_needed(num_tokens: int) -> int:
    return (num_tokens + PAGE - 1) // PAGE


class LatentKVCache:
    """Paged cache of latent-attention layers: one row [normed latent (rank) | rotated shared key part (rot)] per
    token, nothing per head.  One tensor per attention layer, [blocks, PAGE, rank + rot] in the engine's element
    type; layers index it with the same block tables (a page id means the same page in every layer), so the host
    allocator and the block tables are the ones the dense KV cache uses.  ``widths`` maps layer index -> rank + rot
    (layers without attention have no entry)."""

    def __init__(self, widths: dict, num_blocks: int, device, dtype=torch.bfloat16, transposed: dict | None = None):
        self.num_blocks = num_blocks
        self.layers = {li: torch.zeros(num_blocks, PAGE, w, device=device, dtype=dtype) for li, w in widths.items()}
        # layers on the MFMA attention form also keep the latent in transposed pages [blocks, rank, PAGE] (tokens
        # permuted inside a page, ops/layers_reference.py vt_position): its value operand is then one 16-byte load per
        # lane, as with the dense cache's V pages.  `transposed` maps layer index -> rank for those layers.
        self.vt = {li: torch.zeros(num_blocks, rk, PAGE, device=device, dtype=dtype)
                   for li, rk in (transposed or {}).items()}

    def __getitem__(self, li: int) -> torch.Tensor:
        return self.layers[li]

    @staticmethod
    def bytes_per_block(widths: dict, elem_bytes: int = 2) -> int:
        return max(1, sum(widths.values()) * PAGE * elem_bytes)


class RecurrentStateCache:
    """Per-sequence state of recurrent layers, indexed by the engine's decode slot (a sequence owns one slot from
    admission to its end, so the slot is also its state slot): per layer the fp32 recurrence state [slots, C] and the
    convolution tail [slots, taps - 1, C] (the last taps - 1 inputs).  Nothing is cleared when a slot changes hands:
    the kernels start a sequence whose first row is position 0 from zeros.  ``shapes`` maps layer index -> (C, taps)."""

    def __init__(self, shapes: dict, num_slots: int, device):
        self.num_slots = num_slots
        self.state = {li: torch.zeros(num_slots, c, device=device, dtype=torch.float32) for li, (c, _) in shapes.items()}
        self.tail = {li: torch.zeros(num_slots, k - 1, c, device=device, dtype=torch.float32)
                     for li, (c, k) in shapes.items()}

    def move(self, src_idx: torch.Tensor, dst_idx: torch.Tensor) -> None:
        """State of slot src[i] -> slot dst[i] (gathered before it is scattered, so swaps work)."""
        for group in (self.state, self.tail):
            for t in group.values():
                t.index_copy_(0, dst_idx, t.index_select(0, src_idx))


class PagedKVCache:
    """Paged keys and values of softmax-attention layers with any head widths: per attention run one key tensor
    [blocks, PAGE, G, D] and one value tensor [blocks, PAGE, G, V] in the engine's element type, indexed with the same
    block tables and allocator as the other caches (a page id means the same page in every run).  ``shapes`` maps a
    run's key -> (G, D, V); a layer that runs several times (a looped span) has one entry per run."""

    def __init__(self, shapes: dict, num_blocks: int, device, dtype=torch.bfloat16, transposed=()):
        self.num_blocks = num_blocks
        self.k = {r: torch.zeros(num_blocks, PAGE, g, d, device=device, dtype=dtype) for r, (g, d, _) in shapes.items()}
        self.v = {r: torch.zeros(num_blocks, PAGE, g, v, device=device, dtype=dtype) for r, (g, _, v) in shapes.items()}
        # runs on the MFMA attention form also keep the values in transposed pages [blocks, G, V, PAGE] (tokens
        # permuted inside a page, ops/layers_reference.py vt_position): the prompt kernel's value operand is then one
        # 16-byte load per lane; decode steps read the row-major pages
        self.vt = {r: torch.zeros(num_blocks, shapes[r][0], shapes[r][2], PAGE, device=device, dtype=dtype)
                   for r in transposed}

    @staticmethod
    def bytes_per_block(shapes: dict, elem_bytes: int = 2) -> int:
        return max(1, sum(g * (d + v) for g, d, v in shapes.values()) * PAGE * elem_bytes)


class MatrixStateCache(RecurrentStateCache):
    """Per-sequence state of matrix-state mixers, indexed by the decode slot like RecurrentStateCache: per run the
    fp32 state [slots, H, D, V] and, for mixers with a short convolution in front, its tail [slots, taps - 1, C].
    ``shapes`` maps a run's key -> ((H, D, V), C, taps) with C = 0 for mixers without a convolution."""

    def __init__(self, shapes: dict, num_slots: int, device):
        self.num_slots = num_slots
        self.state = {r: torch.zeros(num_slots, *s, device=device, dtype=torch.float32) for r, (s, _, _) in shapes.items()}
        self.tail = {r: torch.zeros(num_slots, k - 1, c, device=device, dtype=torch.float32)
                     for r, (_, c, k) in shapes.items() if c > 0 and k > 1}


class MixedKVCache:
    """The paged caches of a design that has latent-attention runs AND key/value attention runs: a LatentKVCache for
    the former and a PagedKVCache for the latter, over the same page ids, block tables and allocator (a page id means
    the same page in every run of either kind)."""

    def __init__(self, latent_widths: dict, kv_shapes: dict, num_blocks: int, device, dtype=torch.bfloat16,
                 latent_transposed: dict | None = None, kv_transposed=()):
        self.num_blocks = num_blocks
        self.latent = LatentKVCache(latent_widths, num_blocks, device, dtype, transposed=latent_transposed)
        self.paged = PagedKVCache(kv_shapes, num_blocks, device, dtype, transposed=kv_transposed)


class ConvTailCache(RecurrentStateCache):
    """Per-sequence tails of short causal convolutions that have no recurrence behind them, indexed by the decode slot
    like RecurrentStateCache: per key the last taps - 1 inputs [slots, taps - 1, C] in fp32.  ``shapes`` maps a key
    (for instance (run, sublayer)) -> (C, taps); keys with taps <= 1 hold nothing."""

    def __init__(self, shapes: dict, num_slots: int, device):
        self.num_slots = num_slots
        self.state = {}
        self.tail = {k: torch.zeros(num_slots, taps - 1, c, device=device, dtype=torch.float32)
                     for k, (c, taps) in shapes.items() if taps > 1}
