"""KV-cache layout arithmetic (host side), thin over the C ABI.

Mirrors src/metal/step_kv/mod.rs:65-100 and src/metal/step_kernel/mod.rs:511-587 of the
reference: slot-major regions [slot][K: Hkv*hd | V: Hkv*hd], one region per layer,
global layers linear (+8 pad slots), sliding layers a power-of-two ring.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List

from . import capi

N_LAYERS = 30
FULL_LAYERS = (5, 11, 17, 23, 29)  # src/metal/step_kernel/mod.rs:127
CANVAS = 256
STEP_NQ_HEADS = 16
SLIDING_WINDOW = 1024
KV_RING_SLOTS = 4096  # DGQ_KV_RING default


def kv_row_bytes(head_dim: int, kv_dtype: int = capi.DG_F16) -> int:
    return capi.load().dg_kv_row_bytes(head_dim, kv_dtype)


def kv_region_bytes(n_kv_heads: int, head_dim: int, slots: int, kv_dtype: int = capi.DG_F16) -> int:
    return capi.load().dg_kv_region_bytes(n_kv_heads, head_dim, slots, kv_dtype)


def kv_slot(kv_ring_mask: int, pos: int) -> int:
    return capi.load().dg_kv_slot(kv_ring_mask, pos)


def layer_kv_slots(is_full: bool, max_seq: int, ring_slots: int = KV_RING_SLOTS) -> int:
    return capi.load().dg_layer_kv_slots(1 if is_full else 0, max_seq, ring_slots)


@dataclass
class LayerKv:
    layer: int
    is_full: bool
    head_dim: int
    n_kv_heads: int
    slots: int
    kv_ring_mask: int
    kv_region: int  # byte offset

    def offsets(self) -> capi.LayerOffsets:
        lo = capi.LayerOffsets()
        lo.kv_region = self.kv_region
        lo.head_dim = self.head_dim
        lo.n_kv_heads = self.n_kv_heads
        lo.is_full = 1 if self.is_full else 0
        lo.kv_ring_mask = self.kv_ring_mask
        return lo


def build_layout(max_seq: int, kv_dtype: int = capi.DG_F16, ring_slots: int = KV_RING_SLOTS) -> List[LayerKv]:
    """Per-layer KV regions of the 30-layer model, concatenated in one buffer."""
    layers, off = [], 0
    for i in range(N_LAYERS):
        full = i in FULL_LAYERS
        hd, nkv = (512, 2) if full else (256, 8)
        slots = layer_kv_slots(full, max_seq, ring_slots)
        layers.append(LayerKv(i, full, hd, nkv, slots, 0 if full else slots - 1, off))
        off += kv_region_bytes(nkv, hd, slots, kv_dtype)
    return layers


def kv_cache_total_bytes(layers: List[LayerKv], kv_dtype: int = capi.DG_F16) -> int:
    return sum(kv_region_bytes(l.n_kv_heads, l.head_dim, l.slots, kv_dtype) for l in layers)
