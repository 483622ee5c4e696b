"""KV-cache layout arithmetic (host side), thin over the C ABI.

Mirrors src/metal/step_kv/mod.rs:65-100 and src/metal/step_kernel/mod.rs:511-587 of the
reference: slot-major regions [slot][K: Hkv*hd | V: Hkv*hd], one region per layer,
global layers linear (+8 pad slots), sliding layers a power-of-two ring.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Sequence

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


# ---------------------------------------------------------------------------------------
# snapshots and the live-KV fingerprint (src/metal/step_kv/mod.rs:108-151,
# src/metal/step_kernel/runtime.rs:118-148), on a device buffer in either layout
# ---------------------------------------------------------------------------------------

def kv_layers(layers: Sequence[LayerKv], kv_dtype: int = capi.DG_F16, layout: str = "reference"):
    """The dg_kv_layer array the snapshot calls take."""
    lib = capi.load()
    arr = (capi.KvLayer * len(layers))()
    for a, l in zip(arr, layers):
        a.kv_region_bytes, a.n_kv_heads, a.head_dim = l.kv_region, l.n_kv_heads, l.head_dim
        a.slots, a.kv_ring_mask, a.kv_dtype = l.slots, l.kv_ring_mask, kv_dtype
        if layout == "reference":
            lib.dg_kv_layer_reference_layout(C.byref(a))
        elif layout == "head_major":
            lib.dg_kv_layer_head_major_layout(C.byref(a))
        else:
            raise ValueError(layout)
    return arr


def snapshot_bytes(arr, kv_len: int) -> int:
    n = C.c_uint64(0)
    capi.check(capi.load().dg_kv_snapshot_bytes(arr, len(arr), kv_len, C.byref(n), None))
    return n.value


def _stream() -> int:
    import torch
    return torch.cuda.current_stream().cuda_stream


def gather_kv_prefix(buf, arr, kv_len: int):
    """Compact blob (device uint8 tensor) of the live [0, kv_len) KV of every layer."""
    import torch
    blob = torch.empty(max(snapshot_bytes(arr, kv_len), 16), dtype=torch.uint8, device="cuda")
    capi.check(capi.load().dg_kv_snapshot_gather(buf.data_ptr(), arr, len(arr), kv_len, blob.data_ptr(), blob.numel(),
                                                 _stream()))
    return blob[:snapshot_bytes(arr, kv_len)]


def scatter_kv_prefix(buf, arr, kv_len: int, blob) -> None:
    capi.check(capi.load().dg_kv_snapshot_scatter(buf.data_ptr(), arr, len(arr), kv_len, blob.data_ptr(), blob.numel(),
                                                  _stream()))


def live_kv_fnv(buf, arr, kv_len: int, seed_hash: int, window: int = SLIDING_WINDOW) -> int:
    """FNV-1a over the readable KV state: the live stream is gathered on the device, copied to the host, hashed there."""
    import torch
    lib = capi.load()
    n = C.c_uint64(0)
    capi.check(lib.dg_kv_live_bytes(arr, len(arr), kv_len, window, C.byref(n)))
    dev = torch.empty(max(n.value, 16), dtype=torch.uint8, device="cuda")
    capi.check(lib.dg_kv_live_gather(buf.data_ptr(), arr, len(arr), kv_len, window, dev.data_ptr(), dev.numel(), _stream()))
    host = dev[:n.value].cpu().numpy()
    return int(lib.dg_fnv1a64(host.ctypes.data_as(C.c_void_p) if host.size else None, host.size, seed_hash))
