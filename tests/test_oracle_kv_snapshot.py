"""Pins the KV-snapshot restatements (oracle/pyoracle.py: kv_gather_prefix, kv_scatter_prefix,
kv_live_stream, fnv1a64) and checks the host side of the C ABI against them (sizes, offsets,
validation, the host hash); no device work here."""
import ctypes as C

import numpy as np
import pytest

from diffgemma_amd import capi, step_kv


def test_fnv1a64_published_vectors(po):
    # the FNV authors' own test vectors for the 64-bit FNV-1a
    assert po.fnv1a64(b"") == 0xcbf29ce484222325
    assert po.fnv1a64(b"a") == 0xaf63dc4c8601ec8c
    assert po.fnv1a64(b"foobar") == 0x85944171f73967e8
    # continuing a hash is hashing the concatenation (how live_kv_fnv chains onto the token hash)
    assert po.fnv1a64(b"bar", po.fnv1a64(b"foo")) == po.fnv1a64(b"foobar")
    lib = capi.load()
    for data in (b"", b"a", b"foobar", bytes(range(256)) * 3):
        buf = np.frombuffer(data, dtype=np.uint8)
        got = lib.dg_fnv1a64(buf.ctypes.data_as(C.c_void_p) if buf.size else None, buf.size, po.FNV_OFFSET_BASIS)
        assert got == po.fnv1a64(data)


def _two_layers():
    """A linear layer (6 slots, 1 head, hd 8) and a ring layer (4 slots, 2 heads, hd 8), f16-sized elements."""
    lin = step_kv.LayerKv(0, True, 8, 1, 6, 0, 0)
    ring = step_kv.LayerKv(1, False, 8, 2, 4, 3, 6 * 2 * 1 * 8 * 2)
    total = ring.kv_region + 4 * 2 * 2 * 8 * 2
    return [lin, ring], total


def test_gather_layout_by_hand(po):
    layers, total = _two_layers()
    cache = (np.arange(total) % 251).astype(np.uint8)
    blob = po.kv_gather_prefix(cache, layers, kv_len=5)
    g0, g1 = 2 * 1 * 8 * 2, 2 * 2 * 8 * 2
    # linear layer: its first 5 slots; ring layer: min(5, 4) = all 4 physical slots as they lie
    assert blob.size == 5 * g0 + 4 * g1
    assert np.array_equal(blob[:5 * g0], cache[:5 * g0])
    assert np.array_equal(blob[5 * g0:], cache[layers[1].kv_region:layers[1].kv_region + 4 * g1])
    assert po.kv_gather_prefix(cache, layers, 0).size == 0
    # scatter is the inverse on the live part and touches nothing else
    other = np.full(total, 0xEE, np.uint8)
    po.kv_scatter_prefix(other, layers, 5, blob)
    assert np.array_equal(other[:5 * g0], cache[:5 * g0]) and (other[5 * g0:6 * g0] == 0xEE).all()
    assert np.array_equal(po.kv_gather_prefix(other, layers, 5), blob)


def test_live_stream_order_by_hand(po):
    layers, total = _two_layers()
    cache = (np.arange(total) % 251).astype(np.uint8)
    g0, g1 = 32, 64
    r = layers[1].kv_region
    # kv_len 6, window 3: linear layer positions 0..5; ring layer positions 3, 4, 5 -> slots 3, 0, 1
    s = po.kv_live_stream(cache, layers, kv_len=6, window=3)
    want = np.concatenate([cache[:6 * g0]] + [cache[r + k * g1:r + (k + 1) * g1] for k in (3, 0, 1)])
    assert np.array_equal(s, want)
    # kv_len below the window: every position so far
    s = po.kv_live_stream(cache, layers, kv_len=2, window=3)
    assert np.array_equal(s, np.concatenate([cache[:2 * g0], cache[r:r + 2 * g1]]))
    assert po.kv_live_fnv(cache, layers, 6, 3, 12345) == po.fnv1a64(want.tobytes(), 12345)


def test_abi_sizes_offsets_and_validation():
    lib = capi.load()
    layers = step_kv.build_layout(40000, capi.DG_F16, ring_slots=4096)
    arr = step_kv.kv_layers(layers, capi.DG_F16, "reference")
    kv_len = 32768
    offs = (C.c_uint64 * len(arr))()
    total = C.c_uint64(0)
    assert lib.dg_kv_snapshot_bytes(arr, len(arr), kv_len, C.byref(total), offs) == capi.DG_OK
    want, off = [], 0
    for l in layers:
        want.append(off)
        off += min(kv_len, l.slots) * 2 * l.n_kv_heads * l.head_dim * 2
    assert list(offs) == want and total.value == off
    # 5 global layers x 32768 x 4 KiB + 25 sliding layers x 4096 x 8 KiB
    assert total.value == 5 * 32768 * 4096 + 25 * 4096 * 8192
    live = C.c_uint64(0)
    assert lib.dg_kv_live_bytes(arr, len(arr), kv_len, 1024, C.byref(live)) == capi.DG_OK
    assert live.value == 5 * 32768 * 4096 + 25 * 1024 * 8192
    assert lib.dg_kv_live_bytes(arr, len(arr), 100, 1024, C.byref(live)) == capi.DG_OK
    assert live.value == 5 * 100 * 4096 + 25 * 100 * 8192
    # a linear layer cannot be asked for more positions than it holds; head_dim must give 16-byte rows
    assert lib.dg_kv_live_bytes(arr, len(arr), 10**6, 1024, C.byref(live)) == capi.DG_ERR_SHAPE
    bad = step_kv.kv_layers(layers[:1], capi.DG_F16, "reference")
    bad[0].head_dim = 4
    assert lib.dg_kv_snapshot_bytes(bad, 1, 10, C.byref(total), None) == capi.DG_ERR_SHAPE
    bad = step_kv.kv_layers(layers[:1], capi.DG_F16, "reference")
    bad[0].kv_ring_mask = 1000
    assert lib.dg_kv_snapshot_bytes(bad, 1, 10, C.byref(total), None) == capi.DG_ERR_LAYOUT
    assert lib.dg_kv_snapshot_bytes(None, 1, 10, C.byref(total), None) == capi.DG_ERR_NULL
    hm = step_kv.kv_layers(layers[5:6], capi.DG_BF16, "head_major")      # a global layer: 2 heads of 512
    l5 = layers[5]
    assert (hm[0].k_tok_stride, hm[0].k_head_stride, hm[0].v_base_off) == (512, l5.slots * 512, 2 * l5.slots * 512)
