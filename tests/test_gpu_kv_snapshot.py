"""GPU parity (bit-exact: byte moves) of the KV snapshot kernel against the numpy restatement of
gather_kv_prefix / scatter_kv_prefix / live_kv_fnv, on the 30-layer model layout, with the cache
held in the reference's slot-major layout and in head-major planes."""
import numpy as np
import pytest

from diffgemma_amd import capi, step_kv

pytestmark = pytest.mark.gpu


def _model(max_seq, ring_slots):
    layers = step_kv.build_layout(max_seq, capi.DG_F16, ring_slots=ring_slots)
    total = step_kv.kv_cache_total_bytes(layers, capi.DG_F16)
    rng = np.random.default_rng(max_seq)
    return layers, rng.integers(0, 256, total, dtype=np.uint8)


def _to_head_major(cache, layers):
    """The same rows with every region re-laid as K plane [Hkv][slots][hd], V plane."""
    out = cache.copy()
    for l in layers:
        n = l.slots * 2 * l.n_kv_heads * l.head_dim * 2
        reg = cache[l.kv_region:l.kv_region + n].view(np.uint16).reshape(l.slots, 2, l.n_kv_heads, l.head_dim)
        out[l.kv_region:l.kv_region + n] = np.ascontiguousarray(reg.transpose(1, 2, 0, 3)).view(np.uint8).reshape(-1)
    return out


@pytest.mark.parametrize("layout", ["reference", "head_major"])
@pytest.mark.parametrize("kv_len", [0, 1, 300, 1024, 3000, 5000])
def test_gather_scatter_and_fingerprint(gpu_ready, po, layout, kv_len):
    import torch
    layers, cache = _model(5000, 2048)          # rings of 2048 slots, global layers of 5008
    dev_bytes = cache if layout == "reference" else _to_head_major(cache, layers)
    buf = torch.from_numpy(dev_bytes).cuda()
    arr = step_kv.kv_layers(layers, capi.DG_F16, layout)
    want = po.kv_gather_prefix(cache, layers, kv_len)
    blob = step_kv.gather_kv_prefix(buf, arr, kv_len)
    torch.cuda.synchronize()
    assert blob.numel() == want.size
    assert np.array_equal(blob.cpu().numpy(), want)          # the blob does not depend on the cache layout

    # restore into a buffer full of 0xEE: the live part comes back, nothing else is touched
    other = torch.full_like(buf, 0xEE)
    step_kv.scatter_kv_prefix(other, arr, kv_len, blob)
    again = step_kv.gather_kv_prefix(other, arr, kv_len)
    torch.cuda.synchronize()
    assert np.array_equal(again.cpu().numpy(), want)
    ref_other = np.full(cache.size, 0xEE, np.uint8)
    po.kv_scatter_prefix(ref_other, layers, kv_len, want)
    got_other = other.cpu().numpy()
    assert np.array_equal(got_other, ref_other if layout == "reference" else _to_head_major(ref_other, layers))

    # the fingerprint: FNV-1a over the readable state, chained onto a seed
    seed = 0x1234_5678_9abc_def0
    assert step_kv.live_kv_fnv(buf, arr, kv_len, seed, window=1024) == po.kv_live_fnv(cache, layers, kv_len, 1024, seed)


def test_bf16_head_major_planes_of_one_layer(gpu_ready, po):
    """A single wide layer with a cache bigger than one launch's grid stride."""
    import torch
    l = step_kv.LayerKv(0, True, 512, 2, 20000, 0, 4096)       # region at a non-zero offset
    total = l.kv_region + 20000 * 2 * 2 * 512 * 2
    cache = np.random.default_rng(5).integers(0, 256, total, dtype=np.uint8)
    arr = step_kv.kv_layers([l], capi.DG_BF16, "head_major")
    buf = torch.from_numpy(_to_head_major(cache, [l])).cuda()
    blob = step_kv.gather_kv_prefix(buf, arr, 19999)
    torch.cuda.synchronize()
    assert np.array_equal(blob.cpu().numpy(), po.kv_gather_prefix(cache, [l], 19999))
