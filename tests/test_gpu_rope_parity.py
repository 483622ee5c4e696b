"""GPU parity of the producer (per-head RMSNorm + RoPE + KV-cache write) against the CPU oracle,
through the C ABI.  The four reference cases and their tolerances are qk_rope_kv/mod.rs:437-489
(max_tol 1e-2 / 2e-2, cosine >= 0.9999 / 0.999).  At layer-sized shapes and long prefixes the
comparison allows one bf16 / f16 storage step on top: the angle pos * theta^(-2d/hd) is an fp32
product whose last-place differences between two math libraries grow with pos."""
import ctypes as C

import numpy as np
import pytest

from diffgemma_amd import attention as A
from diffgemma_amd import capi, qk_rope_kv as QR, rounding as R
from helpers import assert_oracle, cosine, max_abs_diff

pytestmark = pytest.mark.gpu


def reference_cpu(po, f):
    """The reference's test wrapper (qk_rope_kv/mod.rs:238-262): inputs -> bf16 by truncation, run the
    CPU twin, q/k -> bf16 (its f32_to_bf16_bits truncates), cache -> f16 by truncation."""
    tr = lambda x: R.bf16_bits_to_f32(R.f32_to_bf16_bits_trunc(x))
    d = po.make_rope_desc(f.canvas, f.n_q_heads, f.n_kv_heads, f.head_dim, f.kv_len, is_full=f.is_full,
                          v_from_k=(f.v_proj == 0), kv_write_end=f.kv_write_end, kv_ring_mask=f.kv_ring_mask)
    region = f.kvcache[f.kv_region // 2:]
    q, k, kvc = po.qk_rope_kv_f32(d, tr(f.q), tr(f.k), tr(f.v), R.f16_bits_to_f32(R.f32_to_f16_bits_trunc(region)),
                                  tr(f.q_norm_w), tr(f.k_norm_w))
    full = np.concatenate([f.kvcache[:f.kv_region // 2], R.f16_bits_to_f32(R.f32_to_f16_bits_trunc(kvc))])
    return tr(q), tr(k), full


CASES = {"tiny": (QR.tiny_fixture, 1e-2, 0.9999), "full_layer": (QR.full_layer_fixture, 1e-2, 0.9999),
         "full_attn_v_alias": (QR.full_attn_v_alias_fixture, 1e-2, 0.9999),
         "full_hd512_v_alias": (QR.full_hd512_v_alias_fixture, 2e-2, 0.999)}


@pytest.mark.parametrize("name", list(CASES))
def test_reference_matrix(gpu_ready, po, name):
    make, tol, cs = CASES[name]
    f = make()
    q, k, kvc = reference_cpu(po, f)
    assert_oracle(QR.gpu(f), QR.pack_out(q, k, kvc, f), tol, cs)


def storage_tolerance(ref, ulp_bits):
    """One storage step of the value's own magnitude plus 1e-2 (the reference's absolute bound)."""
    return 1e-2 + np.abs(ref) * 2.0 ** (-ulp_bits)


@pytest.mark.parametrize("shape", [
    # canvas, Hq, Hkv, hd, kv_len, is_full, v_proj, ring mask
    (256, 16, 8, 256, 4096, False, 1, 2047),      # sliding layer on its ring
    (256, 16, 2, 512, 32768, True, 0, 0),         # global layer at the 32k prefix, V aliases k
    (64, 16, 2, 512, 131072, True, 1, 0),         # long context, shrunken canvas
    (37, 8, 4, 128, 333, False, 1, 0),
])
def test_layer_shapes(gpu_ready, po, shape):
    canvas, nq, nkv, hd, kv_len, is_full, v_proj, ring = shape
    f = QR.random_fixture(canvas, nq, nkv, hd, kv_len, is_full=is_full, v_proj=v_proj, seed=hd + canvas,
                          kv_ring_mask=ring)
    q, k, kvc = reference_cpu(po, f)
    rig = QR.RopeRig(f)
    rig.run_dispatch()
    gq, gk, gkv = rig.read()
    assert np.isfinite(gq).all() and np.isfinite(gkv).all()
    assert np.all(np.abs(gq - q) <= storage_tolerance(q, 7)) and cosine(gq, q) >= 0.9999
    assert np.all(np.abs(gk - k) <= storage_tolerance(k, 7)) and cosine(gk, k) >= 0.9999
    assert np.all(np.abs(gkv - kvc) <= storage_tolerance(kvc, 10)) and cosine(gkv, kvc) >= 0.9999
    # rows the launch does not own are bit-identical to what was there
    want_pack, got_pack = QR.pack_out(q, k, kvc, f), QR.pack_out(gq, gk, gkv, f)
    assert got_pack.shape == want_pack.shape
    ds = rig.buf_dbg.cpu().numpy()
    assert ds[0] == 0, f"debug status {ds}"


def _random_case(seed):
    rng = np.random.default_rng(5000 + seed)
    hd = int(rng.choice([32, 64, 128, 256, 512]))
    nkv = int(rng.choice([1, 2, 4, 8]))
    nq = nkv * int(rng.choice([1, 2, 4, 8]))
    canvas = int(rng.choice([1, 3, 16, 37, 64, 256]))
    ring = int(rng.choice([0, 0, 255, 1023, 2047]))
    kv_len = int(rng.choice([0, 1, 100, 1000, 5000, 40000])) if ring == 0 else int(rng.choice([0, 100, 1000, 70000]))
    canvas = min(canvas, ring + 1) if ring else canvas
    is_full, v_proj = bool(rng.integers(0, 2)), int(rng.integers(0, 2))
    kv_write_end = 0xFFFFFFFF if rng.random() < 0.6 else kv_len + int(rng.integers(0, canvas + 1))
    return QR.random_fixture(canvas, nq, nkv, hd, kv_len, is_full=is_full, v_proj=v_proj, seed=seed, kv_ring_mask=ring,
                             kv_write_end=kv_write_end, kv_region=int(rng.choice([0, 4096])))


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes(gpu_ready, po, seed):
    """Seeded sweep over head_dim, head counts, ragged canvases, rings, prefixes, both rotations, V aliasing and
    write suppression, through both reference-shaped entries (host and device StepParams)."""
    f = _random_case(seed)
    q, k, kvc = reference_cpu(po, f)
    for dev in (False, True):
        rig = QR.RopeRig(f)
        (rig.run_dispatch_dev if dev else rig.run_dispatch)()
        gq, gk, gkv = rig.read()
        assert np.isfinite(gq).all() and np.isfinite(gkv).all()
        assert np.all(np.abs(gq - q) <= storage_tolerance(q, 7)) and np.all(np.abs(gk - k) <= storage_tolerance(k, 7))
        assert np.all(np.abs(gkv - kvc) <= storage_tolerance(kvc, 10))
        assert rig.buf_dbg.cpu().numpy()[0] == 0


def test_debug_status_names_the_producer(gpu_ready):
    """A NaN in one head's input makes that head's 1/rms non-finite; the record the kernel leaves is the
    reference's: DbgErrNonFinite = 4 in DbgKernelQkRopeKv = 25, value = the canvas row
    (qk_rope_kv.metal:77; decoded by src/metal/debug_status.rs:33-75).  (An infinity would not do: the sum of
    squares is then +inf and 1/sqrt(+inf) = 0 is finite, in the reference too.)"""
    f = QR.random_fixture(8, 4, 2, 64, 40, is_full=False, v_proj=1, seed=3)
    clean = QR.RopeRig(f)
    clean.run_dispatch()
    assert clean.buf_dbg.cpu().numpy().view(np.uint32)[0] == 0
    tok, head = 5, 3
    f.q[(tok * f.n_q_heads + head) * f.head_dim + 7] = np.float32(np.nan)
    bad = QR.RopeRig(f)
    bad.run_dispatch()
    code, kernel_id, tg_id, value = (int(x) for x in bad.buf_dbg.cpu().numpy().view(np.uint32))
    assert (code, kernel_id) == (4, 25) == (capi.DG_DBG_ERR_NONFINITE, capi.DG_DBG_KERNEL_QK_ROPE_KV)
    assert value == tok and tg_id == (tok << 16) | head


def test_write_suppression_and_untouched_rows(gpu_ready, po):
    """kv_write_end (qk_rope_kv.metal:56-60): pad rows are normed and rotated in place but never reach
    the cache; every slot the launch does not own keeps its bits."""
    f = QR.random_fixture(8, 16, 8, 256, 1020, is_full=False, v_proj=1, seed=9, kv_ring_mask=1023, kv_write_end=1024,
                          kv_region=4096)
    f.kvcache[:] = 0.5
    rig = QR.RopeRig(f)
    before = rig.buf_kv.cpu().numpy().copy()
    rig.run_dispatch()
    after = rig.buf_kv.cpu().numpy()
    row = 2 * f.n_kv_heads * f.head_dim
    changed = np.flatnonzero((before != after).reshape(-1)) // 1
    slots = {int((i - f.kv_region // 2) // row) for i in changed}
    assert slots == {1020, 1021, 1022, 1023}                 # positions 1024.. would wrap onto slots 0..3
    q, k, kvc = reference_cpu(po, f)
    gq, gk, gkv = rig.read()
    assert max_abs_diff(gq, q) <= 2e-2 and max_abs_diff(gkv, kvc) <= 1e-2   # suppressed rows still rotate q


@pytest.mark.parametrize("name", ["tiny", "full_hd512_v_alias"])
def test_dispatch_with_device_step_params_equals_the_host_one(gpu_ready, name):
    """dg_qk_rope_kv_dispatch_dev reads kv_len and kv_write_end from a device StepParams when the kernel runs
    (the reference binds StepParams as a device buffer, qk_rope_kv.metal:30-38): same bits as the host-P entry,
    including a kv_write_end that suppresses part of the canvas."""
    f = CASES[name][0]()
    a, b = QR.RopeRig(f), QR.RopeRig(f)
    a.run_dispatch()
    b.run_dispatch_dev()
    for x, y in zip(a.read(), b.read()):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))
    f2 = QR.random_fixture(8, 16, 8, 256, 1020, is_full=False, v_proj=1, seed=9, kv_ring_mask=1023, kv_write_end=1024,
                           kv_region=4096)
    a, b = QR.RopeRig(f2), QR.RopeRig(f2)
    a.run_dispatch()
    b.run_dispatch_dev()
    for x, y in zip(a.read(), b.read()):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))
    assert b.buf_dbg.cpu().numpy()[0] == 0


def test_general_entry_bf16_head_major_cache(gpu_ready, po):
    """dg_qk_rope_kv with the cache the benchmark's attention reads: bf16, two planes [Hkv][t_cap][d]."""
    import torch
    canvas, nq, nkv, hd, kv_len = 32, 16, 2, 512, 480
    t_cap = kv_len + canvas
    f = QR.random_fixture(canvas, nq, nkv, hd, kv_len, is_full=True, v_proj=0, seed=12)
    tr = lambda x: R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(x))
    d = QR.rope_desc(f, kv_dtype=capi.DG_BF16, truncate=False, layout="head_major", t_cap=t_cap)
    bq, bk = A.to_device_bits(R.f32_to_bf16_bits_rne(f.q)), A.to_device_bits(R.f32_to_bf16_bits_rne(f.k))
    bqw, bkw = A.to_device_bits(R.f32_to_bf16_bits_rne(f.q_norm_w)), A.to_device_bits(R.f32_to_bf16_bits_rne(f.k_norm_w))
    cache = torch.zeros(2 * nkv * t_cap * hd, dtype=torch.int16, device="cuda")
    capi.check(capi.load().dg_qk_rope_kv(C.byref(d), bq.data_ptr(), bk.data_ptr(), None, cache.data_ptr(),
                                         bqw.data_ptr(), bkw.data_ptr(), None, A.stream_handle()))
    torch.cuda.synchronize()
    od = po.make_rope_desc(canvas, nq, nkv, hd, kv_len, is_full=True, v_from_k=True, layout="head_major", t_cap=t_cap)
    q, k, kvc = po.qk_rope_kv_f32(od, tr(f.q), tr(f.k), f.v, np.zeros(2 * nkv * t_cap * hd, np.float32),
                                  tr(f.q_norm_w), tr(f.k_norm_w))
    got = R.bf16_bits_to_f32(cache.cpu().numpy().view(np.uint16))
    assert np.all(np.abs(got - kvc) <= storage_tolerance(kvc, 7)) and cosine(got, kvc) >= 0.9999
    assert np.array_equal(R.bf16_bits_to_f32(bk.cpu().numpy().view(np.uint16)), tr(f.k))    # raw k untouched
    gq = R.bf16_bits_to_f32(bq.cpu().numpy().view(np.uint16))
    assert np.all(np.abs(gq - q) <= storage_tolerance(q, 7))


def test_producer_then_attention(gpu_ready, po):
    """The two kernels back to back, as a denoise step runs them (enc.rs:852-856): the canvas rows the
    producer writes are the rows attention reads."""
    import torch
    canvas, nq, nkv, hd, kv_len = 64, 16, 2, 512, 960
    f = QR.random_fixture(canvas, nq, nkv, hd, kv_len, is_full=True, v_proj=0, seed=21)
    rng = np.random.default_rng(5)
    prefix = rng.standard_normal((kv_len, 2 * nkv * hd)).astype(np.float32)
    prefix /= np.sqrt((prefix.reshape(kv_len, 2 * nkv, hd) ** 2).mean(-1, keepdims=True)).repeat(hd, -1).reshape(kv_len, -1)
    f.kvcache[:kv_len * 2 * nkv * hd] = prefix.ravel()
    rig = QR.RopeRig(f)
    rig.run_dispatch()
    out = torch.zeros(canvas * nq * hd, dtype=torch.float32, device="cuda")
    lse = torch.zeros(canvas * nq, dtype=torch.float32, device="cuda")
    ad = A.make_desc(canvas, nq, nkv, hd, kv_len, q_dtype=capi.DG_BF16, kv_dtype=capi.DG_F16, out_dtype=capi.DG_F32)
    A.forward(ad, rig.buf_q, rig.buf_kv, out, lse, A.alloc_workspace(ad))
    torch.cuda.synchronize()
    q, k, kvc = reference_cpu(po, f)
    gq, gk, gkv = rig.read()
    assert np.all(np.abs(gq - q) <= storage_tolerance(q, 7)) and np.all(np.abs(gkv - kvc) <= storage_tolerance(kvc, 10))
    # attention is compared on identical inputs (what the producer left on the device): with scores
    # spread over tens of units, one storage step in a single q element moves an output row by more
    # than the attention tolerance, on either side alike
    ref, ref_lse = po.attention_f32(po.make_desc(canvas, nq, nkv, hd, kv_len), gq, gkv)
    got = out.cpu().numpy().reshape(ref.shape)
    assert max_abs_diff(got, ref) <= 2e-2 and float(np.mean(np.abs(got - ref))) <= 2e-3
    rel = np.abs(lse.cpu().numpy().reshape(ref_lse.shape) - ref_lse) / np.maximum(np.abs(ref_lse), 1e-6)
    assert rel.max() <= 1e-3


def test_rejects_bad_arguments(gpu_ready):
    f = QR.tiny_fixture()
    d = QR.rope_desc(f)
    lib = capi.load()
    assert lib.dg_qk_rope_kv(C.byref(d), None, None, None, None, None, None, None, None) == capi.DG_ERR_NULL
    rig = QR.RopeRig(f)
    args = (rig.buf_q.data_ptr(), rig.buf_k.data_ptr(), rig.buf_v.data_ptr(), rig.buf_kv.data_ptr(),
            rig.buf_blob.data_ptr(), rig.buf_blob.data_ptr() + 2 * f.head_dim, None, A.stream_handle())
    d.head_dim = 48
    assert lib.dg_qk_rope_kv(C.byref(d), *args) == capi.DG_ERR_SHAPE
    d = QR.rope_desc(f)
    d.kv_dtype = capi.DG_F32
    assert lib.dg_qk_rope_kv(C.byref(d), *args) == capi.DG_ERR_DTYPE
    d = QR.rope_desc(f)
    d.kv_ring_mask = 5
    assert lib.dg_qk_rope_kv(C.byref(d), *args) == capi.DG_ERR_LAYOUT


def test_two_layer_step_in_a_hip_graph(gpu_ready, po):
    """Producer + attention of a sliding (ring) and a global layer captured once and replayed with
    regenerated canvas projections: every replay equals the eager result for the same inputs."""
    import torch
    canvas, nq, kv_len, ring = 64, 16, 3000, 2048
    lib = capi.load()
    gen = torch.Generator(device="cuda")
    layers = []
    for full in (False, True):
        hd, nkv = (512, 2) if full else (256, 8)
        slots = kv_len + canvas if full else ring
        mask = 0 if full else ring - 1
        f = QR.random_fixture(1, nq, nkv, hd, kv_len, is_full=full, v_proj=0 if full else 1, seed=3, kv_ring_mask=mask)
        f.canvas = canvas
        rd = QR.rope_desc(f, kv_dtype=capi.DG_BF16, truncate=False, layout="head_major", t_cap=slots)
        ad = A.make_desc(canvas, nq, nkv, hd, kv_len, window=0 if full else 1024, kv_ring_mask=mask,
                         q_dtype=capi.DG_BF16, kv_dtype=capi.DG_BF16, out_dtype=capi.DG_BF16, layout="head_major",
                         t_cap=slots)
        gen.manual_seed(11)
        cache = torch.randn(2 * nkv * slots * hd, device="cuda", generator=gen).to(torch.bfloat16).view(torch.int16)
        layers.append(dict(rd=rd, ad=ad, cache=cache, ws=A.alloc_workspace(ad),
                           q=torch.empty(canvas * nq * hd, dtype=torch.int16, device="cuda"),
                           k=torch.empty(canvas * nkv * hd, dtype=torch.int16, device="cuda"),
                           v=torch.empty(canvas * nkv * hd, dtype=torch.int16, device="cuda"),
                           qw=A.to_device_bits(R.f32_to_bf16_bits_rne(f.q_norm_w)),
                           kw=A.to_device_bits(R.f32_to_bf16_bits_rne(f.k_norm_w)),
                           out=torch.zeros(canvas * nq * hd, dtype=torch.int16, device="cuda")))

    def regenerate(it):
        gen.manual_seed(100 + it)
        for lay in layers:
            for n in ("q", "k", "v"):
                lay[n].copy_(torch.randn(lay[n].numel(), device="cuda", generator=gen).to(torch.bfloat16).view(torch.int16))

    def encode():
        for lay in layers:
            capi.check(lib.dg_qk_rope_kv(C.byref(lay["rd"]), lay["q"].data_ptr(), lay["k"].data_ptr(), lay["v"].data_ptr(),
                                         lay["cache"].data_ptr(), lay["qw"].data_ptr(), lay["kw"].data_ptr(), None,
                                         A.stream_handle()))
            A.forward(lay["ad"], lay["q"], lay["cache"], lay["out"], None, lay["ws"])

    regenerate(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        encode()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    regenerate(0)
    with torch.cuda.graph(g):
        encode()
    for it in range(1, 4):
        regenerate(it)
        encode()                                   # eager, on the same inputs
        torch.cuda.synchronize()
        want = [lay["out"].clone() for lay in layers]
        regenerate(it)                             # the producer rotated q in place: restore the inputs
        for lay in layers:
            lay["out"].zero_()
        g.replay()
        torch.cuda.synchronize()
        for w, lay in zip(want, layers):
            assert torch.equal(w, lay["out"]), it
            assert np.isfinite(R.bf16_bits_to_f32(lay["out"].cpu().numpy().view(np.uint16))).all()
