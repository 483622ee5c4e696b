"""Pins the oracle's producer (per-head RMSNorm + RoPE + KV-cache write, reference
src/shaders/attn/cpu.rs:31-145) against what the mathematics fixes, not against a retyped loop:
closed forms on one-hot inputs (which elements are paired, the sign convention, the frequency
exponent and theta), invariants (unit RMS, pair norms, identity at position 0, angle addition),
and the wiring of the whole producer expressed through the separately pinned primitives.
The reference's own tests for this kernel are generator + tolerance comparisons of its CPU and
GPU twins (qk_rope_kv/mod.rs:437-489); it holds no golden vectors for it."""
import numpy as np
import pytest

from diffgemma_amd import qk_rope_kv as QR

RMS_EPS = 1e-6


def angle(pos, d, hd, theta):
    return pos * float(theta) ** (-2.0 * d / hd)       # float64 closed form


# ------------------------------------------------------------------ rms_norm_head
@pytest.mark.parametrize("hd", [32, 64, 256, 512])
def test_rms_norm_unit_rms_and_weight(po, hd):
    rng = np.random.default_rng(hd)
    x = (rng.standard_normal(hd) * 3.0).astype(np.float32)
    y = po.rms_norm_head(x)
    assert abs(np.sqrt(np.mean(y.astype(np.float64) ** 2)) - 1.0) < 1e-5      # unit RMS
    assert np.allclose(y / y[0], x / x[0], rtol=1e-5)                        # a pure rescale
    w = (1.0 + 0.2 * rng.standard_normal(hd)).astype(np.float32)
    assert np.allclose(po.rms_norm_head(x, w), y * w, rtol=2e-6, atol=1e-7)   # weight multiplies element-wise
    # eps enters as mean(x^2) + eps: a zero vector stays zero and finite
    assert np.array_equal(po.rms_norm_head(np.zeros(hd, np.float32)), np.zeros(hd, np.float32))
    tiny = np.full(hd, 1e-4, np.float32)
    want = 1e-4 / np.sqrt(1e-8 + RMS_EPS)
    assert np.allclose(po.rms_norm_head(tiny), want, rtol=1e-5)


# ------------------------------------------------------------------ rotation: closed forms on one-hot inputs
@pytest.mark.parametrize("hd,pos", [(32, 3), (256, 77), (256, 4000)])
def test_split_half_pairs_and_angle(po, hd, pos):
    theta, rot, half = 1.0e4, hd, hd // 2
    for d in (0, 1, 5, half - 1):
        e = np.zeros(hd, np.float32)
        e[d] = 1.0
        y = po.rope(e, rot, hd, theta, pos, proportional=False)
        a = angle(pos, d, hd, theta)
        tol = 2e-6 * max(1.0, a) + 1e-6            # fp32 angle: relative error grows with the angle
        assert abs(y[d] - np.cos(a)) < tol and abs(y[d + half] - np.sin(a)) < tol
        y[d] = y[d + half] = 0.0
        assert not y.any()                          # nothing else moves
        e = np.zeros(hd, np.float32)
        e[d + half] = 1.0
        y = po.rope(e, rot, hd, theta, pos, proportional=False)
        assert abs(y[d] + np.sin(a)) < tol and abs(y[d + half] - np.cos(a)) < tol   # (x0 c - x1 s, x0 s + x1 c)


@pytest.mark.parametrize("hd,pos", [(64, 3), (512, 23), (512, 9000)])
def test_proportional_pairs_rotated_part_and_angle(po, hd, pos):
    theta, rot = 1.0e6, hd // 4
    half_head, half_rot = hd // 2, rot // 2
    for d in (0, 1, half_rot - 1):
        e = np.zeros(hd, np.float32)
        e[d] = 1.0
        y = po.rope(e, rot, hd, theta, pos, proportional=True)
        a = angle(pos, d, hd, theta)                # exponent uses head_dim, not the rotary width
        tol = 2e-6 * max(1.0, a) + 1e-6
        assert abs(y[d] - np.cos(a)) < tol and abs(y[half_head + d] - np.sin(a)) < tol
        y[d] = y[half_head + d] = 0.0
        assert not y.any()
    # everything outside [0, rot/2) and [hd/2, hd/2 + rot/2) is left alone
    rng = np.random.default_rng(1)
    x = rng.standard_normal(hd).astype(np.float32)
    y = po.rope(x, rot, hd, theta, pos, proportional=True)
    keep = np.ones(hd, bool)
    keep[:half_rot] = False
    keep[half_head:half_head + half_rot] = False
    assert np.array_equal(y[keep], x[keep]) and not np.array_equal(y[~keep], x[~keep])


@pytest.mark.parametrize("proportional", [False, True])
def test_rotation_invariants(po, proportional):
    hd = 128
    theta, rot = (1.0e6, hd // 4) if proportional else (1.0e4, hd)
    half_rot, off = rot // 2, hd // 2
    rng = np.random.default_rng(2)
    x = rng.standard_normal(hd).astype(np.float32)
    assert np.array_equal(po.rope(x, rot, hd, theta, 0, proportional), x)           # position 0: identity
    y = po.rope(x, rot, hd, theta, 11, proportional)
    n0 = x[:half_rot] ** 2 + x[off:off + half_rot] ** 2
    n1 = y[:half_rot] ** 2 + y[off:off + half_rot] ** 2
    assert np.allclose(n0, n1, rtol=1e-5)                                            # pair norms preserved
    z = po.rope(po.rope(x, rot, hd, theta, 5, proportional), rot, hd, theta, 6, proportional)
    assert np.allclose(z, y, atol=2e-5)                                              # angles add


# ------------------------------------------------------------------ the whole producer, through the pinned primitives
def run_oracle(po, f, **kw):
    d = po.make_rope_desc(f.canvas, f.n_q_heads, f.n_kv_heads, f.head_dim, f.kv_len, is_full=f.is_full,
                          v_from_k=(f.v_proj == 0), kv_write_end=f.kv_write_end, kv_ring_mask=f.kv_ring_mask, **kw)
    return po.qk_rope_kv_f32(d, f.q, f.k, f.v, f.kvcache, f.q_norm_w, f.k_norm_w)


FIXTURES = [QR.tiny_fixture, QR.full_layer_fixture, QR.full_attn_v_alias_fixture, QR.full_hd512_v_alias_fixture]


@pytest.mark.parametrize("make", FIXTURES)
def test_producer_wiring_on_reference_fixtures(po, make):
    f = make()
    hd, nq, nkv = f.head_dim, f.n_q_heads, f.n_kv_heads
    theta, rot = (1.0e6, hd // 4) if f.is_full else (1.0e4, hd)
    q2, k2, kvc = run_oracle(po, f)
    q0, k0, v0 = f.q.reshape(f.canvas, nq, hd), f.k.reshape(f.canvas, nkv, hd), f.v.reshape(f.canvas, nkv, hd)
    q2, k2 = q2.reshape(f.canvas, nq, hd), k2.reshape(f.canvas, nkv, hd)
    cache = kvc.reshape(-1, 2, nkv, hd)                       # reference layout [slot][K|V][head][d]
    for tok in range(f.canvas):
        pos = f.kv_len + tok
        for h in range(nq):                                   # Q: q weight, rotated at pos, in place
            want = po.rope(po.rms_norm_head(q0[tok, h], f.q_norm_w), rot, hd, theta, pos, f.is_full)
            assert np.array_equal(q2[tok, h], want)
        for h in range(nkv):
            want_k = po.rope(po.rms_norm_head(k0[tok, h], f.k_norm_w), rot, hd, theta, pos, f.is_full)
            assert np.array_equal(cache[pos, 0, h], want_k)   # K row of slot pos
            if f.v_proj == 0:                                 # V aliases the RAW k: k stays untouched
                assert np.array_equal(k2[tok, h], k0[tok, h])
                assert np.array_equal(cache[pos, 1, h], po.rms_norm_head(k0[tok, h]))
            else:
                assert np.array_equal(k2[tok, h], want_k)
                assert np.array_equal(cache[pos, 1, h], po.rms_norm_head(v0[tok, h]))   # V: no weight, no rotation
    assert not cache[:f.kv_len].any()                         # rows of the prefix are not touched


def test_fixture_generators_agree(po):
    """The C++ restatement of the reference's fixtures and the numpy one the GPU tests use."""
    for name, make in [("tiny", QR.tiny_fixture), ("full_layer", QR.full_layer_fixture),
                       ("full_hd512_v_alias", QR.full_hd512_v_alias_fixture)]:
        dims, q, k, v, qw, kw = po.rope_fixture(name)
        f = make()
        assert (dims["canvas"], dims["n_q_heads"], dims["n_kv_heads"], dims["head_dim"], dims["kv_len"]) == \
               (f.canvas, f.n_q_heads, f.n_kv_heads, f.head_dim, f.kv_len)
        for a, b in ((q, f.q), (k, f.k), (v, f.v), (qw, f.q_norm_w), (kw, f.k_norm_w)):
            assert np.allclose(a, b, atol=3e-7)
        # closed-form spot values (qk_rope_kv/mod.rs:89-95,161-167)
    _, q, k, _, qw, kw = po.rope_fixture("full_hd512_v_alias")
    assert abs(q[100] - np.sin(100 * 0.031) * 0.55) < 1e-6 and abs(k[7] - np.cos(7 * 0.029) * 0.48) < 1e-6
    assert abs(qw[500] - 1.05) < 1e-6 and abs(kw[500] - 0.975) < 1e-6


def test_write_suppression_ring_and_layout(po):
    f = QR.random_fixture(6, 4, 2, 64, 29, is_full=False, v_proj=1, seed=3, kv_ring_mask=31, kv_write_end=32)
    f.kvcache[:] = 7.0
    _, _, kvc = run_oracle(po, f)
    cache = kvc.reshape(32, 2, 2, 64)
    written = {(29 + t) & 31 for t in range(6) if 29 + t < 32}             # positions 29, 30, 31 only
    for slot in range(32):
        assert (not np.any(cache[slot] == 7.0)) == (slot in written)
    # positions 32.. would have wrapped onto slots 0.. : suppressed (qk_rope_kv.metal:56-60)
    assert np.all(cache[0] == 7.0)
    # rotation uses the absolute position even though the slot is wrapped
    f2 = QR.random_fixture(2, 4, 2, 64, 40, is_full=False, v_proj=1, seed=3, kv_ring_mask=31)
    _, k2, kvc2 = run_oracle(po, f2)
    want = po.rope(po.rms_norm_head(f2.k.reshape(2, 2, 64)[1, 0], f2.k_norm_w), 64, 64, 1.0e4, 41, False)
    assert np.array_equal(kvc2.reshape(32, 2, 2, 64)[41 & 31, 0, 0], want)
    # head-major planes: same rows, other strides; and they are the rows the attention oracle reads
    f3 = QR.random_fixture(3, 4, 2, 32, 5, is_full=True, v_proj=0, seed=4)
    t_cap = 8
    kv0 = np.zeros(2 * 2 * t_cap * 32, np.float32)
    d = po.make_rope_desc(3, 4, 2, 32, 5, is_full=True, v_from_k=True, layout="head_major", t_cap=t_cap)
    _, _, planes = po.qk_rope_kv_f32(d, f3.q, f3.k, f3.v, kv0, f3.q_norm_w, f3.k_norm_w)
    _, _, ref = run_oracle(po, f3)
    planes = planes.reshape(2, 2, t_cap, 32)
    ref = ref.reshape(8, 2, 2, 32)
    for pos in range(5, 8):
        for h in range(2):
            assert np.array_equal(planes[0, h, pos], ref[pos, 0, h]) and np.array_equal(planes[1, h, pos], ref[pos, 1, h])
    ad = po.make_desc(3, 4, 2, 32, 5, layout="head_major", t_cap=t_cap)
    ar = po.make_desc(3, 4, 2, 32, 5)
    qn = np.ones((3, 4, 32), np.float32)
    planes_full, ref_full = planes.copy(), ref.copy()
    planes_full[:, :, :5] = 0.25
    ref_full[:5] = 0.25
    o1, _ = po.attention_f32(ad, qn, planes_full.ravel())
    o2, _ = po.attention_f32(ar, qn, ref_full.ravel())
    assert np.array_equal(o1, o2)
