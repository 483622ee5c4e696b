"""Pins the CPU oracle (oracle/dg_attn_oracle.cpp) before anything is compared against it.

Each check is chosen so that a plausible mistake in the restatement (dropped scale term,
wrong KV offset, transposed head map, off-by-one in the causal/window bound, wrong ring
map) fails it.  No test here re-types the oracle's own recurrence: the comparisons are
against scipy's softmax/logsumexp, against closed forms, or between two independent code
paths of the oracle (predicate mask vs. boolean bitmap, blocked vs. unblocked, split+merge
vs. single pass) on inputs where the mask semantics are decided by construction.
"""
import numpy as np
import pytest

from diffgemma_amd import attention as A
from diffgemma_amd import rounding as R
from helpers import dense_reference, max_abs_diff, ref_kv_split

FIXTURES = {
    "tiny": A.tiny_fixture,
    "wide": A.wide_fixture,
    "full_hd512": A.full_hd512_fixture,
    "full_grp8_hd512": A.full_grp8_hd512_fixture,
    "sliding_hd256": A.sliding_hd256_fixture,
}


def odesc(po, f, **kw):
    return po.make_desc(f.canvas, f.n_q_heads, f.n_kv(), f.head_dim(), f.kv_len, **kw)


# ---------------------------------------------------------------- rounding known answers
def test_bf16_known_answers(po):
    lib = po.load()
    # src/shaders/common/bf16.rs:47-55 uses 1.234567 and 0.001234567 as its round-trip values
    for v in (1.234567, 0.001234567):
        bits = np.float32(v).view(np.uint32) >> 16
        assert lib.dgo_f32_to_bf16_trunc(v) == bits
        assert lib.dgo_bf16_to_f32(int(bits)) == np.uint32(int(bits) << 16).view(np.float32)
    assert lib.dgo_f32_to_bf16_trunc(1.0) == 0x3F80
    assert lib.dgo_f32_to_bf16_trunc(-2.0) == 0xC000
    # truncation vs nearest-even differ exactly when the dropped half is above the midpoint
    x = np.uint32(0x3F80C000).view(np.float32)  # 1.0 + 0.75 ulp_bf16
    assert lib.dgo_f32_to_bf16_trunc(float(x)) == 0x3F80
    assert lib.dgo_f32_to_bf16_rne(float(x)) == 0x3F81
    tie = np.uint32(0x3F808000).view(np.float32)  # exact tie -> even mantissa
    assert lib.dgo_f32_to_bf16_rne(float(tie)) == 0x3F80
    tie2 = np.uint32(0x3F818000).view(np.float32)
    assert lib.dgo_f32_to_bf16_rne(float(tie2)) == 0x3F82


def test_f16_known_answers(po):
    lib = po.load()
    assert lib.dgo_f32_to_f16_trunc(1.0) == 0x3C00
    assert lib.dgo_f32_to_f16_trunc(-0.5) == 0xB800
    assert lib.dgo_f32_to_f16_trunc(1e6) == 0x7BFF       # clamp to 65504 (f16.rs:29)
    assert lib.dgo_f32_to_f16_trunc(-1e6) == 0xFBFF
    assert lib.dgo_f32_to_f16_trunc(1e-6) == 0x0000      # subnormal range flushes to +0 (f16.rs:41-43)
    assert lib.dgo_f32_to_f16_trunc(-1e-6) == 0x8000
    assert lib.dgo_f32_to_f16_trunc(float("nan")) & 0x7FFF == 0x7E00
    assert lib.dgo_f32_to_f16_trunc(1.0 + 1.5 * 2 ** -10) == 0x3C01  # truncates, numpy would round to 0x3C02
    assert lib.dgo_f16_to_f32(0x3555) == pytest.approx(0.333251953125)
    assert lib.dgo_f16_to_f32(0x0001) == 2.0 ** -24          # subnormal decode (f16.rs:8-13)


def test_f16_rne_matches_numpy(po):
    rng = np.random.default_rng(7)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10,
                        (rng.standard_normal(5000) * 1e-5).astype(np.float32),
                        np.array([65504.0, 65519.0, 65520.0, 1e9, -1e9, 0.0, -0.0, 6e-8, 3e-8, 2.98e-8], np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = po.to_bits(x, po.ROUND_F16_RNE)
    assert np.array_equal(got, want)
    # decode agrees with numpy for every finite half pattern
    allbits = np.arange(0, 0x7C00, dtype=np.uint16)
    assert np.array_equal(po.from_bits(allbits, True), allbits.view(np.float16).astype(np.float32))


def test_python_rounding_matches_oracle(po):
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(50000) * 4).astype(np.float32)
    assert np.array_equal(R.f32_to_bf16_bits_trunc(x), po.to_bits(x, po.ROUND_BF16_TRUNC))
    assert np.array_equal(R.f32_to_bf16_bits_rne(x), po.to_bits(x, po.ROUND_BF16_RNE))
    assert np.array_equal(R.f32_to_f16_bits_trunc(x), po.to_bits(x, po.ROUND_F16_TRUNC))
    assert np.array_equal(R.f32_to_f16_bits_rne(x), po.to_bits(x, po.ROUND_F16_RNE))


# ---------------------------------------------------------------- fixtures
@pytest.mark.parametrize("name,dims", [("tiny", None), ("wide", None),
                                       ("model_attn", (4, 16, 8, 512, 28)), ("model_attn", (16, 16, 2, 512, 28)),
                                       ("model_attn", (4, 16, 8, 256, 128)), ("model_full", (8, 16, 2, 512, 100))])
def test_fixture_generators_agree(po, name, dims):
    """numpy generators (product side) vs the oracle's C++ restatement of the same closed forms."""
    if name == "tiny":
        f, (q, kv) = A.tiny_fixture(), po.fixture("tiny")
    elif name == "wide":
        f, (q, kv) = A.wide_fixture(), po.fixture("wide")
    elif name == "model_attn":
        f = A.model_attn_fixture(*dims, is_full=dims[3] == 512)
        q, kv = po.fixture("model_attn", *dims)
    else:
        c, nq, nkv, hd, kvl = dims
        f = A.model_full_fixture(kvl, canvas=c)
        q, kv = po.fixture("model_full", *dims)
    # sin/cos of f32 arguments: libm and numpy may differ in the last ulp
    assert max_abs_diff(f.q, q) < 2e-6
    assert max_abs_diff(f.kvcache, kv) < 2e-7 + 1e-6


def test_fixture_closed_form_spot_values():
    f = A.tiny_fixture()
    kv = f.kvcache.reshape(4, 2, 2, 32)   # [t][K|V][h][d]
    assert kv[0, 0, 0, 0] == 0.0                                   # sin(0)
    assert kv[0, 1, 0, 0] == 1.0                                   # cos(0)
    assert kv[3, 0, 1, 5] == pytest.approx(np.sin((3 * 17 + 3 + 5) * 0.05), abs=1e-6)
    assert kv[2, 1, 1, 7] == pytest.approx(np.cos((2 * 13 + 5 + 7) * 0.04), abs=1e-6)
    assert f.q[10] == pytest.approx(np.sin(10 * 0.11) * 0.6, abs=1e-6)
    g = A.full_grp8_hd512_fixture()
    assert (g.canvas, g.n_q_heads, g.n_kv(), g.head_dim(), g.kv_len) == (16, 16, 2, 512, 28)
    kvg = g.kvcache.reshape(44, 2, 2, 512)
    assert kvg[7, 0, 1, 9] == pytest.approx(np.sin((7 * 19 + 7 + 9) * 0.0031) * 0.4, abs=1e-6)
    assert kvg[7, 1, 1, 9] == pytest.approx(np.cos((7 * 23 + 11 + 9) * 0.0027) * 0.35, abs=1e-6)


def test_synthetic_fill_kv_range(po):
    bits = po.synthetic_fill_kv(4096, 12345)
    vals = np.abs(bits.view(np.float16).astype(np.float32))
    assert vals.min() >= 0.125 and vals.max() < 0.25
    assert 0.3 < np.mean(bits >> 15) < 0.7          # both signs occur
    assert np.array_equal(bits, po.synthetic_fill_kv(4096, 12345))
    assert not np.array_equal(bits, po.synthetic_fill_kv(4096, 12347))


def test_synthetic_fill_kv_known_answer(po):
    """The generator is xorshift64* (shifts 12, 25, 27, multiplier 0x2545F4914F6CDD1D); its published
    outputs from state 1 are 5180492295206395165, 12380297144915551517, 13389498078930870103.  The fill
    takes bits 32..47 of an output as r and stores (r & 0x3FF) | 0x3000 | ((r & 0x400) << 5), worked out
    by hand below: a wrong shift, multiplier, word slice or bit placement changes these words."""
    #  0x47E4CE4B896CDD1D -> r = 0xCE4B: mantissa 0x24B, bit 10 set   -> 0x8000 | 0x3000 | 0x24B
    #  0xABCFA6A8E079651D -> r = 0xA6A8: mantissa 0x2A8, bit 10 set   -> 0x8000 | 0x3000 | 0x2A8
    #  0xB9D10D8FEB731F57 -> r = 0x0D8F: mantissa 0x18F, bit 10 set   -> 0x8000 | 0x3000 | 0x18F
    want = np.array([0xB24B, 0xB2A8, 0xB18F], dtype=np.uint16)
    assert np.array_equal(po.synthetic_fill_kv(3, 1), want)
    assert np.array_equal(po.synthetic_fill_kv(3, 0), want)       # the seed's lowest bit is forced on
    assert float(want[:1].view(np.float16)[0]) == -(0.125 * (1 + 0x24B / 1024))


# ---------------------------------------------------------------- recurrence vs textbook
@pytest.mark.parametrize("name", list(FIXTURES))
@pytest.mark.parametrize("strict", [0, 1])
def test_recurrence_matches_textbook_softmax(po, name, strict):
    f = FIXTURES[name]()
    d = odesc(po, f, strict_order=strict)
    out, lse = po.attention_f32(d, f.q, f.kvcache)
    k, v = ref_kv_split(f)
    mask = np.ones((f.canvas, f.t_total()), bool)
    want, want_lse = dense_reference(f.q.reshape(f.canvas, f.n_q_heads, -1), k, v, mask)
    assert max_abs_diff(out, want) < 5e-6
    assert np.max(np.abs(lse - want_lse) / np.maximum(np.abs(want_lse), 1.0)) < 1e-5
    out64, lse64 = po.attention_f64(d, f.q, f.kvcache)
    assert max_abs_diff(out64, want) < 1e-12
    assert max_abs_diff(lse64, want_lse) < 1e-10


def test_no_scale_is_applied(po):
    """A 1/sqrt(d) factor would change this result; the reference applies none (ARCHITECTURE.md:152-153)."""
    f = A.wide_fixture()
    out, _ = po.attention_f32(odesc(po, f), f.q, f.kvcache)
    k, v = ref_kv_split(f)
    mask = np.ones((f.canvas, f.t_total()), bool)
    scaled, _ = dense_reference(f.q.reshape(f.canvas, f.n_q_heads, -1), k, v, mask, scale=1 / np.sqrt(64))
    assert max_abs_diff(out, scaled) > 1e-3
    out_s, _ = po.attention_f32(odesc(po, f, scale=1 / np.sqrt(64)), f.q, f.kvcache)
    assert max_abs_diff(out_s, scaled) < 5e-6


def test_gqa_head_map(po):
    """kvh = qh / (Hq/Hkv): heads of one group fed the same Q row give the same output;
    heads of different groups do not."""
    f = A.full_grp8_hd512_fixture()
    q = f.q.reshape(f.canvas, f.n_q_heads, -1).copy()
    q[:] = q[:, :1, :]
    out, _ = po.attention_f32(odesc(po, f), q, f.kvcache)
    for h in range(1, 8):
        assert np.array_equal(out[:, h], out[:, 0])
    for h in range(9, 16):
        assert np.array_equal(out[:, h], out[:, 8])
    assert max_abs_diff(out[:, 0], out[:, 8]) > 1e-4


def test_kv_layouts_agree(po):
    f = A.sliding_hd256_fixture()
    t = f.t_total()
    ref, lse = po.attention_f32(odesc(po, f), f.q, f.kvcache)
    k, v = ref_kv_split(f)
    planes = np.stack([k.transpose(1, 0, 2), v.transpose(1, 0, 2)])  # [2][Hkv][T][d]
    cap = t + 5
    padded = np.zeros((2, f.n_kv(), cap, f.head_dim()), np.float32)
    padded[:, :, :t] = planes
    out, lse2 = po.attention_f32(odesc(po, f, layout="head_major", t_cap=cap), f.q, padded)
    assert np.array_equal(out, ref) and np.array_equal(lse, lse2)


# ---------------------------------------------------------------- mask semantics
def test_visibility_predicate_table(po):
    """attention.metal:49-63 spelled out on a tiny case."""
    d = po.make_desc(4, 2, 1, 8, 10, causal_rows=2, window=4)
    vis = po.visible_matrix(d)
    # non-causal rows (2,3): keys >= kv_len-(window-1) = 7, through the whole canvas
    for tok in (2, 3):
        assert list(np.nonzero(vis[tok])[0]) == list(range(7, 14))
    # causal row r sits at qpos = 10 + r and sees [qpos-3, qpos]
    assert list(np.nonzero(vis[0])[0]) == [7, 8, 9, 10]
    assert list(np.nonzero(vis[1])[0]) == [8, 9, 10, 11]
    d2 = po.make_desc(4, 2, 1, 8, 10, causal_rows=2, causal_sees_masked=1)
    vis2 = po.visible_matrix(d2)
    assert list(np.nonzero(vis2[0])[0]) == list(range(0, 11)) + [12, 13]
    assert list(np.nonzero(vis2[1])[0]) == list(range(0, 12)) + [12, 13]
    d3 = po.make_desc(4, 2, 1, 8, 10, window=4, t_lo_override=3)
    assert list(np.nonzero(po.visible_matrix(d3)[0])[0]) == list(range(3, 14))


def test_visible_pair_counts(po):
    """Pair counts the benchmark's FLOP figures rest on."""
    lib = po.load()
    import ctypes as C
    cases = [
        (dict(causal_rows=128), 256, 16, 2, 512, 32768, 8429632),
        (dict(causal_rows=128, causal_sees_masked=1), 256, 16, 2, 512, 32768, 8446016),
        (dict(window=1024), 256, 16, 8, 256, 4096, 256 * 1279),
        (dict(window=1024, t_lo_override=4096 - 768), 256, 16, 8, 256, 4096, 256 * 1024),
        (dict(), 256, 16, 2, 512, 131072, 256 * 131328),
        (dict(causal_rows=256), 256, 16, 2, 512, 100, 256 * 100 + 256 * 257 // 2),
    ]
    for kw, c, hq, hkv, hd, kvl, want in cases:
        d = po.make_desc(c, hq, hkv, hd, kvl, **kw)
        assert lib.dgo_visible_pairs(C.byref(d)) == want


@pytest.mark.parametrize("window", [8, 33, 100])
def test_window_equals_all_valid_on_subrange(po, window):
    """Denoise window: same result as an unwindowed call whose cache starts at t_lo."""
    f = A.sliding_hd256_fixture()  # kv_len 128, canvas 4
    out_w, lse_w = po.attention_f32(odesc(po, f, window=window), f.q, f.kvcache)
    t_lo = max(0, f.kv_len - (window - 1))
    kv = f.kvcache.reshape(f.t_total(), -1)[t_lo:]
    d = po.make_desc(f.canvas, f.n_q_heads, f.n_kv(), f.head_dim(), f.kv_len - t_lo)
    out_s, lse_s = po.attention_f32(d, f.q, kv)
    assert np.array_equal(out_w, out_s) and np.array_equal(lse_w, lse_s)
    full, _ = po.attention_f32(odesc(po, f), f.q, f.kvcache)
    assert max_abs_diff(out_w, full) > 1e-6   # the window really removed keys


def test_causal_rows_equal_all_valid_on_prefix(po):
    """Causal row r == all-valid attention over keys [0, kv_len+r] (attention_gemm/mod.rs:306-359)."""
    f = A.full_grp8_hd512_fixture()
    out_c, lse_c = po.attention_f32(odesc(po, f, causal_rows=f.canvas), f.q, f.kvcache)
    q3 = f.q.reshape(f.canvas, f.n_q_heads, -1)
    k, v = ref_kv_split(f)
    for r in (0, 1, 7, f.canvas - 1):
        n = f.kv_len + r + 1
        want, want_lse = dense_reference(q3[r:r + 1], k[:n], v[:n], np.ones((1, n), bool))
        assert max_abs_diff(out_c[r], want[0]) < 5e-6
        assert np.max(np.abs(lse_c[r] - want_lse[0]) / np.abs(want_lse[0])) < 2e-6
    # the last causal row sees everything: identical to the denoise row
    out_a, _ = po.attention_f32(odesc(po, f), f.q, f.kvcache)
    assert np.array_equal(out_c[-1], out_a[-1])
    # and on a fixture with flat scores the first causal row visibly differs from the denoise row
    w = A.wide_fixture()
    wc, _ = po.attention_f32(odesc(po, w, causal_rows=w.canvas), w.q, w.kvcache)
    wa, _ = po.attention_f32(odesc(po, w), w.q, w.kvcache)
    assert max_abs_diff(wc[0], wa[0]) > 1e-4 and np.array_equal(wc[-1], wa[-1])


@pytest.mark.parametrize("window", [0, 5, 11])
def test_causal_super_chunk_is_its_sub_chunks(po, window):
    """A causal call over n_subs * c rows at kv_len == the per-sub-chunk calls the reference encodes
    (rows [s*c, (s+1)*c) at kv_len + s*c; src/metal/step_kernel/runtime.rs:370-389), and every row
    with a window is the dense result over keys [pos-(window-1), pos]."""
    rng = np.random.default_rng(5)
    c, subs, hq, hkv, hd, kvl = 4, 3, 4, 2, 32, 9
    canvas, t_all = c * subs, kvl + c * subs
    q = rng.standard_normal((canvas, hq, hd)).astype(np.float32)
    kv = rng.standard_normal((t_all, 2, hkv, hd)).astype(np.float32)
    big, big_lse = po.attention_f32(po.make_desc(canvas, hq, hkv, hd, kvl, causal_rows=canvas, window=window), q, kv)
    for s_ in range(subs):
        d = po.make_desc(c, hq, hkv, hd, kvl + s_ * c, causal_rows=c, window=window)
        out, lse = po.attention_f32(d, q[s_ * c:(s_ + 1) * c], kv[:kvl + (s_ + 1) * c])
        assert np.array_equal(out, big[s_ * c:(s_ + 1) * c]) and np.array_equal(lse, big_lse[s_ * c:(s_ + 1) * c])
    for r in range(canvas):
        pos = kvl + r
        lo = max(0, pos - (window - 1)) if window else 0
        want, want_lse = dense_reference(q[r:r + 1], kv[lo:pos + 1, 0], kv[lo:pos + 1, 1], np.ones((1, pos + 1 - lo), bool))
        assert max_abs_diff(big[r], want[0]) < 5e-6
        assert np.max(np.abs(big_lse[r] - want_lse[0])) < 2e-5


def test_mixed_mask_is_rowwise_composition(po):
    f = A.full_grp8_hd512_fixture()   # canvas 16
    cr = 6
    mixed, lse_m = po.attention_f32(odesc(po, f, causal_rows=cr), f.q, f.kvcache)
    causal, lse_c = po.attention_f32(odesc(po, f, causal_rows=f.canvas), f.q, f.kvcache)
    denoise, lse_d = po.attention_f32(odesc(po, f), f.q, f.kvcache)
    assert np.array_equal(mixed[:cr], causal[:cr]) and np.array_equal(mixed[cr:], denoise[cr:])
    assert np.array_equal(lse_m[:cr], lse_c[:cr]) and np.array_equal(lse_m[cr:], lse_d[cr:])


@pytest.mark.parametrize("kw", [dict(), dict(causal_rows=5), dict(causal_rows=16), dict(window=9),
                                dict(causal_rows=7, window=9), dict(causal_rows=7, causal_sees_masked=1),
                                dict(window=9, t_lo_override=3)])
def test_predicate_path_equals_bitmap_path(po, kw):
    """Two independent code paths: the streaming recurrence with the predicate mask and the
    dense-score path with a boolean bitmap (src/model/attention.rs:354-394)."""
    f = A.full_grp8_hd512_fixture()
    d = odesc(po, f, **kw)
    out, _ = po.attention_f32(d, f.q, f.kvcache)
    k, v = ref_kv_split(f)
    mask = po.visible_matrix(d)
    bm = po.attention_bitmap_f32(f.q.reshape(f.canvas, f.n_q_heads, -1), k, v, mask, f.n_q_heads, f.n_kv(),
                                 f.head_dim())
    assert max_abs_diff(out, bm) < 2e-5   # two fp32 evaluation orders, scores of magnitude ~1e2
    want, _ = dense_reference(f.q.reshape(f.canvas, f.n_q_heads, -1), k, v, mask)
    assert max_abs_diff(out, want) < 5e-6


def test_bitmap_sparse_mask(po):
    """Arbitrary (non-interval) mask through the bitmap path vs scipy."""
    rng = np.random.default_rng(11)
    m, t, hq, hkv, hd = 6, 19, 4, 2, 16
    q = rng.standard_normal((m, hq, hd)).astype(np.float32)
    k = rng.standard_normal((t, hkv, hd)).astype(np.float32)
    v = rng.standard_normal((t, hkv, hd)).astype(np.float32)
    mask = rng.random((m, t)) < 0.4
    mask[:, 0] = True
    out = po.attention_bitmap_f32(q, k, v, mask, hq, hkv, hd)
    want, _ = dense_reference(q, k, v, mask)
    assert max_abs_diff(out, want) < 1e-5


def test_ring_map(po):
    f = A.sliding_hd256_fixture()   # T = 132
    lin, lse = po.attention_f32(odesc(po, f), f.q, f.kvcache)
    # a ring at least as large as T is the identity map
    big = np.zeros((256, f.n_kv() * f.head_dim() * 2), np.float32)
    big[:f.t_total()] = f.kvcache.reshape(f.t_total(), -1)
    out, lse2 = po.attention_f32(odesc(po, f, kv_ring_mask=255), f.q, big)
    assert np.array_equal(out, lin) and np.array_equal(lse, lse2)
    # a wrapped ring: only the window is live; place position p at slot p & 63
    window = 40
    ring = np.full((64, f.n_kv() * f.head_dim() * 2), np.nan, np.float32)
    rows = f.kvcache.reshape(f.t_total(), -1)
    t_lo = f.kv_len - (window - 1)
    for p in range(t_lo, f.t_total()):
        ring[p & 63] = rows[p]
    out_r, lse_r = po.attention_f32(odesc(po, f, window=window, kv_ring_mask=63), f.q, ring)
    out_l, lse_l = po.attention_f32(odesc(po, f, window=window), f.q, f.kvcache)
    assert np.array_equal(out_r, out_l) and np.array_equal(lse_r, lse_l)


# ---------------------------------------------------------------- blocked / split + merge
@pytest.mark.parametrize("name", ["full_hd512", "full_grp8_hd512", "sliding_hd256"])
@pytest.mark.parametrize("round_kv", [True, False])
def test_blocked_matches_unblocked(po, name, round_kv):
    """The reference's own invariance test (attention_flash/mod_tests.rs:25-58): causal mask,
    bk in {1,3,8,16,64,4096}, max|diff| < 1e-3 after the bf16 output store."""
    f = FIXTURES[name]()
    q = R.bf16_bits_to_f32(R.f32_to_bf16_bits_trunc(f.q))
    kv = R.f16_bits_to_f32(R.f32_to_f16_bits_trunc(f.kvcache)) if round_kv else f.kvcache
    d = odesc(po, f, causal_rows=f.canvas, strict_order=1)   # sequential sums, as both reference twins do
    ref, ref_lse = po.attention_f32(d, q, kv)
    ref_b = po.round_array(ref, po.ROUND_BF16_TRUNC)
    for bk in (1, 3, 8, 16, 64, 4096):
        out, lse = po.attention_blocked_f32(d, q, kv, bk)
        assert max_abs_diff(po.round_array(out, po.ROUND_BF16_TRUNC), ref_b) < 1e-3
        assert max_abs_diff(out, ref) < 2e-6
        assert np.max(np.abs(lse - ref_lse) / np.abs(ref_lse)) < 2e-6


@pytest.mark.parametrize("cuts", [(0, 7, 44), (0, 1, 2, 30, 44), (0, 16, 16, 44), (0, 44)])
def test_split_then_merge_equals_single_pass(po, cuts):
    f = A.full_grp8_hd512_fixture()   # T = 44
    d = odesc(po, f, causal_rows=5)
    ref, ref_lse = po.attention_f32(d, f.q, f.kvcache)
    parts = [po.attention_partial_f32(d, f.q, f.kvcache, a, b) for a, b in zip(cuts[:-1], cuts[1:])]
    out, lse = po.merge_partials_f32(parts, f.head_dim())
    assert max_abs_diff(out, ref.reshape(out.shape)) < 2e-5   # fp32 summation order, scores ~1e2
    assert np.max(np.abs(lse - ref_lse.ravel()) / np.abs(ref_lse.ravel())) < 2e-6   # LSE ~ 1e3 here
    # the merge is the textbook closed form
    m = np.stack([p[1] for p in parts]).astype(np.float64)
    l = np.stack([p[2] for p in parts]).astype(np.float64)
    acc = np.stack([p[0] for p in parts]).astype(np.float64)
    mx = m.max(0)
    w = np.where(l > 0, np.exp(m - mx), 0.0)
    den = (w * l).sum(0)
    want = (w[:, :, None] * acc).sum(0) / den[:, None]
    assert max_abs_diff(out, want) < 1e-6
    assert np.max(np.abs(lse - (mx + np.log(den))) / np.abs(lse)) < 1e-6


# ---------------------------------------------------------------- special cases
def test_all_keys_equal_gives_mean_v(po):
    c, hq, hkv, hd, kvl = 3, 4, 2, 32, 9
    t = c + kvl
    rng = np.random.default_rng(5)
    q = rng.standard_normal((c, hq, hd)).astype(np.float32)
    kv = np.zeros((t, 2, hkv, hd), np.float32)
    krow = rng.standard_normal((hkv, hd)).astype(np.float32)
    kv[:, 0] = krow
    kv[:, 1] = rng.standard_normal((t, hkv, hd)).astype(np.float32)
    out, lse = po.attention_f32(po.make_desc(c, hq, hkv, hd, kvl), q, kv)
    for h in range(hq):
        assert max_abs_diff(out[:, h], np.broadcast_to(kv[:, 1, h // 2].mean(0), (c, hd))) < 1e-5
        s = q[:, h] @ krow[h // 2]
        assert max_abs_diff(lse[:, h], s + np.log(t)) < 1e-4


def test_dominant_key_selects_its_value_row(po):
    c, hq, hkv, hd, kvl = 2, 2, 1, 64, 30
    t = c + kvl
    rng = np.random.default_rng(6)
    q = rng.standard_normal((c, hq, hd)).astype(np.float32)
    kv = (rng.standard_normal((t, 2, hkv, hd)) * 0.1).astype(np.float32)
    kv[17, 0, 0] = q[1, 0] * 8.0   # row 1 / head 0 is aligned with key 17
    out, lse = po.attention_f32(po.make_desc(c, hq, hkv, hd, kvl), q, kv)
    assert max_abs_diff(out[1, 0], kv[17, 1, 0]) < 1e-5
    assert lse[1, 0] == pytest.approx(8.0 * float(q[1, 0] @ q[1, 0]), rel=1e-5)


def test_empty_prefix_and_short_canvas(po):
    """kv_len = 0 (canvas only) and the retry canvases 128 / 64 the reference falls back to."""
    rng = np.random.default_rng(8)
    for c in (1, 64, 128):
        hq, hkv, hd = 4, 2, 32
        q = rng.standard_normal((c, hq, hd)).astype(np.float32)
        kv = rng.standard_normal((c, 2, hkv, hd)).astype(np.float32)
        out, lse = po.attention_f32(po.make_desc(c, hq, hkv, hd, 0), q, kv)
        want, want_lse = dense_reference(q, kv[:, 0], kv[:, 1], np.ones((c, c), bool))
        assert max_abs_diff(out, want) < 1e-5 and max_abs_diff(lse, want_lse) < 1e-4


def test_row_with_no_visible_key(po):
    """attention_mma2.metal:297: l == 0 stores 0; the closed-form LSE of an empty row is -inf."""
    f = A.tiny_fixture()
    d = odesc(po, f, t_lo_override=f.t_total())
    out, lse = po.attention_f32(d, f.q, f.kvcache)
    assert np.all(out == 0.0) and np.all(np.isneginf(lse))


def test_rms_norm_helpers(po):
    rng = np.random.default_rng(9)
    x = rng.standard_normal(512).astype(np.float32) * 3
    y = po.rms_norm_no_scale(x)
    assert np.mean(y.astype(np.float64) ** 2) == pytest.approx(1.0, rel=1e-4)
    want = x / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-6)
    assert max_abs_diff(y, want) < 1e-5


# ---------------------------------------------------------------- committed golden vectors
def test_golden_vectors(po):
    """Outputs of the float64 closed form, committed by tests/golden/make_golden.py."""
    import os
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "attention_golden.npz"))
    for name in FIXTURES:
        f = FIXTURES[name]()
        for tag, kw in (("denoise", {}), ("causal", dict(causal_rows=f.canvas)),
                        ("mixed_win", dict(causal_rows=f.canvas // 2, window=3))):
            out, lse = po.attention_f32(odesc(po, f, **kw), f.q, f.kvcache)
            idx = g[f"{name}/{tag}/idx"]
            assert max_abs_diff(out.ravel()[idx], g[f"{name}/{tag}/out"]) < 1e-5, (name, tag)
            assert max_abs_diff(lse.ravel(), g[f"{name}/{tag}/lse"]) < 5e-4, (name, tag)
