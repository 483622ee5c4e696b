"""Pins the oracle's top-k sparse attention (oracle/dg_attn_oracle.cpp: dgo_attention_topk_f32,
dgo_topk_row_k) before the HIP kernels are compared against it.

The reference's own checks (src/shaders/attn/attention_topk/cpu.rs:124-323: k >= n_valid recovers
dense attention, k = 1 returns the arg-max key's V row, finite output on model shapes, ragged causal
tail) are repeated on its fixtures; the selection itself is pinned against a numpy brute force on
inputs whose dot products are exact in fp32 (small dyadic values), so that score ties are plentiful
and the selected index sets have to agree exactly, tie-break included."""
import numpy as np
import pytest

from diffgemma_amd import attention as A
from helpers import dense_reference, max_abs_diff


def _sin_fixture(canvas, nq, nkv, hd, kv_len, qf, qa, kf, ka, cos=False):
    """The closed-form fixtures of attention_topk/cpu.rs:134-160,254-279."""
    q = (np.sin(np.arange(canvas * nq * hd, dtype=np.float32) * np.float32(qf)) * np.float32(qa)).astype(np.float32)
    i = np.arange((kv_len + canvas) * nkv * hd * 2, dtype=np.float32) * np.float32(kf)
    kv = ((np.cos(i) if cos else np.sin(i)) * np.float32(ka)).astype(np.float32)
    return q.reshape(canvas, nq, hd), kv.reshape(kv_len + canvas, 2, nkv, hd)


@pytest.mark.parametrize("causal", [True, False])
def test_k_at_least_the_visible_keys_recovers_dense(po, causal):
    q, kv = _sin_fixture(4, 8, 8, 16, 20, 0.07, 0.5, 0.003, 0.3)
    d = po.make_desc(4, 8, 8, 16, 20, causal_rows=4 if causal else 0)
    topk = po.attention_topk_f32(d, (1024, 0, 0, 0), q, kv)
    dense, _ = po.attention_f32(d, q, kv)
    assert max_abs_diff(topk, dense) < 2e-6
    mask = np.ones((4, 24), bool)
    if causal:
        mask = np.arange(24)[None, :] <= (20 + np.arange(4))[:, None]
    want, _ = dense_reference(q, kv[:, 0], kv[:, 1], mask)
    assert max_abs_diff(topk, want) < 2e-6


def test_k1_returns_the_value_row_of_the_argmax_key(po):
    canvas, nq, nkv, hd, kvl = 2, 4, 4, 8, 6
    q, kv = _sin_fixture(canvas, nq, nkv, hd, kvl, 0.11, 0.4, 0.005, 0.3, cos=True)
    d = po.make_desc(canvas, nq, nkv, hd, kvl, causal_rows=canvas)
    out, idx, cnt = po.attention_topk_f32(d, (1, 0, 0, 0), q, kv, sel_cap=1)
    for tok in range(canvas):
        for h in range(nq):
            s = kv[:kvl + tok + 1, 0, h].astype(np.float64) @ q[tok, h].astype(np.float64)
            best = int(np.argmax(s))
            assert cnt[tok, h] == 1 and idx[tok, h, 0] == best
            assert np.array_equal(out[tok, h], kv[best, 1, h])


def _brute(q, kv, vis, k_of_row, group):
    """numpy restatement from the definition: keep the k best (score desc, index asc), float64 softmax."""
    canvas, nq, hd = q.shape
    out = np.zeros((canvas, nq, hd))
    sel = {}
    for tok in range(canvas):
        ts = np.nonzero(vis[tok])[0]
        for h in range(nq):
            s = kv[ts, 0, h // group].astype(np.float64) @ q[tok, h].astype(np.float64)
            k = k_of_row(tok, len(ts))
            order = np.lexsort((ts, -s))[:k]
            sel[tok, h] = ts[order]
            if k == 0:
                continue
            p = np.exp(s[order] - s[order].max())
            out[tok, h] = (p / p.sum()) @ kv[ts[order], 1, h // group].astype(np.float64)
    return out, sel


CASES = [
    # canvas, nq, nkv, hd, kv_len, causal_rows, window, k
    (6, 4, 2, 32, 40, 0, 0, 8),
    (6, 4, 2, 32, 40, 6, 0, 8),
    (8, 6, 3, 16, 12, 5, 0, 5),      # mixed rows
    (5, 4, 4, 32, 30, 5, 9, 4),      # causal + window
    (7, 8, 1, 16, 3, 7, 0, 6),       # ragged tail: early rows see fewer than k keys
    (4, 4, 2, 16, 50, 0, 0, 1),
    (4, 4, 2, 16, 50, 0, 0, 54),     # k == visible keys
]


@pytest.mark.parametrize("case", CASES)
def test_selection_against_numpy_brute_force(po, case):
    canvas, nq, nkv, hd, kvl, cr, win, k = case
    rng = np.random.default_rng(hash(case) & 0xFFFF)
    # dyadic values with few bits: every dot product is exact in fp32, so ties are exact ties
    q = (rng.integers(-2, 3, (canvas, nq, hd)) / 4).astype(np.float32)
    kv = (rng.integers(-2, 3, (kvl + canvas, 2, nkv, hd)) / 4).astype(np.float32)
    kv[:, 1] = rng.standard_normal(kv[:, 1].shape).astype(np.float32)        # V: anything
    d = po.make_desc(canvas, nq, nkv, hd, kvl, causal_rows=cr, window=win)
    t_all = kvl + canvas
    vis = np.zeros((canvas, t_all), bool)       # the mask from its definition (attention.metal:49-63)
    for tok in range(canvas):
        pos = kvl + tok
        hi = pos + 1 if tok < cr else t_all
        anchor = pos if tok < cr else kvl
        lo = max(0, anchor - (win - 1)) if win else 0
        vis[tok, lo:hi] = True
    out, idx, cnt = po.attention_topk_f32(d, (k, 0, 0, 0), q, kv, sel_cap=max(k, 1))
    want, sel = _brute(q, kv, vis, lambda tok, n: min(k, n), nq // nkv)
    ties = 0
    for tok in range(canvas):
        for h in range(nq):
            assert cnt[tok, h] == len(sel[tok, h])
            assert np.array_equal(idx[tok, h, :cnt[tok, h]], sel[tok, h]), (tok, h)
            s = kv[sel[tok, h], 0, h // (nq // nkv)] @ q[tok, h]
            ties += len(s) - len(np.unique(s))
    assert max_abs_diff(out, want) < 5e-6
    if k > 2 and hd <= 16:
        assert ties > 0      # the case really exercised the tie-break


def test_tie_goes_to_the_lower_index(po):
    """Two identical key rows with different V rows and room for only one of them."""
    canvas, nq, nkv, hd, kvl = 1, 1, 1, 8, 9
    q = np.ones((1, 1, hd), np.float32)
    kv = np.zeros((kvl + 1, 2, 1, hd), np.float32)
    kv[:, 0, 0, 0] = np.arange(kvl + 1) * -1.0          # scores 0, -1, -2, ...: key 0 is best
    kv[3, 0, 0] = kv[7, 0, 0] = 0.0
    kv[3, 0, 0, 0] = kv[7, 0, 0, 0] = 5.0               # keys 3 and 7 tie at the top
    kv[:, 1, 0, 0] = np.arange(kvl + 1)                 # V row t holds t
    d = po.make_desc(canvas, nq, nkv, hd, kvl)
    out, idx, cnt = po.attention_topk_f32(d, (1, 0, 0, 0), q, kv, sel_cap=2)
    assert cnt[0, 0] == 1 and idx[0, 0, 0] == 3 and out[0, 0, 0] == 3.0
    out, idx, cnt = po.attention_topk_f32(d, (2, 0, 0, 0), q, kv, sel_cap=2)
    assert list(idx[0, 0]) == [3, 7] and out[0, 0, 0] == 5.0    # equal scores -> equal weights


def test_row_k_rule_known_answers(po):
    dyn = (256, 128, 64, 512)      # src/flags/accessors.rs:217: grid 256, t/128 clamped to [64, 512]
    assert po.topk_row_k(dyn, 33024, False) == 258           # denoise row at a 32768 prefix: 33024 / 128
    assert po.topk_row_k(dyn, 14600, True) == 116            # causal: 14600 -> 14848 (grid) / 128
    assert po.topk_row_k(dyn, 14593, True) == 116 and po.topk_row_k(dyn, 14848, True) == 116
    assert po.topk_row_k(dyn, 14849, True) == 118            # next grid cell: 15104 / 128
    assert po.topk_row_k(dyn, 14600, False) == 114           # not rounded up for a bidirectional row
    assert po.topk_row_k(dyn, 100, True) == 64               # k_min
    assert po.topk_row_k(dyn, 5, True) == 5                  # never more than the visible keys
    assert po.topk_row_k(dyn, 200000, False) == 512          # k_max
    assert po.topk_row_k((64, 0, 0, 0), 1000, True) == 64    # fixed k
    assert po.topk_row_k((64, 0, 0, 0), 10, False) == 10
    assert po.topk_row_k((0, 0, 0, 0), 10, False) == 1       # cpu.rs:59: k.max(1)


def test_adaptive_k_depends_on_the_position_only(po):
    """The number of kept keys of a causal row is a function of its absolute position, however the
    prompt was chunked (the reason the reference derives k per row, accessors.rs:191-209)."""
    hq, hkv, hd = 2, 1, 16
    rng = np.random.default_rng(3)
    total = 9000
    kv = rng.standard_normal((total, 2, hkv, hd)).astype(np.float32)
    qrow = rng.standard_normal((1, hq, hd)).astype(np.float32)
    dyn = (256, 128, 2, 512)
    pos = 8300
    got = []
    for kv_len, canvas in ((8192, 256), (8300, 1), (8250, 64)):
        tok = pos - kv_len
        q = np.zeros((canvas, hq, hd), np.float32)
        q[tok] = qrow
        d = po.make_desc(canvas, hq, hkv, hd, kv_len, causal_rows=canvas)
        out, idx, cnt = po.attention_topk_f32(d, dyn, q, kv[:kv_len + canvas], tok_list=[tok], sel_cap=128)
        got.append((int(cnt[tok, 0]), out[tok].copy(), np.sort(idx[tok, 0, :cnt[tok, 0]])))
    assert got[0][0] == (8448 // 128) == 66
    for g in got[1:]:
        assert g[0] == got[0][0] and np.array_equal(g[1], got[0][1]) and np.array_equal(g[2], got[0][2])


def test_model_shape_finite_and_ragged_causal_tail(po):
    """cpu.rs:303-323: canvas 256 behind 4 keys: row 0 sees 5 keys, row 255 sees 260; k = 64."""
    f = A.model_bench_fixture(512, 4, True)
    d = po.make_desc(f.canvas, f.n_q_heads, f.n_kv(), f.head_dim(), f.kv_len, causal_rows=f.canvas)
    toks = [0, 1, 58, 59, 60, 255]
    out, idx, cnt = po.attention_topk_f32(d, (64, 0, 0, 0), f.q, f.kvcache, tok_list=toks, sel_cap=64)
    assert np.isfinite(out).all()
    for tok in toks:
        assert (cnt[tok] == min(64, f.kv_len + tok + 1)).all()
        assert (idx[tok, :, :cnt[tok, 0]] <= f.kv_len + tok).all()
