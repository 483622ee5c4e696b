"""Shared helpers for the parity tests (comparison metrics follow the reference's
assert_oracle, src/shaders/common/test_util.rs:23-58, and python/diffgemma_parity/vec_stats.py:24-41)."""
import numpy as np


def max_abs_diff(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))))


def mean_abs_diff(a, b):
    return float(np.mean(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))))


def cosine(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    na, nb = np.linalg.norm(a), np.linalg.norm(b)
    if na == 0 and nb == 0:
        return 1.0
    return float(a @ b / (na * nb))


def assert_oracle(a, b, max_tol, min_cos):
    mx, cs = max_abs_diff(a, b), cosine(a, b)
    assert mx <= max_tol and cs >= min_cos, f"oracle mismatch max_abs={mx:.6f} cos={cs:.6f} (tol={max_tol}, min_cos={min_cos})"
    assert np.all(np.isfinite(a)), "output has non-finite values"


def dense_reference(q, k, v, mask, scale=1.0):
    """Textbook softmax(QK^T)V with scipy, float64.  q [M,Hq,d], k/v [T,Hkv,d], mask [M,T] bool.
    Returns (out [M,Hq,d], lse [M,Hq])."""
    from scipy.special import logsumexp, softmax
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    m, hq, d = q.shape
    hkv = k.shape[1]
    g = hq // hkv
    out = np.zeros((m, hq, d))
    lse = np.zeros((m, hq))
    for h in range(hq):
        s = q[:, h, :] @ k[:, h // g, :].T * scale
        s = np.where(mask, s, -np.inf)
        p = softmax(s, axis=1)
        out[:, h, :] = p @ v[:, h // g, :]
        lse[:, h] = logsumexp(s, axis=1)
    return out, lse


def ref_kv_split(f):
    """Reference slot-major fixture cache -> (k, v) each [T, Hkv, d]."""
    t = f.t_total()
    kv = np.asarray(f.kvcache, np.float32).reshape(t, 2, f.n_kv(), f.head_dim())
    return kv[:, 0], kv[:, 1]


def schedule_oracle_check(sched, po, layer_index, toks):
    """Layer `layer_index` of a diffgemma_amd.schedule.DenoiseSchedule: its output rows `toks` (and, for a
    dense layer, their log-sum-exp) against the CPU oracle, on the inputs the device holds after the
    producer ran (rotated q, cache with the canvas rows written)."""
    import time
    from diffgemma_amd import rounding as R
    lay = sched.layers[layer_index]
    canvas, nq = sched.canvas, sched.n_q_heads
    qh = R.bf16_bits_to_f32(lay.q.cpu().numpy().view(np.uint16))
    kvh = R.bf16_bits_to_f32(lay.cache.cpu().numpy().view(np.uint16))
    od = po.make_desc(canvas, nq, lay.n_kv_heads, lay.head_dim, sched.kv_len, window=lay.window,
                      kv_ring_mask=lay.ring_mask, layout="head_major", t_cap=lay.slots)
    toks = np.asarray(toks, dtype=np.uint32)
    t0 = time.perf_counter()
    lse_rel = None
    if lay.full and sched.global_topk:
        ref = po.attention_topk_f32(od, sched.k_cfg, qh, kvh, tok_list=toks)
        if isinstance(ref, tuple):
            ref = ref[0]
    else:
        ref, ref_lse = po.attention_f32(od, qh, kvh, tok_list=toks)
        got_lse = lay.lse.cpu().numpy().reshape(canvas, nq)
        lse_rel = float(np.max(np.abs(got_lse[toks] - ref_lse[toks]) / np.abs(ref_lse[toks])))
    oracle_s = time.perf_counter() - t0
    got = R.bf16_bits_to_f32(lay.out.cpu().numpy().view(np.uint16)).reshape(canvas, nq, lay.head_dim)
    d = np.abs(got[toks] - ref[toks])
    return {"max_abs": float(d.max()), "mean_abs": float(d.mean()), "finite": bool(np.isfinite(got).all()),
            "lse_rel": lse_rel, "oracle_s": oracle_s}
