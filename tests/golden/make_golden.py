#!/usr/bin/env python3
"""Writes tests/golden/attention_golden.npz: expected outputs for the reference's closed-form
attention fixtures under three masks, computed in float64 with scipy's softmax/logsumexp
(helpers.dense_reference) from a visibility matrix built here from the mask rules in
src/shaders/attn/attention/attention.metal:49-63 of the reference.  Nothing from the oracle
library is used, so the file pins the oracle rather than echoing it.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from diffgemma_amd import attention as A  # noqa: E402
from helpers import dense_reference, ref_kv_split  # noqa: E402

FIXTURES = {
    "tiny": A.tiny_fixture, "wide": A.wide_fixture, "full_hd512": A.full_hd512_fixture,
    "full_grp8_hd512": A.full_grp8_hd512_fixture, "sliding_hd256": A.sliding_hd256_fixture,
}


def visibility(canvas, kv_len, causal_rows, window):
    t_all = kv_len + canvas
    vis = np.zeros((canvas, t_all), bool)
    for tok in range(canvas):
        causal = tok < causal_rows
        qpos = kv_len + tok
        hi = min(t_all, qpos + 1) if causal else t_all
        lo = 0
        if window:
            anchor = qpos if causal else kv_len
            lo = max(0, anchor - (window - 1))
        vis[tok, lo:hi] = True
    return vis


def main():
    out = {}
    for name, fn in FIXTURES.items():
        f = fn()
        k, v = ref_kv_split(f)
        q = f.q.reshape(f.canvas, f.n_q_heads, -1)
        for tag, cr, win in (("denoise", 0, 0), ("causal", f.canvas, 0), ("mixed_win", f.canvas // 2, 3)):
            o, lse = dense_reference(q, k, v, visibility(f.canvas, f.kv_len, cr, win))
            flat = o.ravel()
            idx = np.arange(0, flat.size, max(1, flat.size // 257), dtype=np.int64)
            out[f"{name}/{tag}/idx"] = idx
            out[f"{name}/{tag}/out"] = flat[idx]
            out[f"{name}/{tag}/lse"] = lse.ravel()
    path = os.path.join(HERE, "attention_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
