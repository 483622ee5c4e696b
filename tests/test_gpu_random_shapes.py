"""Seeded random sweep of shapes and masks through the dense MFMA path, the scalar cross-check
kernel and the top-k path against the CPU oracle: ragged canvases, every head_dim, GQA ratios,
causal / windowed / mixed rows, explicit split counts.  The cases are fixed by the seeds."""
import numpy as np
import pytest

from diffgemma_amd import attention_topk as T
from diffgemma_amd import capi, workloads as W
from test_gpu_parity import MAX_ABS, MEAN_ABS, check_tolerances, run_workload
from test_gpu_topk_parity import run_topk
from helpers import max_abs_diff, mean_abs_diff

pytestmark = pytest.mark.gpu


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    hd = int(rng.choice([32, 64, 128, 256, 512]))
    hkv = int(rng.choice([1, 2, 4, 8]))
    group = int(rng.choice([1, 2, 3, 8]))
    canvas = int(rng.choice([1, 7, 32, 100, 256, 300]))
    kv_len = int(rng.choice([0, 5, 31, 64, 777, 2049, 6000]))
    mode = int(rng.integers(0, 4))
    causal_rows = [0, canvas, canvas // 2, 0][mode]
    window = int(rng.choice([0, 0, 17, 200, 1024])) if mode != 2 or rng.random() < 0.5 else 0
    splits = int(rng.choice([0, 0, 1, 3, 9]))
    return canvas, hkv * group, hkv, hd, kv_len, causal_rows, window, splits


@pytest.mark.parametrize("seed", range(40))
def test_dense_random_shape(gpu_ready, po, seed):
    canvas, hq, hkv, hd, kvl, cr, win, splits = _case(seed)
    w = W.Workload(f"rnd{seed}", canvas, hq, hkv, hd, kvl, causal_rows=cr, window=win, seed=seed)
    toks = None if canvas * (kvl + canvas) * hq * hd < 6e9 else np.unique(np.linspace(0, canvas - 1, 24).round().astype(np.uint32))
    # (the two flags change which kernel instance runs, never the result: some seeds carry them)
    flags = (capi.DG_ATTN_F_KV_FROM_HBM if seed % 2 else 0) | (capi.DG_ATTN_F_STREAMED_MERGE if seed % 3 == 1 else 0)
    # every third seed leaves the partial-row format to the library (fp32 for a bf16 cache) instead of asking for f16
    check_tolerances(*run_workload(po, w, n_splits=splits, toks=toks, flags=flags, default_partials=seed % 3 == 2))
    if seed % 4 == 0:
        check_tolerances(*run_workload(po, w, kernel=capi.DG_KERNEL_SCALAR, toks=toks))


@pytest.mark.parametrize("seed", range(16))
def test_topk_random_shape(gpu_ready, po, seed):
    canvas, hq, hkv, hd, kvl, cr, win, _ = _case(100 + seed)
    rng = np.random.default_rng(seed)
    k_cfg = T.adaptive_k() if seed % 3 == 0 else (int(rng.choice([1, 5, 64, 200, 1000])), 0, 0, 0)
    toks = None if canvas <= 64 else np.unique(np.linspace(0, canvas - 1, 16).round().astype(np.uint32))
    got, ref = run_topk(po, canvas, hq, hkv, hd, kvl, k_cfg, causal_rows=cr, window=win, seed=seed, toks=toks)
    assert np.isfinite(got).all()
    assert max_abs_diff(got, ref) <= 2e-2 and mean_abs_diff(got, ref) <= 2e-3
