"""dg_attn_forward_static, the entry point that allocates nothing: its split partial rows live in
device memory inside the library instead of a caller's workspace.  It has to give what
dg_attn_forward gives, bit for bit (same kernels), on calls that follow each other and share the
one scratch: a larger call first, a smaller one after it."""
import ctypes as C

import numpy as np
import pytest

from diffgemma_amd import attention as A
from diffgemma_amd import capi, workloads as W

pytestmark = pytest.mark.gpu


def both_ways(w, **desc_kw):
    import torch
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc(**desc_kw)
    assert capi.resolved_splits(d) > 1                      # the calls do use scratch
    assert 0 < capi.workspace_bytes(d) <= capi.load().dg_attn_static_scratch_bytes()
    n = w.canvas * w.n_q_heads
    out_a = torch.zeros(n * w.head_dim, dtype=torch.int16, device="cuda")
    out_b = torch.full((n * w.head_dim,), 0x7fc0, dtype=torch.int16, device="cuda")
    lse_a = torch.zeros(n, dtype=torch.float32, device="cuda")
    lse_b = torch.full((n,), float("nan"), dtype=torch.float32, device="cuda")
    A.forward(d, qd, kd, out_a, lse_a, A.alloc_workspace(d))
    capi.check(capi.load().dg_attn_forward_static(C.byref(d), qd.data_ptr(), kd.data_ptr(), out_b.data_ptr(),
                                                  lse_b.data_ptr(), A.stream_handle()))
    torch.cuda.synchronize()
    return out_a.cpu().numpy(), out_b.cpu().numpy(), lse_a.cpu().numpy(), lse_b.cpu().numpy()


def test_static_scratch_entry_equals_workspace_entry_on_two_calls_in_a_row(gpu_ready):
    big = W.scaled(W.config("cfg3_global"), 8192, "no_alloc_big")                                  # hd 512, 8 splits, f16 partial rows
    small = W.Workload("no_alloc_small", 64, 16, 8, 256, 1500, causal_rows=20, window=1024, seed=9)   # hd 256, fewer rows and splits
    for w, kw in ((big, {}), (small, {"n_splits": 3}), (small, {"n_splits": 2, "flags": capi.DG_ATTN_F_F32_PARTIALS})):
        out_a, out_b, lse_a, lse_b = both_ways(w, **kw)
        assert np.array_equal(out_a, out_b), w.name
        assert np.array_equal(lse_a.view(np.uint32), lse_b.view(np.uint32)), w.name
        assert np.isfinite(lse_a).all()


def test_static_scratch_entry_rejects_what_does_not_fit(gpu_ready):
    import torch
    lib = capi.load()
    d = W.config("cfg3_global").desc(flags=capi.DG_ATTN_F_F32_PARTIALS)       # 64.3 MiB of fp32 partial rows
    assert capi.workspace_bytes(d) > lib.dg_attn_static_scratch_bytes()
    dummy = torch.zeros(64, dtype=torch.int16, device="cuda")                 # never touched: the call enqueues nothing
    rc = lib.dg_attn_forward_static(C.byref(d), dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(), None,
                                    A.stream_handle())
    assert rc == capi.DG_ERR_SCRATCH_LIMIT
    assert "scratch" in capi.strerror(rc)
    torch.cuda.synchronize()
    assert int(dummy.abs().sum()) == 0
