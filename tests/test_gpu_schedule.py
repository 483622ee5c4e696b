"""The 30-layer attention schedule of a denoise iteration (25 sliding + 5 global layers at prefix
32768), captured in a HIP graph and replayed for 16 iterations over one cached prefix: the shape of
the reference's denoise loop (src/metal/step_generate/turn.rs:575-623, one command buffer per step
src/metal/step_kernel/runtime.rs:573-631, full layers src/metal/step_kernel/mod.rs:127)."""
import numpy as np
import pytest

from helpers import schedule_oracle_check

pytestmark = pytest.mark.gpu

N_ITER = 16


@pytest.fixture(scope="module")
def sched(gpu_ready):
    from diffgemma_amd import schedule
    return schedule.DenoiseSchedule().build()


def test_schedule_shape(sched):
    from diffgemma_amd import step_kv
    assert len(sched.layers) == step_kv.N_LAYERS == 30
    assert [l.index for l in sched.layers if l.full] == list(step_kv.FULL_LAYERS)
    for l in sched.layers:
        assert (l.head_dim, l.n_kv_heads) == ((512, 2) if l.full else (256, 8))
        assert l.slots == (sched.kv_len + sched.canvas if l.full else sched.ring)
    # 5 global layers of config 3's key count without its causal rows + 25 sliding layers of 1279 keys
    want = 5 * 4 * 512 * 16 * 256 * (32768 + 256) + 25 * 4 * 256 * 16 * 256 * 1279
    assert sched.flops_per_iteration == want


def test_replay_equals_eager_for_16_iterations_and_meets_the_oracle(sched, po):
    """Every iteration regenerates the canvas projections from seed + iteration (the prefix rows of
    the caches stay), runs the 60 launches eagerly, then replays the captured graph on the same
    inputs: every layer's output must be the same bits.  Layers 0, 5 and 29 of the first and the
    last iteration are checked against the CPU oracle on a row sample."""
    import torch
    sched.regenerate(0)
    sched.run_eager()           # a first pass, also what a capture wants before it
    torch.cuda.synchronize()
    sched.regenerate(0)
    sched.capture()
    toks = [0, 77, 128, 255]
    for it in range(N_ITER):
        sched.regenerate(it)
        sched.run_eager()
        torch.cuda.synchronize()
        eager = sched.outputs()
        for lay in sched.layers:
            lay.out.fill_(-1)
        sched.regenerate(it)    # the producer rotated q in place: same inputs again for the replay
        sched.replay()
        torch.cuda.synchronize()
        for lay, want in zip(sched.layers, eager):
            assert torch.equal(lay.out, want), (it, lay.index)
        if it in (0, N_ITER - 1):
            for idx in (0, 5, 29):
                r = schedule_oracle_check(sched, po, idx, toks)
                assert r["finite"] and r["max_abs"] <= 2e-2 and r["mean_abs"] <= 2e-3, (it, idx, r)
                assert r["lse_rel"] <= 1e-3, (it, idx, r)      # per-row log-sum-exp, strictly relative


def test_iterations_differ(sched):
    """The regenerated canvas really changes what the layers compute (a stale graph input would not)."""
    import torch
    if sched.graph is None:
        sched.regenerate(0)
        sched.run_eager()
        torch.cuda.synchronize()
        sched.capture()
    sched.regenerate(3)
    sched.replay()
    torch.cuda.synchronize()
    a = sched.layers[5].out.clone()
    sched.regenerate(4)
    sched.replay()
    torch.cuda.synchronize()
    assert not torch.equal(a, sched.layers[5].out)
