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


def test_one_recorded_graph_follows_the_committed_prefix(gpu_ready, po):
    """The reference binds StepParams as a device buffer (src/metal/step_kernel/enc.rs:2177-2220), so the step it
    encoded serves every committed prefix (src/metal/step_generate/turn.rs:575-660: kv_len += 256 per committed
    block).  Same here with the *_dev entry points: one graph recorded at prefix 32768, replayed there and, after
    only the device word changed, at 33024.  At both lengths the replay equals plain launches bit for bit and
    meets the oracle; at the first it also equals the graph-free schedule that bakes kv_len into its launches."""
    import torch
    from diffgemma_amd import schedule
    kv0, kv1 = 32768, 33024
    sc = schedule.DenoiseSchedule(kv_len=kv0, kv_len_max=kv1).build()
    plain = schedule.DenoiseSchedule(kv_len=kv0).build()
    for a, b in zip(sc.layers, plain.layers):      # the same cache rows behind both (they are drawn per layer size)
        src = a.cache.view(2, a.n_kv_heads, a.slots, a.head_dim)
        b.cache.view(2, b.n_kv_heads, b.slots, b.head_dim).copy_(src[:, :, :b.slots])
    sc.regenerate(0)
    sc.run_eager()
    torch.cuda.synchronize()
    sc.regenerate(0)
    sc.capture()
    for it, kv in enumerate((kv0, kv1)):
        sc.set_kv_len(kv)
        sc.regenerate(it)
        sc.run_eager()
        torch.cuda.synchronize()
        eager = sc.outputs()
        eager_lse = [lay.lse.clone() for lay in sc.layers]
        if it == 0:
            plain.regenerate(0)
            plain.run_eager()
            torch.cuda.synchronize()
            for lay, other in zip(sc.layers, plain.layers):
                assert torch.equal(lay.out, other.out), lay.index
        for lay in sc.layers:
            lay.out.fill_(-1)
        # the eager pass wrote this iteration's canvas rows into the caches and rotated q in place: same inputs again
        sc.regenerate(it)
        sc.replay()
        torch.cuda.synchronize()
        for lay, want, want_lse in zip(sc.layers, eager, eager_lse):
            assert torch.equal(lay.out, want) and torch.equal(lay.lse, want_lse), (kv, lay.index)
        for idx in (0, 5, 29):
            r = schedule_oracle_check(sc, po, idx, [0, 128, 255])
            assert r["finite"] and r["max_abs"] <= 2e-2 and r["mean_abs"] <= 2e-3 and r["lse_rel"] <= 1e-3, (kv, idx, r)
    # the two prefixes really gave different rows (the canvas differs too; this guards against a stale device word)
    assert sc.kv_len == kv1
