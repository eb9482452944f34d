"""The entry point that allocates nothing (mmr_reshard_batch_static): same kernels as mmr_reshard_batch, tables in
the GPU's static scratch array.  Checked through the C ABI against mmr_reshard_batch and against the oracle, bit for
bit, on two calls in a row, the second with a smaller input; and with two contexts taking turns on the one array."""
import sys

import pytest

import multimesh_jax_amd as mm
from multimesh_jax_amd import _binding as B, workloads

from gpu_helpers import make_stores, read_all
from helpers import oracle_outputs, test_config

pytestmark = pytest.mark.gpu


def say(msg):
    print("[gpu-test] " + msg, flush=True)
    sys.stdout.flush()


def _both_ways(ctx, arrays):
    """Reshards `arrays` through the allocating entry point and through the static one (separate, poison-filled
    destination stores); returns both sets of destination shards and the device bytes allocated in between."""
    gs = [workloads.generate(a) for a in arrays]
    srcs, dsts_ref = make_stores(ctx, arrays, gs)
    _, dsts_static = make_stores(ctx, arrays, gs)
    ctx.ReshardBatch(srcs, dsts_ref)
    ctx.Sync()
    before = ctx.stats
    ctx.ReshardBatchStatic(srcs, dsts_static)
    ctx.Sync()
    after = ctx.stats
    ref = [read_all(ctx, d) for d in dsts_ref]
    got = [read_all(ctx, d) for d in dsts_static]
    for a, g, out in zip(arrays, gs, got):  # and against the oracle, like every other GPU test
        expect = oracle_outputs(a, g)
        assert sorted(out) == sorted(expect)
        for dev in expect:
            assert out[dev].tobytes() == expect[dev].tobytes(), (a["name"], dev)
    return ref, got, before, after


def _assert_equal(arrays, ref, got):
    for a, r, g in zip(arrays, ref, got):
        assert sorted(r) == sorted(g)
        for dev in r:
            assert g[dev].tobytes() == r[dev].tobytes(), (a["name"], dev)


def test_static_entry_point_matches_batch_on_two_calls_in_a_row():
    with mm.ReshardContext(0) as ctx:
        # first call: configuration 2 at 1/2 scale (copy groups, 16,384 chunks) together with the ragged arrays of
        # configuration 5 at 1/8 scale (span groups with pad fills) and a transposed layout (tile chunks)
        first = workloads.config(2, 2) + workloads.config(5, 8) + workloads.config(13, 8)
        say("static entry point, first call: %d arrays" % len(first))
        ref, got, before, after = _both_ways(ctx, first)
        _assert_equal(first, ref, got)
        assert after["bytes_allocated"] == before["bytes_allocated"]
        assert after["plans_built"] == before["plans_built"] and after["bindings_built"] == before["bindings_built"]
        assert after["kernel_launches"] - before["kernel_launches"] >= 3
        # second call, smaller: the array still holds the first call's tables beyond what this one overwrites
        second = workloads.config(5, 16)
        say("static entry point, second call: %d arrays" % len(second))
        ref, got, before, after = _both_ways(ctx, second)
        _assert_equal(second, ref, got)
        assert after["bytes_allocated"] == before["bytes_allocated"]


def test_static_entry_point_refuses_plans_beyond_the_array():
    with mm.ReshardContext(0) as ctx:
        # ragged rows lowered to one record per workgroup (the span kernel switched off): ~36,000 records of 72 bytes,
        # more than the array holds
        ctx.set_plan_options(0, 0, 0, B.MMR_PLAN_NO_SPAN)
        arrays = test_config(10, 2)
        gs = [workloads.generate(a) for a in arrays]
        srcs, dsts = make_stores(ctx, arrays, gs, poison=None)
        say("static entry point, oversized plan")
        with pytest.raises(B.MmrError) as e:
            ctx.ReshardBatchStatic(srcs, dsts)
        assert e.value.status_name == "INVALID_ARGUMENT" and "static scratch" in str(e.value)
        ctx.ReshardBatch(srcs, dsts)  # the allocating entry point takes it
        ctx.Sync()


def test_two_contexts_take_turns_on_the_static_array():
    """The array is one per GPU and process.  Two contexts (two streams) that call the static entry point in turn,
    with no host synchronisation in between, are ordered on the device: each call's stream waits for the kernels of
    the array's previous user.  Results against the oracle."""
    a_arrays = workloads.config(2, 4)
    b_arrays = workloads.config(5, 8)
    a_gs = [workloads.generate(a) for a in a_arrays]
    b_gs = [workloads.generate(a) for a in b_arrays]
    with mm.ReshardContext(0) as ca, mm.ReshardContext(0) as cb:
        a_sets = [make_stores(ca, a_arrays, a_gs) for _ in range(3)]
        b_sets = [make_stores(cb, b_arrays, b_gs) for _ in range(3)]
        ca.Sync()
        cb.Sync()
        say("two contexts, six interleaved static calls")
        before = (ca.stats["device_allocations"], cb.stats["device_allocations"])
        for k in range(3):
            ca.ReshardBatchStatic(*a_sets[k])
            cb.ReshardBatchStatic(*b_sets[k])
        # (a call may wait on the host for its own context's previous upload to leave the pinned staging buffer; the
        # order between the two contexts is kept on the device)
        assert (ca.stats["device_allocations"], cb.stats["device_allocations"]) == before
        ca.Sync()
        cb.Sync()
        for ctx, arrays, gs, sets in ((ca, a_arrays, a_gs, a_sets), (cb, b_arrays, b_gs, b_sets)):
            for _, dsts in sets:
                for a, g, d in zip(arrays, gs, dsts):
                    expect = oracle_outputs(a, g)
                    got = read_all(ctx, d)
                    for dev in expect:
                        assert got[dev].tobytes() == expect[dev].tobytes(), (a["name"], dev)
