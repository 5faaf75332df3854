"""ellm_attn_run_ragged on calls large enough for the kernel that deals the keys of all K/V planes
to the workgroups in equal shares (decode_balanced.hip), against the CPU oracle: sequence lengths
on and off the 64-key unit, one long sequence among short ones (a plane cut into hundreds of
pieces: two fold levels), whole short planes inside one workgroup's share, head layouts, batch
below capacity, repeated launches with other lengths (the arrival counters return to zero)."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, LSE_TOL, compare, rand_storage, to_dev, to_host

pytestmark = pytest.mark.gpu


def _operator(q, k, v, dtype, scale):
    import torch

    import ellm_amd

    _, bcap, hq, _ = q.shape
    hkv, cap = k.shape[1], k.shape[2]
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    dout = torch.full_like(dq, float("nan"))
    dlse = torch.full((1, bcap, hq), float("nan"), dtype=torch.float32, device="cuda")
    op = ellm_amd.Attention(dq, dk, dv, dout, bcap, hq, hkv, D, [hkv * cap * D, cap * D, D, 1], scale,
                            lse=dlse, sequence_capacity=cap, max_position_interval=1)
    return op, (dq, dk, dv, dout, dlse)


def _run_and_check(op, bufs, q, k, v, dtype, scale, positions, bound=None, want_path=1):
    import torch

    dq, dk, dv, dout, dlse = bufs
    b = len(positions)
    bound = int(max(positions)) if bound is None else bound
    assert op.ragged_path(bound, b) == want_path
    dout.fill_(float("nan"))
    dlse.fill_(float("nan"))
    dpos = torch.from_numpy(np.asarray(positions, dtype=np.uint32).view(np.int32)).cuda()
    op.run_ragged(dpos, bound, b)
    torch.cuda.synchronize()
    got, got_lse = to_host(dout, dtype), dlse.cpu().numpy()
    clamped = np.minimum(np.asarray(positions, dtype=np.uint32), bound)
    want, want_lse = orc.attention(q, k, v, scale, dtype, positions=clamped, batch=b)
    res = compare(got[:, :b], orc.from_storage(want, dtype)[:, :b], dtype)
    lse_err = float(np.abs(got_lse[:, :b] - want_lse[:, :b]).max())
    print(res, f"lse_err={lse_err:.2e}", flush=True)
    assert res["ok"], res
    assert lse_err <= LSE_TOL, lse_err
    if b < q.shape[1]:
        assert np.isnan(got[:, b:]).all()   # sequences beyond the live batch are never written
    return got, got_lse


# (name, batch capacity, q heads, kv heads, capacity, positions)
CASES = [
    ("qwen3_uneven_24", 24, 32, 4, 4096,
     [4095, 0, 17, 63, 64, 65, 4000, 127, 128, 129, 2047, 2048, 1, 3000, 62, 191, 192, 193, 1023, 1024, 1025, 5, 3333, 700]),
    ("one_long_among_short_two_fold_levels", 12, 8, 1, 40000, [39999] + [3, 70, 64, 0, 127, 5, 9, 200, 63, 1, 2]),
    ("all_equal_unit_multiples", 16, 32, 4, 8192, [8191] * 16),
    ("g32_two_head_groups", 6, 32, 1, 24000, [23999, 100, 2500, 64, 4097, 31]),
    ("g3_odd_group", 10, 6, 2, 14000, [13999, 4998, 1, 0, 2500, 2499, 63, 64, 65, 4097]),
    ("mha_heads", 8, 4, 4, 9000, [4000, 3000, 2000, 1000, 8999, 10, 100, 640]),
    ("batch_below_capacity", 30, 16, 4, 3400, [3399, 5, 1500, 64] * 5),
    ("shares_smaller_than_planes_many_sequences", 200, 8, 2, 1400, list(range(200, 1400, 6))),
    # more than 64 sequences (lengths scanned in LDS) and one plane cut into hundreds of pieces
    ("one_long_among_many_short", 70, 8, 1, 20000, [19999] + [(7 * i) % 300 for i in range(69)]),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16], ids=["f16", "bf16"])
def test_balanced_ragged_step_matches_oracle(case, dtype):
    name, bcap, hq, hkv, cap, positions = case
    print("case", name, flush=True)
    q = rand_storage((1, bcap, hq, D), 41, dtype)
    k = rand_storage((bcap, hkv, cap, D), 42, dtype)
    v = rand_storage((bcap, hkv, cap, D), 43, dtype)
    scale = 1.0 / np.sqrt(D)
    op, bufs = _operator(q, k, v, dtype, scale)
    try:
        _run_and_check(op, bufs, q, k, v, dtype, scale, positions, bound=cap - 1)
    finally:
        op.close()


def test_repeated_launches_with_other_lengths_and_bit_reproducible():
    """One handle, launch after launch with different lengths (different piece counts per plane, one
    and two fold levels): every launch finds the counters at zero; the same lengths give the same bits."""
    dtype = orc.F16
    bcap, hq, hkv, cap = 8, 32, 4, 20000
    q = rand_storage((1, bcap, hq, D), 51, dtype)
    k = rand_storage((bcap, hkv, cap, D), 52, dtype)
    v = rand_storage((bcap, hkv, cap, D), 53, dtype)
    scale = 1.0 / np.sqrt(D)
    op, bufs = _operator(q, k, v, dtype, scale)
    try:
        first = [19999, 3, 10000, 64, 5000, 63, 15000, 1]
        a, a_lse = _run_and_check(op, bufs, q, k, v, dtype, scale, first, bound=cap - 1)
        _run_and_check(op, bufs, q, k, v, dtype, scale, [100] * 8, bound=cap - 1)
        _run_and_check(op, bufs, q, k, v, dtype, scale, [19999] + [0] * 7, bound=cap - 1)
        _run_and_check(op, bufs, q, k, v, dtype, scale, [7, 19000, 18000, 17000], bound=cap - 1)
        b, b_lse = _run_and_check(op, bufs, q, k, v, dtype, scale, first, bound=cap - 1)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert np.array_equal(a_lse.view(np.uint32), b_lse.view(np.uint32))
        # positions above the stated bound are clamped to it on the device
        _run_and_check(op, bufs, q, k, v, dtype, scale, [19999, 12000, 5, 9000, 14999, 15000, 15001, 64], bound=15000)
    finally:
        op.close()


def test_small_calls_keep_the_plain_kernel():
    dtype = orc.F16
    q = rand_storage((1, 4, 16, D), 61, dtype)
    k = rand_storage((4, 2, 1024, D), 62, dtype)
    v = rand_storage((4, 2, 1024, D), 63, dtype)
    scale = 1.0 / np.sqrt(D)
    op, bufs = _operator(q, k, v, dtype, scale)
    try:
        _run_and_check(op, bufs, q, k, v, dtype, scale, [1000, 5, 640, 63], want_path=0)
        import ellm_amd
        with pytest.raises(ellm_amd.EllmError):
            op.ragged_path(1024, 4)      # beyond the capacity
        with pytest.raises(ellm_amd.EllmError):
            op.ragged_path(100, 5)       # beyond the batch capacity
    finally:
        op.close()


def test_recorded_step_replays_like_eager_while_the_lengths_move():
    """The step (attention over per-sequence positions + advance of the positions) recorded once
    through ellm_graph_* and replayed: the lengths change between replays, and with them the split of
    the keys over the workgroups, which the kernel derives from the device array at every launch.
    Every replay must equal the eager launch on the same lengths, bit for bit."""
    import torch

    import ellm_amd

    dtype = orc.F16
    bcap, hq, hkv, cap = 12, 32, 4, 6000
    q = rand_storage((1, bcap, hq, D), 71, dtype)
    k = rand_storage((bcap, hkv, cap, D), 72, dtype)
    v = rand_storage((bcap, hkv, cap, D), 73, dtype)
    scale = 1.0 / np.sqrt(D)
    op, (dq, dk, dv, dout, dlse) = _operator(q, k, v, dtype, scale)
    start = np.array([5000, 3, 62, 63, 64, 1000, 2500, 127, 4090, 700, 1, 3333], dtype=np.uint32)
    steps, by = 4, 37
    try:
        assert op.ragged_path(cap - 1, bcap) == 1
        stream = torch.cuda.Stream()

        def walk(use_graph):
            pos = torch.from_numpy(start.view(np.int32).copy()).cuda()
            outs = []
            graph = None
            with torch.cuda.stream(stream):
                for n in range(steps):
                    dout.fill_(float("nan"))

                    def step():
                        op.run_ragged(pos, cap - 1, bcap, stream=stream)
                        ellm_amd.positions_advance(pos, by, stream=stream)

                    if not use_graph:
                        step()
                    else:
                        if graph is None:
                            stream.synchronize()
                            with ellm_amd.StepGraph(stream) as graph:
                                step()
                        graph.launch()
                    stream.synchronize()
                    outs.append((dout.view(torch.int16).cpu().numpy().copy(), dlse.cpu().numpy().copy()))
                    _ = float(dout.float().sum())     # eager work between replays
            if graph is not None:
                graph.close()
            return outs, pos.cpu().numpy().view(np.uint32)

        eager, pos_e = walk(False)
        replay, pos_g = walk(True)
        assert np.array_equal(pos_e, start + steps * by) and np.array_equal(pos_g, pos_e)
        for n in range(steps):
            assert np.array_equal(eager[n][0], replay[n][0]), n
            assert np.array_equal(eager[n][1].view(np.uint32), replay[n][1].view(np.uint32)), n
        # and the last step against the oracle
        last = start + (steps - 1) * by
        want, want_lse = orc.attention(q, k, v, scale, dtype, positions=last, batch=bcap)
        got = orc.from_storage(replay[-1][0].view(np.uint16), dtype)
        res = compare(got, orc.from_storage(want, dtype), dtype)
        assert res["ok"], res
        assert np.abs(replay[-1][1] - want_lse).max() <= LSE_TOL
    finally:
        op.close()


@pytest.mark.parametrize("scale", [-0.07, 0.0, 1.0])
def test_unusual_scales_and_garbage_beyond_the_positions(scale):
    """Negative, zero and large scales; cache rows after a sequence's position hold NaN / Inf / huge
    values, which must not leak (the stream clamps its reads to the last valid row)."""
    dtype = orc.F16
    bcap, hq, hkv, cap = 16, 16, 4, 4200
    positions = [4199, 0, 63, 64, 1000, 2047, 2048, 3000, 17, 4100, 128, 129, 500, 3999, 1, 2500]
    q = rand_storage((1, bcap, hq, D), 81, dtype)
    k = rand_storage((bcap, hkv, cap, D), 82, dtype, scale=0.3)
    v = rand_storage((bcap, hkv, cap, D), 83, dtype)
    kf, vf = k.view(np.float16), v.view(np.float16)
    for b, pos in enumerate(positions):
        kf[b, :, pos + 1:] = [np.nan, np.inf, -np.inf, 6.0e4][b % 4]
        vf[b, :, pos + 1:] = [np.inf, np.nan, 6.0e4, -np.inf][b % 4]
    op, bufs = _operator(q, k, v, dtype, scale)
    try:
        got, _ = _run_and_check(op, bufs, q, k, v, dtype, scale, positions, bound=cap - 1)
        assert np.isfinite(got).all()
    finally:
        op.close()
