"""ellm_attn_run_noalloc (the single-token step on the library's static device scratch, for
callers that cannot allocate) against ellm_attn_run / ellm_attn_run_ragged (the same step on
a handle's own workspace): same kernel, same split plan, so the outputs and the log-sum-exp
must be equal bit for bit (the calls with per-sequence positions here are small, so the handle
keeps the kernel the no-alloc entry point always uses; large ones go to the handle's kernel for
sequences of different lengths, which splits the keys differently).  Two calls in a row share the static scratch; the second is
smaller, so whatever the first one left behind (partials, counters) must not show.
Also checked against the CPU oracle within the operator's tolerance."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, compare, rand_storage, to_dev, to_host

pytestmark = pytest.mark.gpu


def _case(seed, batch, hq, hkv, cap, dtype):
    q = rand_storage((1, batch, hq, D), seed, dtype)
    k = rand_storage((batch, hkv, cap, D), seed + 1, dtype)
    v = rand_storage((batch, hkv, cap, D), seed + 2, dtype)
    return q, k, v


def _run_pair(q, k, v, dtype, batch, position=None, positions=None):
    """Returns ((out, lse) through the handle, (out, lse) through the no-alloc entry point)."""
    import torch

    import ellm_amd

    _, bcap, hq, _ = q.shape
    hkv, cap = k.shape[1], k.shape[2]
    scale = 1.0 / np.sqrt(D)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    results = []
    for use_noalloc in (False, True):
        dout = torch.full_like(dq, float("nan"))
        dlse = torch.full((1, bcap, hq), float("nan"), dtype=torch.float32, device="cuda")
        op = ellm_amd.Attention(dq, dk, dv, dout, bcap, hq, hkv, D, [hkv * cap * D, cap * D, D, 1], scale,
                                lse=dlse, sequence_capacity=cap, max_position_interval=1)
        dpos = None
        if positions is not None:
            dpos = torch.from_numpy(np.asarray(positions, dtype=np.uint32).view(np.int32)).cuda()
        bound = int(np.max(positions)) if positions is not None else position
        if use_noalloc:
            op.run_noalloc(bound, batch, positions=dpos)
        elif positions is not None:
            op.run_ragged(dpos, bound, batch)
        else:
            op.run(position, 1, batch)
        torch.cuda.synchronize()
        results.append((dout.view(torch.int16).cpu().numpy().copy(), dlse.cpu().numpy().copy(),
                        to_host(dout, dtype)))
        op.close()
    return results


def _check(q, k, v, dtype, batch, position=None, positions=None):
    (o_h, l_h, _), (o_n, l_n, f_n) = _run_pair(q, k, v, dtype, batch, position, positions)
    live = slice(0, batch)
    assert np.array_equal(o_h[:, live], o_n[:, live]), "outputs differ from the handle's path"
    assert np.array_equal(l_h[:, live].view(np.uint32), l_n[:, live].view(np.uint32))
    pos = positions if positions is not None else [position] * batch
    want, want_lse = orc.attention(q, k, v, 1.0 / np.sqrt(D), dtype,
                                   positions=np.asarray(pos, dtype=np.uint32), batch=batch)
    r = compare(f_n[:, live], orc.from_storage(want, dtype), dtype)
    assert r["ok"], r
    assert np.abs(l_n[:, live] - want_lse).max() <= 1e-4


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
def test_noalloc_equals_handle_two_calls_second_smaller(dtype):
    # first call: 3 sequences x 6000 keys, 4 planes... many splits per plane, two merge levels
    q, k, v = _case(11, 3, 16, 2, 6144, dtype)
    _check(q, k, v, dtype, batch=3, position=5999)
    # second call, smaller in every way (fewer sequences, shorter caches, per-sequence positions):
    # fewer splits, one merge level; the scratch still holds the first call's partials
    q, k, v = _case(21, 2, 16, 2, 1024, dtype)
    _check(q, k, v, dtype, batch=2, positions=[700, 333])
    # and an unsplit launch (too few keys to split): touches no scratch at all
    q, k, v = _case(31, 2, 8, 8, 256, dtype)
    _check(q, k, v, dtype, batch=2, position=100)


def test_noalloc_long_single_sequence_two_merge_levels():
    q, k, v = _case(41, 1, 32, 4, 40000, orc.F16)
    _check(q, k, v, orc.F16, batch=1, position=39999)
    q, k, v = _case(51, 1, 32, 4, 3000, orc.F16)
    _check(q, k, v, orc.F16, batch=1, position=2500)


def test_noalloc_rejects_what_the_scratch_cannot_hold():
    import torch

    import ellm_amd

    # GQA groups of 64 query heads on two long planes: 2 x 64 heads x 128 splits = 16384 rows
    hq, hkv, cap, batch = 64, 1, 65536, 2
    dq = torch.zeros((1, batch, hq, D), dtype=torch.float16, device="cuda")
    dk = torch.zeros((batch, hkv, cap, D), dtype=torch.float16, device="cuda")
    dout = torch.zeros_like(dq)
    op = ellm_amd.Attention(dq, dk, dk, dout, batch, hq, hkv, D, [hkv * cap * D, cap * D, D, 1], 0.1,
                            sequence_capacity=cap, max_position_interval=1)
    with pytest.raises(ellm_amd.EllmError) as e:
        op.run_noalloc(cap - 1, batch)
    assert e.value.status == 3 and "static scratch" in e.value.message
    with pytest.raises(ellm_amd.EllmError):
        op.run_noalloc(cap, batch)           # position beyond the capacity
    op.run(cap - 1, 1, batch)                # the handle's path takes the same shape
    torch.cuda.synchronize()
    op.close()


def test_noalloc_takes_shapes_near_its_documented_limit():
    """97 sequences x 16 query heads on one K/V head, five splits a plane: 7760 of the 8192 partial
    rows the header promises (an earlier fit check also demanded cluster partials that a plan with
    at most 16 splits a plane never writes, and refused this shape)."""
    q, k, v = _case(61, 97, 16, 1, 1280, orc.F16)
    _check(q, k, v, orc.F16, batch=97, position=1279)
    # 40 sequences x 64 query heads on 4 K/V heads (groups of 16), three splits: 7680 rows
    q, k, v = _case(71, 40, 64, 4, 1024, orc.F16)
    _check(q, k, v, orc.F16, batch=40, position=1023)


def test_noalloc_recorded_into_a_graph_replays_like_eager():
    """The stated use: the call recorded once into a graph (counter clear + attention, both kernel
    nodes) and replayed while the per-sequence positions move on inside the graph; eager work and
    synchronisations between replays.  Every replay equals the eager call bit for bit, and the last
    one the oracle."""
    import torch

    import ellm_amd

    dtype = orc.F16
    bcap, hq, hkv, cap = 6, 32, 4, 3000
    q, k, v = _case(81, bcap, hq, hkv, cap, dtype)
    scale = 1.0 / np.sqrt(D)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    dout = torch.full_like(dq, float("nan"))
    dlse = torch.full((1, bcap, hq), float("nan"), dtype=torch.float32, device="cuda")
    op = ellm_amd.Attention(dq, dk, dv, dout, bcap, hq, hkv, D, [hkv * cap * D, cap * D, D, 1], scale,
                            lse=dlse, sequence_capacity=cap, max_position_interval=1)
    start = np.array([2500, 3, 64, 1000, 127, 1999], dtype=np.uint32)
    steps, by = 4, 41
    stream = torch.cuda.Stream()

    def walk(use_graph):
        pos = torch.from_numpy(start.view(np.int32).copy()).cuda()
        outs, graph = [], None
        with torch.cuda.stream(stream):
            for _ in range(steps):
                dout.fill_(float("nan"))

                def step():
                    op.run_noalloc(cap - 1, bcap, positions=pos, stream=stream)
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
        return outs

    try:
        eager = walk(False)
        replay = walk(True)
        for n in range(steps):
            assert np.array_equal(eager[n][0], replay[n][0]), n
            assert np.array_equal(eager[n][1].view(np.uint32), replay[n][1].view(np.uint32)), n
        last = start + (steps - 1) * by
        want, want_lse = orc.attention(q, k, v, scale, dtype, positions=last, batch=bcap)
        got = orc.from_storage(replay[-1][0].view(np.uint16), dtype)
        r = compare(got, orc.from_storage(want, dtype), dtype)
        assert r["ok"], r
        assert np.abs(replay[-1][1] - want_lse).max() <= 1e-4
    finally:
        op.close()
