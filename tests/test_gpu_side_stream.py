"""The two halves of a mixed step (a prompt chunk of one sequence, one new token of the others)
issued side by side through ellm_side_stream_*: same bits as one after the other on one
stream, eagerly and replayed from a recorded graph, and within tolerance of the oracle."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, compare, rand_storage, to_dev, to_host

pytestmark = pytest.mark.gpu

B, HQ, HKV, CAP = 5, 8, 2, 700
P0, CHUNK = 300, 200
START = np.array([650, 33, 257, 511], dtype=np.int32)   # last cached position of sequences 1..4
SCALE = 0.11


def _setup(dtype):
    import torch

    import ellm_amd

    k = rand_storage((B, HKV, CAP, D), 401, dtype, scale=1.5)
    v = rand_storage((B, HKV, CAP, D), 402, dtype)
    qc = rand_storage((CHUNK, 1, HQ, D), 403, dtype)
    qt = rand_storage((1, B - 1, HQ, D), 404, dtype)
    dk, dv, dqc, dqt = to_dev(k, dtype), to_dev(v, dtype), to_dev(qc, dtype), to_dev(qt, dtype)
    oc, ot = torch.zeros_like(dqc), torch.zeros_like(dqt)
    strides = [HKV * CAP * D, CAP * D, D, 1]
    chunk_op = ellm_amd.Attention(dqc, dk, dv, oc, 1, HQ, HKV, D, strides, SCALE,
                                  sequence_capacity=CAP, max_position_interval=CHUNK)
    token_op = ellm_amd.Attention(dqt, dk[1:], dv[1:], ot, B - 1, HQ, HKV, D, strides, SCALE,
                                  sequence_capacity=CAP, max_position_interval=1)
    return dict(k=k, v=v, qc=qc, qt=qt, dk=dk, dv=dv, dqc=dqc, dqt=dqt, oc=oc, ot=ot,
                chunk_op=chunk_op, token_op=token_op)


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16], ids=["f16", "bf16"])
def test_side_by_side_equals_one_after_the_other(dtype):
    import torch

    import ellm_amd

    s = _setup(dtype)
    stream = torch.cuda.Stream()
    side = ellm_amd.SideStream()
    pos = torch.tensor(START, dtype=torch.int32, device="cuda")
    max_pos = CAP - 1

    def one_after_the_other():
        s["chunk_op"].run(P0, CHUNK, 1, stream=stream)
        s["token_op"].run_ragged(pos, max_pos, B - 1, stream=stream)

    def side_by_side():
        side.fork(stream)
        s["token_op"].run_ragged(pos, max_pos, B - 1, stream=side)
        s["chunk_op"].run(P0, CHUNK, 1, stream=stream)
        side.join(stream)

    torch.cuda.synchronize()
    one_after_the_other()
    stream.synchronize()
    want_c, want_t = s["oc"].clone(), s["ot"].clone()
    for _ in range(3):
        s["oc"].zero_()
        s["ot"].zero_()
        torch.cuda.synchronize()
        side_by_side()
        stream.synchronize()     # the join makes the caller's stream wait for the side stream too
        assert torch.equal(s["oc"], want_c) and torch.equal(s["ot"], want_t)

    # against the oracle
    ref_c, _ = orc.attention(s["qc"], s["k"][:1], s["v"][:1], SCALE, dtype, position_index=P0)
    assert compare(to_host(want_c, dtype), orc.from_storage(ref_c, dtype), dtype)["ok"]
    ref_t, _ = orc.attention(s["qt"], s["k"][1:], s["v"][1:], SCALE, dtype, positions=START.astype(np.uint32))
    assert compare(to_host(want_t, dtype), orc.from_storage(ref_t, dtype), dtype)["ok"]

    # recorded: the side launches are a parallel branch of the graph; the positions move on
    # inside the graph, so every replay attends to one more key per sequence
    with ellm_amd.StepGraph(stream) as graph:
        side.fork(stream)
        s["token_op"].run_ragged(pos, max_pos, B - 1, stream=side)
        ellm_amd.positions_advance(pos, 1, stream=side)
        s["chunk_op"].run(P0, CHUNK, 1, stream=stream)
        side.join(stream)
    eager_pos = torch.tensor(START, dtype=torch.int32, device="cuda")
    for replay in range(4):
        s["oc"].zero_()
        s["ot"].zero_()
        torch.cuda.synchronize()
        graph.launch()
        stream.synchronize()
        got_c, got_t = s["oc"].clone(), s["ot"].clone()
        assert np.array_equal(pos.cpu().numpy(), START + replay + 1)
        # the same step, eagerly, on one stream (and some unrelated work between the replays)
        s["oc"].zero_()
        s["ot"].zero_()
        s["chunk_op"].run(P0, CHUNK, 1, stream=stream)
        s["token_op"].run_ragged(eager_pos, max_pos, B - 1, stream=stream)
        ellm_amd.positions_advance(eager_pos, 1, stream=stream)
        stream.synchronize()
        assert torch.equal(got_c, s["oc"]) and torch.equal(got_t, s["ot"]), replay
    assert not torch.equal(got_t, want_t)     # the replays did see other lengths than the first step
    graph.close()
    side.close()
    s["chunk_op"].close()
    s["token_op"].close()


def test_side_stream_argument_checks():
    import ellm_amd

    lib = ellm_amd.load_library()
    assert lib.ellm_side_stream_create(None) != 0
    assert lib.ellm_side_stream_fork(None, None) != 0
    assert b"null side stream" in lib.ellm_last_error_string()
    assert lib.ellm_side_stream_join(None, None) != 0
    assert lib.ellm_side_stream_get(None) is None
    assert lib.ellm_side_stream_destroy(None) == 0
