"""Two handles driven from two streams at once: a handle's workspace and arrival counters are its own,
so launches of different handles may overlap; each must give what it gives alone, bit for bit."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, rand_storage, to_dev

pytestmark = pytest.mark.gpu


def test_two_handles_on_two_streams_overlap_without_interference():
    import torch

    import ellm_amd

    dtype = orc.F16
    scale = 1.0 / np.sqrt(D)
    shapes = [(4, 32, 4, 6000), (3, 16, 2, 9000)]       # both split their planes: partials, counters, folds
    ops, bufs, alone = [], [], []
    for n, (b, hq, hkv, cap) in enumerate(shapes):
        q = to_dev(rand_storage((1, b, hq, D), 91 + n, dtype), dtype)
        k = to_dev(rand_storage((b, hkv, cap, D), 93 + n, dtype), dtype)
        v = to_dev(rand_storage((b, hkv, cap, D), 95 + n, dtype), dtype)
        out = torch.zeros_like(q)
        pos = torch.tensor([cap - 1 - 97 * i for i in range(b)], dtype=torch.int32, device="cuda")
        ops.append(ellm_amd.Attention(q, k, v, out, b, hq, hkv, D, [hkv * cap * D, cap * D, D, 1], scale,
                                      sequence_capacity=cap, max_position_interval=1))
        bufs.append((q, k, v, out, pos, b, cap))
    try:
        for op, (q, k, v, out, pos, b, cap) in zip(ops, bufs):
            res = []
            op.run(cap - 1, 1, b)
            torch.cuda.synchronize()
            res.append(out.view(torch.int16).cpu().numpy().copy())
            op.run_ragged(pos, cap - 1, b)
            torch.cuda.synchronize()
            res.append(out.view(torch.int16).cpu().numpy().copy())
            alone.append(res)
        streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        for ragged in (False, True):
            for rep in range(20):
                for n, (op, (q, k, v, out, pos, b, cap)) in enumerate(zip(ops, bufs)):
                    with torch.cuda.stream(streams[n]):
                        out.zero_()
                        if ragged:
                            op.run_ragged(pos, cap - 1, b, stream=streams[n])
                        else:
                            op.run(cap - 1, 1, b, stream=streams[n])
                for n in range(2):
                    streams[n].synchronize()
                    got = bufs[n][3].view(torch.int16).cpu().numpy()
                    assert np.array_equal(got, alone[n][1 if ragged else 0]), (ragged, rep, n)
    finally:
        for op in ops:
            op.close()
