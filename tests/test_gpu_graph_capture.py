"""The entry points of a single-token step (cache write with key norm + rotation, then
attention with per-sequence positions read from device memory) recorded into a HIP graph
and replayed: every replay must equal the eager result for the positions of that step.
Nothing in these entry points allocates, synchronises or clears memory with a memset, so
they can be captured; the positions advance on the device between replays."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, compare, rand_storage, to_dev, to_host, torch_dtype

pytestmark = pytest.mark.gpu


def _rope_table(positions, dtype, theta=1.0e6):
    jj = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(positions, dtype=np.float64)[:, None] * theta ** (-2.0 * jj / D)[None, :]
    t = np.empty((positions, D), dtype=np.float32)
    t[:, 0::2], t[:, 1::2] = np.cos(ang), np.sin(ang)
    return orc.to_storage(t, dtype)


def test_decode_step_replayed_from_a_graph_matches_eager_and_the_oracle():
    import torch

    import ellm_amd

    dtype = orc.F16
    b, hq, hkv, cap, layers = 6, 16, 2, 2048, 2
    start = np.array([700, 3, 1500, 64, 1023, 2000], dtype=np.int32)   # ragged cache lengths
    steps = 4
    rope = _rope_table(cap, dtype)
    # the caches already hold `start[i]` tokens per sequence (plain rows; only new keys are rotated)
    k0 = rand_storage((layers, b, hkv, cap, D), 51, dtype)
    v0 = rand_storage((layers, b, hkv, cap, D), 52, dtype)
    new_k = rand_storage((steps, layers, 1, b, hkv, D), 53, dtype, scale=2.0)
    new_v = rand_storage((steps, layers, 1, b, hkv, D), 54, dtype)
    qs = rand_storage((steps, layers, 1, b, hq, D), 55, dtype)

    def run(use_graph):
        cache = ellm_amd.KVCache(layers, b, hkv, cap, ellm_amd.DTYPE_F16)
        ops, outs, dq, dk, dv = [], [], [], [], []
        for l in range(layers):
            kt, vt = cache.layer_tensors(l, torch_dtype(dtype))
            kt.copy_(to_dev(k0[l], dtype))
            vt.copy_(to_dev(v0[l], dtype))
            _, _, strides = cache.layer(l)
            q = torch.zeros((1, b, hq, D), dtype=torch.float16, device="cuda")
            out = torch.zeros_like(q)
            ops.append(ellm_amd.Attention(q, kt, vt, out, b, hq, hkv, D, strides, 0.11,
                                          sequence_capacity=cap, max_position_interval=1))
            outs.append(out)
            dq.append(q)
            dk.append(torch.zeros((1, b, hkv, D), dtype=torch.float16, device="cuda"))
            dv.append(torch.zeros((1, b, hkv, D), dtype=torch.float16, device="cuda"))
        drope = to_dev(rope, dtype)
        pos = torch.from_numpy(start.copy()).cuda()
        max_pos = int(start.max()) + steps

        def one_step():
            for l in range(layers):
                cache.append_norm_rope(l, 0, dk[l], dv[l], drope, positions=pos, max_position=max_pos)
                ops[l].run_ragged(pos, max_pos, b)
            pos.add_(1)

        def feed(s):
            for l in range(layers):
                dq[l].copy_(to_dev(qs[s, l], dtype))
                dk[l].copy_(to_dev(new_k[s, l], dtype))
                dv[l].copy_(to_dev(new_v[s, l], dtype))

        results = []
        graph = None
        if use_graph:
            side = torch.cuda.Stream()
            feed(0)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                with torch.cuda.graph(graph, stream=side):
                    one_step()
            torch.cuda.synchronize()
            # capture does not execute: positions and caches are still at the start
        for s in range(steps):
            feed(s)
            torch.cuda.synchronize()
            if use_graph:
                graph.replay()
            else:
                one_step()
            torch.cuda.synchronize()
            results.append([to_host(o, dtype).copy() for o in outs])
            _ = (dq[0].float() * 2).sum().item()      # eager work and a sync between replays
        final_k = [to_host(cache.layer_tensors(l, torch_dtype(dtype))[0], dtype).copy() for l in range(layers)]
        final_pos = pos.cpu().numpy()
        for op in ops:
            op.close()
        cache.close()
        return results, final_k, final_pos

    eager, k_eager, pos_eager = run(False)
    replay, k_replay, pos_replay = run(True)
    assert np.array_equal(pos_eager, start + steps) and np.array_equal(pos_replay, start + steps)
    for s in range(steps):
        for l in range(layers):
            assert np.array_equal(eager[s][l], replay[s][l]), (s, l)   # same kernels, same bits
    for l in range(layers):
        assert np.array_equal(k_eager[l], k_replay[l])

    # and against the oracle pipeline for the last step of layer 1
    l = 1
    kc, vc = k0[l].copy(), v0[l].copy()
    for s in range(steps):
        assert orc.kv_append_norm_rope(kc, vc, 0, new_k[s, l], new_v[s, l], rope, 1e-6, dtype,
                                       positions=start + s) == 0
    want, _ = orc.attention(qs[steps - 1, l], kc, vc, 0.11, dtype,
                            positions=(start + steps - 1).astype(np.uint32))
    assert compare(replay[steps - 1][l], orc.from_storage(want, dtype), dtype)["ok"]
