"""A request walked with the library's schedule (chunked prompt, then single tokens), the
single-token steps replayed from a graph recorded through the C ABI (ellm_graph_*), against
the same walk launched eagerly and against the oracle."""
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


def test_chunked_prompt_then_recorded_single_token_steps():
    import torch

    import ellm_amd

    dtype = orc.F16
    b, hq, hkv, cap = 2, 8, 2, 512
    prompt, chunk, generate = 150, 64, 5
    total = prompt + generate
    calls = ellm_amd.schedule_calls(0, prompt, chunk, total)
    assert calls[:3] == [(0, 64), (64, 64), (128, 22)] and calls[3:] == [(150 + i, 1) for i in range(5)]
    rope = _rope_table(cap, dtype)
    k_all = rand_storage((total, b, hkv, D), 61, dtype, scale=2.0)
    v_all = rand_storage((total, b, hkv, D), 62, dtype)
    q_all = rand_storage((total, b, hq, D), 63, dtype)

    def walk(use_graph):
        stream = torch.cuda.Stream()
        cache = ellm_amd.KVCache(1, b, hkv, cap, ellm_amd.DTYPE_F16)
        kt, vt = cache.layer_tensors(0, torch_dtype(dtype))
        _, _, strides = cache.layer(0)
        dk_all, dv_all, dq_all = to_dev(k_all, dtype), to_dev(v_all, dtype), to_dev(q_all, dtype)
        drope = to_dev(rope, dtype)
        out_all = torch.zeros_like(dq_all)
        # the chunked prompt: one operator over the whole Q / O buffers (as the reference's
        # static graph has), run per call of the schedule
        qbuf = torch.zeros((chunk, b, hq, D), dtype=torch.float16, device="cuda")
        obuf = torch.zeros_like(qbuf)
        op = ellm_amd.Attention(qbuf, kt, vt, obuf, b, hq, hkv, D, strides, 0.2,
                                sequence_capacity=cap, max_position_interval=chunk)
        q1 = torch.zeros((1, b, hq, D), dtype=torch.float16, device="cuda")
        o1 = torch.zeros_like(q1)
        k1 = torch.zeros((1, b, hkv, D), dtype=torch.float16, device="cuda")
        v1 = torch.zeros_like(k1)
        op1 = ellm_amd.Attention(q1, kt, vt, o1, b, hq, hkv, D, strides, 0.2,
                                 sequence_capacity=cap, max_position_interval=1)
        pos = torch.full((b,), prompt, dtype=torch.int32, device="cuda")
        graph = None
        with torch.cuda.stream(stream):
            for (p0, n) in calls:
                if n > 1 or p0 < prompt:
                    cache.append_norm_rope(0, p0, dk_all[p0:p0 + n], dv_all[p0:p0 + n], drope)
                    qbuf[:n].copy_(dq_all[p0:p0 + n])
                    op.run(p0, n, b)
                    out_all[p0:p0 + n].copy_(obuf[:n])
                    continue
                q1.copy_(dq_all[p0:p0 + 1])
                k1.copy_(dk_all[p0:p0 + 1])
                v1.copy_(dv_all[p0:p0 + 1])

                def step():
                    cache.append_norm_rope(0, 0, k1, v1, drope, positions=pos, max_position=total)
                    op1.run_ragged(pos, total, b)
                    ellm_amd.positions_advance(pos, 1)

                if not use_graph:
                    step()
                else:
                    if graph is None:
                        stream.synchronize()
                        with ellm_amd.StepGraph(stream) as graph:
                            step()
                    graph.launch()
                out_all[p0:p0 + 1].copy_(o1)
                stream.synchronize()
                _ = float(o1.float().sum())            # eager work between replays
        stream.synchronize()
        res = to_host(out_all, dtype).copy(), to_host(kt, dtype).copy(), pos.cpu().numpy()
        if graph is not None:
            graph.close()
        op.close()
        op1.close()
        cache.close()
        return res

    out_e, k_e, pos_e = walk(False)
    out_g, k_g, pos_g = walk(True)
    assert np.array_equal(pos_e, [total] * b) and np.array_equal(pos_g, [total] * b)
    assert np.array_equal(out_e, out_g) and np.array_equal(k_e, k_g)
    # oracle: rotate all keys, then one causal pass over the whole request
    kc = np.zeros((b, hkv, cap, D), dtype=np.float16)
    vc = np.zeros_like(kc)
    assert orc.kv_append_norm_rope(kc, vc, 0, k_all, v_all, rope, 1e-6, dtype) == 0
    want, _ = orc.attention(q_all, kc, vc, 0.2, dtype, position_index=0)
    assert compare(out_g, orc.from_storage(want, dtype), dtype)["ok"]


def test_graph_rejects_the_null_stream():
    import ellm_amd

    lib = ellm_amd.load_library()
    assert lib.ellm_graph_begin(None) != 0
    assert b"null stream" in lib.ellm_last_error_string()
