"""One attention layer of a single-token step, end to end through the C ABI: fused Q/K/V
projection (writes the cache in place) -> attention over the cache -> output projection +
residual -> positions advanced on the device; launched eagerly and replayed from a graph
recorded through the library.  Every stage is checked against the oracle run on that
stage's own inputs as the GPU produced them, with the stage's tolerance."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, compare, compare_ulps, rand_storage, to_dev, to_host, torch_dtype

pytestmark = pytest.mark.gpu


def _rope_table(positions, dtype, theta=1.0e6):
    jj = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(positions, dtype=np.float64)[:, None] * theta ** (-2.0 * jj / D)[None, :]
    t = np.empty((positions, D), dtype=np.float32)
    t[:, 0::2], t[:, 1::2] = np.cos(ang), np.sin(ang)
    return orc.to_storage(t, dtype)


def test_layer_step_eager_graph_and_oracle():
    import torch

    import ellm_amd

    dtype = orc.F16
    b, hq, hkv, cap, hidden = 5, 8, 2, 256, 512
    steps = 3
    start = np.array([17, 0, 200, 64, 99], dtype=np.int32)
    scale = 1.0 / np.sqrt(D)
    rope = _rope_table(cap, dtype)
    wq = rand_storage((hq * D, hidden), 1, dtype, scale=hidden ** -0.5)
    wk = rand_storage((hkv * D, hidden), 2, dtype, scale=hidden ** -0.5)
    wv = rand_storage((hkv * D, hidden), 3, dtype, scale=hidden ** -0.5)
    wo = rand_storage((hidden, hq * D), 4, dtype, scale=(hq * D) ** -0.5)
    k0 = rand_storage((b, hkv, cap, D), 5, dtype)
    v0 = rand_storage((b, hkv, cap, D), 6, dtype)
    xs = rand_storage((steps, 1, b, hidden), 7, dtype)

    def run(use_graph):
        stream = torch.cuda.Stream()
        cache = ellm_amd.KVCache(1, b, hkv, cap, ellm_amd.DTYPE_F16)
        kt, vt = cache.layer_tensors(0, torch_dtype(dtype))
        kt.copy_(to_dev(k0, dtype))
        vt.copy_(to_dev(v0, dtype))
        _, _, strides = cache.layer(0)
        x = torch.zeros((1, b, hidden), dtype=torch.float16, device="cuda")
        q = torch.zeros((1, b, hq, D), dtype=torch.float16, device="cuda")
        att = torch.zeros_like(q)
        out = torch.zeros_like(x)
        dev = [to_dev(a, dtype) for a in (wq, wk, wv, wo, rope)]
        qkv = ellm_amd.MatMul3(x, dev[0], q, dev[1], kt, dev[2], vt, dev[4], D, b, hq, hkv, strides, cap)
        attn = ellm_amd.Attention(q, kt, vt, att, b, hq, hkv, D, strides, scale, sequence_capacity=cap,
                                  max_position_interval=1)
        oproj = ellm_amd.MatMulAdd(att.view(1, b, hq * D), dev[3], x, out)   # residual = the layer input
        pos = torch.from_numpy(start.copy()).cuda()
        max_pos = int(start.max()) + steps
        results, graph = [], None
        with torch.cuda.stream(stream):
            def step():
                qkv.run_ragged(pos, max_pos, b)
                attn.run_ragged(pos, max_pos, b)
                oproj.run(0, 1, b)
                ellm_amd.positions_advance(pos, 1)

            for s in range(steps):
                x.copy_(to_dev(xs[s], dtype))
                stream.synchronize()
                if not use_graph:
                    step()
                else:
                    if graph is None:
                        with ellm_amd.StepGraph(stream) as graph:
                            step()
                    graph.launch()
                stream.synchronize()
                results.append(tuple(to_host(t, dtype).copy() for t in (q, att, out)) + (to_host(kt, dtype).copy(),
                                                                                         to_host(vt, dtype).copy()))
                _ = float(out.float().sum())      # eager work between replays
        final_pos = pos.cpu().numpy()
        if graph is not None:
            graph.close()
        for op in (qkv, attn, oproj):
            op.close()
        cache.close()
        return results, final_pos

    eager, pos_e = run(False)
    replay, pos_g = run(True)
    assert np.array_equal(pos_e, start + steps) and np.array_equal(pos_g, start + steps)
    for s in range(steps):
        for a, c in zip(eager[s], replay[s]):
            assert np.array_equal(a, c), s                     # same kernels, same bits

    # oracle, stage by stage, on the inputs the GPU stages saw
    kc, vc = k0.copy(), v0.copy()
    for s in range(steps):
        gq, gatt, gout, gk, gv = replay[s]
        positions = (start + s).astype(np.uint32)
        oq = np.zeros((1, b, hq, D), dtype=np.uint16)
        assert orc.matmul3(xs[s], wq, wk, wv, oq, kc, vc, rope, (hkv * cap * D, cap * D, D, 1), cap, 0, 1, dtype,
                           positions=positions) == 0
        assert compare_ulps(gq, orc.from_storage(oq, dtype), dtype)["ok"]
        assert compare_ulps(gk, orc.from_storage(kc, dtype), dtype)["ok"]
        assert compare_ulps(gv, orc.from_storage(vc, dtype), dtype)["ok"]
        # attention on the GPU's own q and cache (stage tolerance, not accumulated)
        sq, sk, sv = (orc.to_storage(a, dtype) for a in (gq, gk, gv))
        want_att, _ = orc.attention(sq, sk, sv, scale, dtype, positions=positions)
        assert compare(gatt, orc.from_storage(want_att, dtype), dtype)["ok"]
        # output projection on the GPU's attention rows
        satt = orc.to_storage(gatt.reshape(1, b, hq * D), dtype)
        want_out = orc.matmul_add(satt, wo, xs[s], dtype)
        assert compare_ulps(gout, orc.from_storage(want_out, dtype), dtype)["ok"]
        # carry the GPU's cache forward so that later steps stay stage-local
        kc, vc = sk.copy(), sv.copy()


def test_chunked_prefill_projection_feeds_attention():
    """Two chunks of a prompt: the fused projection writes each chunk's K/V into the cache at
    its positions and the chunk's queries to the scratch, attention then reads the cache
    up to each query's position; stagewise against the oracle."""
    import torch

    import ellm_amd

    dtype = orc.BF16
    b, hq, hkv, cap, hidden = 2, 4, 2, 512, 256
    chunks = [(0, 300), (300, 77)]
    scale = 1.0 / np.sqrt(D)
    rope = _rope_table(cap, dtype)
    wq = rand_storage((hq * D, hidden), 11, dtype, scale=hidden ** -0.5)
    wk = rand_storage((hkv * D, hidden), 12, dtype, scale=hidden ** -0.5)
    wv = rand_storage((hkv * D, hidden), 13, dtype, scale=hidden ** -0.5)
    xs = rand_storage((377, b, hidden), 14, dtype)

    cache = ellm_amd.KVCache(1, b, hkv, cap, ellm_amd.DTYPE_BF16)
    kt, vt = cache.layer_tensors(0, torch_dtype(dtype))
    kt.zero_()
    vt.zero_()
    _, _, strides = cache.layer(0)
    x = torch.zeros((300, b, hidden), dtype=torch.bfloat16, device="cuda")
    q = torch.zeros((300, b, hq, D), dtype=torch.bfloat16, device="cuda")
    att = torch.zeros_like(q)
    dev = [to_dev(a, dtype) for a in (wq, wk, wv, rope)]
    qkv = ellm_amd.MatMul3(x, dev[0], q, dev[1], kt, dev[2], vt, dev[3], D, b, hq, hkv, strides, cap)
    attn = ellm_amd.Attention(q, kt, vt, att, b, hq, hkv, D, strides, scale, sequence_capacity=cap,
                              max_position_interval=300)
    kc = np.zeros((b, hkv, cap, D), dtype=np.uint16)
    vc = np.zeros_like(kc)
    for p0, n in chunks:
        x[:n].copy_(to_dev(xs[p0:p0 + n], dtype))
        qkv.run(p0, n, b)
        attn.run(p0, n, b)
        torch.cuda.synchronize()
        gq, gatt = to_host(q, dtype)[:n], to_host(att, dtype)[:n]
        gk, gv = to_host(kt, dtype), to_host(vt, dtype)
        oq = np.zeros((n, b, hq, D), dtype=np.uint16)
        assert orc.matmul3(np.ascontiguousarray(xs[p0:p0 + n]), wq, wk, wv, oq, kc, vc, rope,
                           (hkv * cap * D, cap * D, D, 1), cap, p0, n, dtype) == 0
        assert compare_ulps(gq, orc.from_storage(oq, dtype), dtype)["ok"]
        assert compare_ulps(gk, orc.from_storage(kc, dtype), dtype)["ok"]
        assert compare_ulps(gv, orc.from_storage(vc, dtype), dtype)["ok"]
        sq, sk, sv = (orc.to_storage(a, dtype) for a in (gq, gk, gv))
        want, _ = orc.attention(sq, sk, sv, scale, dtype, position_index=p0)
        assert compare(gatt, orc.from_storage(want, dtype), dtype)["ok"]
        kc, vc = sk.copy(), sv.copy()
    qkv.close()
    attn.close()
    cache.close()


def test_recorded_chunk_step_on_a_long_cache_replays_like_eager():
    """A prompt chunk's attention block (fused projection on one-head tiles -> chunk attention with
    its key range split over workgroups and merged -> output projection) recorded once and
    replayed with fresh activations: every replay equals the eager run of the same inputs bit
    for bit, and the first one matches the oracle."""
    import torch

    import ellm_amd

    dtype = orc.F16
    b, hq, hkv, cap, hidden, p0, n = 2, 8, 2, 2048, 256, 1700, 70
    scale = 1.0 / np.sqrt(D)
    rope = _rope_table(cap, dtype)
    wq = rand_storage((hq * D, hidden), 21, dtype, scale=hidden ** -0.5)
    wk = rand_storage((hkv * D, hidden), 22, dtype, scale=hidden ** -0.5)
    wv = rand_storage((hkv * D, hidden), 23, dtype, scale=hidden ** -0.5)
    wo = rand_storage((hidden, hq * D), 24, dtype, scale=(hq * D) ** -0.5)
    k0 = rand_storage((b, hkv, cap, D), 25, dtype)
    v0 = rand_storage((b, hkv, cap, D), 26, dtype)
    lib = ellm_amd.load_library()
    assert lib.ellm_projection_path(n * b, hq + 2 * hkv, hidden) in (1, 2)

    cache = ellm_amd.KVCache(1, b, hkv, cap, ellm_amd.DTYPE_F16)
    kt, vt = cache.layer_tensors(0, torch.float16)
    _, _, strides = cache.layer(0)
    x = torch.zeros((n, b, hidden), dtype=torch.float16, device="cuda")
    q = torch.zeros((n, b, hq, D), dtype=torch.float16, device="cuda")
    att = torch.zeros_like(q)
    res = torch.zeros((n, b, hidden), dtype=torch.float16, device="cuda")
    out = torch.zeros_like(res)
    dev = [to_dev(a, dtype) for a in (wq, wk, wv, rope, wo)]
    qkv = ellm_amd.MatMul3(x, dev[0], q, dev[1], kt, dev[2], vt, dev[3], D, b, hq, hkv, strides, cap)
    attn = ellm_amd.Attention(q, kt, vt, att, b, hq, hkv, D, strides, scale, sequence_capacity=cap,
                              max_position_interval=n)
    oproj = ellm_amd.MatMulAdd(att.view(n, b, hq * D), dev[4], res, out)

    def step(stream):
        qkv.run(p0, n, b, stream=stream)
        attn.run(p0, n, b, stream=stream)
        oproj.run(p0, n, b, stream=stream)

    def fresh(i):
        kt.copy_(to_dev(k0, dtype))
        vt.copy_(to_dev(v0, dtype))
        x.copy_(to_dev(rand_storage((n, b, hidden), 100 + i, dtype), dtype))
        res.copy_(to_dev(rand_storage((n, b, hidden), 200 + i, dtype), dtype))
        out.zero_()
        att.zero_()

    stream = torch.cuda.Stream()
    eager = []
    for i in range(3):
        fresh(i)
        torch.cuda.synchronize()
        step(stream)
        stream.synchronize()
        eager.append((att.clone(), out.clone(), kt.clone()))
    with ellm_amd.StepGraph(stream) as graph:
        step(stream)
    for i in range(3):
        fresh(i)
        torch.cuda.synchronize()
        graph.launch()
        stream.synchronize()
        for got, want in zip((att, out, kt), eager[i]):
            assert torch.equal(got, want), i
    # the first inputs against the oracle: projection rows, then attention over the cache they wrote
    fresh(0)
    torch.cuda.synchronize()
    graph.launch()
    stream.synchronize()
    gq, gatt = to_host(q, dtype), to_host(att, dtype)
    sk, sv = (orc.to_storage(to_host(t, dtype), dtype) for t in (kt, vt))
    want, _ = orc.attention(orc.to_storage(gq, dtype), sk, sv, scale, dtype, position_index=p0)
    assert compare(gatt, orc.from_storage(want, dtype), dtype)["ok"]
    want_out = orc.matmul_add(orc.to_storage(gatt, dtype).reshape(n, b, hq * D), wo,
                              rand_storage((n, b, hidden), 200, dtype), dtype, batch_size=b)
    assert compare_ulps(to_host(out, dtype), orc.from_storage(want_out, dtype), dtype)["ok"]
    graph.close()
    for op in (qkv, attn, oproj):
        op.close()
    cache.close()


def test_recorded_long_chunk_uses_the_large_projection_tiles():
    """A chunk long enough for the 256 x 256 projection tiles (the one kernel here that needs
    per-wave scratch memory), recorded and replayed: equal to the eager run bit for bit."""
    import torch

    import ellm_amd

    dtype = orc.F16
    n, b, hq, hkv, hidden = 5700, 1, 8, 2, 64
    cap = n
    lib = ellm_amd.load_library()
    assert lib.ellm_projection_path(n, hq + 2 * hkv, hidden) == 3
    rope = _rope_table(cap, dtype)
    w = [rand_storage((h * D, hidden), 31 + i, dtype, scale=hidden ** -0.5) for i, h in enumerate((hq, hkv, hkv))]
    cache = ellm_amd.KVCache(1, b, hkv, cap, ellm_amd.DTYPE_F16)
    kt, vt = cache.layer_tensors(0, torch.float16)
    _, _, strides = cache.layer(0)
    x = torch.zeros((n, b, hidden), dtype=torch.float16, device="cuda")
    q = torch.zeros((n, b, hq, D), dtype=torch.float16, device="cuda")
    att = torch.zeros_like(q)
    dev = [to_dev(a, dtype) for a in (*w, rope)]
    qkv = ellm_amd.MatMul3(x, dev[0], q, dev[1], kt, dev[2], vt, dev[3], D, b, hq, hkv, strides, cap)
    attn = ellm_amd.Attention(q, kt, vt, att, b, hq, hkv, D, strides, 1.0 / np.sqrt(D), sequence_capacity=cap,
                              max_position_interval=n)
    stream = torch.cuda.Stream()

    def step():
        qkv.run(0, n, b, stream=stream)
        attn.run(0, n, b, stream=stream)

    def fresh(i):
        x.copy_(to_dev(rand_storage((n, b, hidden), 300 + i, dtype), dtype))
        for t in (q, att, kt, vt):
            t.zero_()

    eager = []
    for i in range(2):
        fresh(i)
        torch.cuda.synchronize()
        step()
        stream.synchronize()
        eager.append((q.clone(), att.clone(), kt.clone(), vt.clone()))
    with ellm_amd.StepGraph(stream) as graph:
        step()
    for i in range(2):
        fresh(i)
        torch.cuda.synchronize()
        graph.launch()
        stream.synchronize()
        for got, want in zip((q, att, kt, vt), eager[i]):
            assert torch.equal(got, want), i
    # a few rows of the projection against the oracle (rows as sequences of a one-token call)
    rows = np.array([0, 255, 256, 4095, 5699], dtype=np.uint32)
    hid = rand_storage((n, b, hidden), 301, dtype)[rows, 0][None]
    oq = np.zeros((1, len(rows), hq, D), dtype=np.uint16)
    okc = np.zeros((len(rows), hkv, cap, D), dtype=np.uint16)
    ovc = np.zeros_like(okc)
    assert orc.matmul3(np.ascontiguousarray(hid), *w, oq, okc, ovc, rope, (hkv * cap * D, cap * D, D, 1), cap, 0, 1,
                       dtype, positions=rows) == 0
    assert compare_ulps(to_host(q, dtype)[rows, 0], orc.from_storage(oq, dtype)[0], dtype)["ok"]
    graph.close()
    qkv.close()
    attn.close()
    cache.close()
