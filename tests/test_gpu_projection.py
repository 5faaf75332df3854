"""Parity of the projections either side of attention (ellm_matmul3_*, ellm_matmul_add_*)
with the oracle, through the C ABI.  Tolerance: one unit in the last place of the storage
type (both sides accumulate in binary32 and round once)."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, compare_ulps, rand_storage, to_dev, to_host, torch_dtype

pytestmark = pytest.mark.gpu


def _rope_table(positions, dtype, theta=1.0e6):
    jj = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(positions, dtype=np.float64)[:, None] * theta ** (-2.0 * jj / D)[None, :]
    t = np.empty((positions, D), dtype=np.float32)
    t[:, 0::2], t[:, 1::2] = np.cos(ang), np.sin(ang)
    return orc.to_storage(t, dtype)


def _code(dtype):
    import ellm_amd

    return ellm_amd.DTYPE_F16 if dtype == orc.F16 else ellm_amd.DTYPE_BF16


def _run_matmul3(hidden, wq, wk, wv, rope, dtype, pitch, hq, hkv, cap, p0, interval, batch,
                 positions=None, reference_layout=False, rope_strides=(D, 0)):
    """GPU and oracle on the same inputs; returns ((q, k, v) gpu, (q, k, v) oracle) decoded."""
    import torch

    import ellm_amd

    cap_i = hidden.shape[0]
    dq = torch.zeros((cap_i, pitch, hq, D), dtype=torch_dtype(dtype), device="cuda")
    if reference_layout:   # k_state [position][sequence][head][128], read through permuted strides
        dk = torch.zeros((cap, pitch, hkv, D), dtype=torch_dtype(dtype), device="cuda")
        dv = torch.zeros_like(dk)
        strides = (hkv * D, D, pitch * hkv * D, 1)
        cache = None
    else:
        cache = ellm_amd.KVCache(1, pitch, hkv, cap, _code(dtype))
        dk, dv = cache.layer_tensors(0, torch_dtype(dtype))
        dk.zero_()
        dv.zero_()
        _, _, strides = cache.layer(0)
    keep = [to_dev(a, dtype) for a in (hidden, wq, wk, wv, rope)]
    op = ellm_amd.MatMul3(keep[0], keep[1], dq, keep[2], dk, keep[3], dv, keep[4], D, pitch, hq, hkv,
                          strides, cap, rope_position_stride=rope_strides[0],
                          rope_head_stride=rope_strides[1], max_position_interval=cap_i)
    if positions is not None:
        dpos = torch.from_numpy(positions.astype(np.int32)).cuda()
        op.run_ragged(dpos, int(positions.max()), batch)
    else:
        op.run(p0, interval, batch)
    torch.cuda.synchronize()
    got = (to_host(dq, dtype), to_host(dk, dtype), to_host(dv, dtype))
    op.close()
    if cache is not None:
        cache.close()
    oq = np.zeros((cap_i, pitch, hq, D), dtype=np.uint16)
    ok = np.zeros(tuple(dk.shape), dtype=np.uint16)
    ov = np.zeros_like(ok)
    assert orc.matmul3(hidden, wq, wk, wv, oq, ok, ov, rope, strides, cap, p0, interval, dtype,
                       batch_size=batch, positions=positions, rope_position_stride=rope_strides[0],
                       rope_head_stride=rope_strides[1]) == 0
    want = tuple(orc.from_storage(a, dtype) for a in (oq, ok, ov))
    return got, want


def _weights(k, hq, hkv, dtype, seed):
    s = k ** -0.5
    return (rand_storage((hq * D, k), seed, dtype, scale=s), rand_storage((hkv * D, k), seed + 1, dtype, scale=s),
            rand_storage((hkv * D, k), seed + 2, dtype, scale=s))


FEW_ROWS, TILES_128, TILES_256X1, TILES_256X2 = 0, 1, 2, 3     # ellm_projection_path


def _path(rows, heads, k):
    import ellm_amd

    return ellm_amd.load_library().ellm_projection_path(rows, heads, k)


CASES = [
    # interval, pitch, batch, k, hq, hkv, cap, p0, dtype
    # 128-token x one-head tiles (more than 64 rows, and no more tiles than compute units)
    (300, 1, 1, 256, 8, 2, 512, 17, orc.F16),      # three token tiles, the last partial
    (513, 1, 1, 192, 2, 2, 1024, 3, orc.BF16),     # five token tiles, bfloat16
    (33, 5, 4, 64, 3, 1, 64, 9, orc.BF16),         # one chunk of K, odd head count
    # 256-token x one-head tiles
    (9, 100, 97, 2048, 32, 4, 64, 7, orc.F16),     # 897 rows of the benchmark model, sequences beyond batch_size skipped
    (79, 128, 101, 64, 3, 1, 128, 5, orc.BF16),    # 10085 rows: last tile partial, odd head count, one chunk of K
    # 256 x 256 tiles (many rows; K kept small so that the oracle stays quick)
    (2081, 8, 5, 64, 3, 1, 4096, 9, orc.F16),      # 16645 rows: last token tile partial, odd head count, batch < pitch
    (130, 128, 128, 128, 2, 2, 256, 3, orc.BF16),  # 16640 rows, bfloat16, two chunks of K
    (5, 7, 5, 64, 3, 1, 64, 9, orc.F16),           # odd head count, sequences beyond batch_size skipped
    (1, 16, 16, 2048, 32, 4, 256, 100, orc.F16),   # the single-token step of the benchmark model
    (40, 3, 2, 128, 4, 4, 64, 0, orc.BF16),
    # few rows (the weight-streaming kernel): two token blocks x two column blocks, rows through LDS
    (2, 16, 12, 2048, 32, 4, 64, 5, orc.F16),
    (1, 16, 16, 1024, 4, 2, 64, 9, orc.BF16),      # four waves, one column block
    (1, 8, 8, 8192, 2, 1, 32, 3, orc.F16),         # two rounds of K per wave, operands fetched directly
    (2, 12, 12, 4096, 34, 2, 32, 1, orc.F16),      # wide output but rows too long for two column blocks in LDS
    # 33 .. 64 rows: several passes over weight operands kept in registers
    (1, 60, 57, 2048, 32, 4, 64, 7, orc.F16),      # 57 rows: two passes of two token blocks, last one partial
    (3, 20, 20, 1024, 6, 2, 64, 2, orc.BF16),      # 60 rows, four waves: four passes of one token block
    (2, 32, 32, 4096, 3, 1, 32, 0, orc.F16),       # 64 rows, sixteen waves
    # 65 .. 128 rows: one 128-token tile per head
    (1, 100, 97, 2048, 32, 4, 64, 7, orc.F16),
    (3, 40, 40, 1024, 6, 2, 64, 2, orc.BF16),
    (2, 64, 64, 4096, 3, 1, 32, 0, orc.F16),
]


@pytest.mark.parametrize("interval,pitch,batch,k,hq,hkv,cap,p0,dtype", CASES)
def test_matmul3_against_the_oracle(interval, pitch, batch, k, hq, hkv, cap, p0, dtype):
    hidden = rand_storage((interval, pitch, k), 11, dtype)
    wq, wk, wv = _weights(k, hq, hkv, dtype, 20)
    rope = _rope_table(cap, dtype)
    got, want = _run_matmul3(hidden, wq, wk, wv, rope, dtype, pitch, hq, hkv, cap, p0, interval, batch)
    for name, g, w in zip("qkv", got, want):
        r = compare_ulps(g, w, dtype)
        assert r["ok"], (name, r)
    # rows of sequences beyond batch_size and positions outside the call stay untouched (zero)
    assert not got[0][:, batch:].any()
    assert not got[1][batch:].any() and not got[1][:, :, :p0].any() and not got[1][:, :, p0 + interval:].any()


def test_cases_reach_every_projection_kernel():
    seen = {_path((i - 1) * pitch + b, hq + 2 * hkv, k) for (i, pitch, b, k, hq, hkv, _, _, _) in CASES}
    every = {FEW_ROWS, TILES_128, TILES_256X1, TILES_256X2}
    assert seen == every, seen
    seen = {_path((i - 1) * pitch + b, n // D, k) for (i, pitch, b, k, n, _) in ADD_CASES}
    assert seen == every, seen
    # the benchmark shapes: 32768 rows on the large tiles, the reference's serving shape
    # (64 positions x 24 sequences, src/serving/start copy.rs:30) on the one-head tiles
    assert _path(32768, 40, 2048) == TILES_256X2 and _path(32768, 16, 4096) == TILES_256X2
    assert _path(64 * 24, 40, 2048) == TILES_256X1 and _path(64 * 24, 16, 4096) == TILES_128
    assert _path(16, 40, 2048) == FEW_ROWS


def test_matmul3_ragged_step_of_many_sequences():
    """A single-token step of more sequences than the few-rows kernel takes: per-sequence
    positions on the tile kernel."""
    dtype = orc.F16
    pitch, batch, k, hq, hkv, cap = 200, 150, 256, 3, 2, 96
    assert _path(batch, hq + 2 * hkv, k) == TILES_128
    hidden = rand_storage((1, pitch, k), 61, dtype)
    wq, wk, wv = _weights(k, hq, hkv, dtype, 62)
    rope = _rope_table(cap, dtype)
    pos = np.random.default_rng(63).integers(0, cap, size=pitch).astype(np.uint32)
    got, want = _run_matmul3(hidden, wq, wk, wv, rope, dtype, pitch, hq, hkv, cap, 0, 1, batch, positions=pos)
    for g, w in zip(got, want):
        assert compare_ulps(g, w, dtype)["ok"]
    assert not got[1][batch:].any()


def test_matmul3_ragged_single_token_step():
    dtype = orc.F16
    pitch, batch, k, hq, hkv, cap = 9, 6, 128, 4, 2, 128
    hidden = rand_storage((1, pitch, k), 31, dtype)
    wq, wk, wv = _weights(k, hq, hkv, dtype, 32)
    rope = _rope_table(cap, dtype)
    pos = np.array([0, 127, 5, 64, 33, 99, 1, 2, 3], dtype=np.uint32)
    got, want = _run_matmul3(hidden, wq, wk, wv, rope, dtype, pitch, hq, hkv, cap, 0, 1, batch, positions=pos)
    for g, w in zip(got, want):
        assert compare_ulps(g, w, dtype)["ok"]
    assert not got[1][batch:].any()


def test_matmul3_in_the_reference_state_layout_and_table_indexing():
    """k_state / v_state as the reference keeps them ([position][sequence][head][128], read by
    attention through permuted strides) and its rotary table indexed by output column only
    (position stride 0, head stride 128: src/compiler/mul/matmul3.rs:243-251)."""
    dtype = orc.F16
    pitch, batch, k, hq, hkv, cap = 24, 24, 64, 3, 3, 4       # test_tensor_matmul3_f16_seq1_batch24's batch
    hidden = rand_storage((1, pitch, k), 41, dtype)
    wq, wk, wv = _weights(k, hq, hkv, dtype, 42)
    rope = rand_storage((max(hq, hkv) * D,), 45, dtype)
    got, want = _run_matmul3(hidden, wq, wk, wv, rope, dtype, pitch, hq, hkv, cap, 2, 1, batch,
                             reference_layout=True, rope_strides=(0, D))
    for g, w in zip(got, want):
        assert compare_ulps(g, w, dtype)["ok"]
    assert got[1][2].any() and not got[1][:2].any() and not got[1][3:].any()     # only position 2 written


ADD_CASES = [
    (300, 1, 1, 512, 256, orc.F16),                # 128-token tiles
    (257, 2, 2, 128, 128, orc.F16),
    (65, 24, 20, 4096, 256, orc.BF16),             # 1556 rows of which 20 in 24 live, K of the benchmark model
    (1250, 4, 4, 64, 1536, orc.F16),               # 256-token x one-head tiles: 5000 rows, last tile partial
    (600, 12, 9, 128, 640, orc.BF16),              # same tiles: 7197 rows of which 9 in 12 live, bfloat16
    (4100, 4, 3, 64, 640, orc.F16),                # 256 x 256 tiles: 16399 rows, last tile partial, odd head count
    (2049, 8, 8, 192, 512, orc.BF16),              # 16392 rows, bfloat16, three chunks of K
    (3, 5, 4, 64, 384, orc.BF16),
    (1, 16, 16, 4096, 2048, orc.F16),              # the output projection of the benchmark model, one token
    (1, 8, 8, 2048, 256, orc.BF16),                # few rows, bfloat16
    (2, 16, 10, 2048, 4096, orc.F16),              # few rows, two token blocks, wide output
    (1, 64, 64, 2048, 256, orc.F16),               # 64 rows, two passes
    (3, 20, 13, 4096, 128, orc.BF16),              # 53 rows of which 39 live, sixteen waves
    (1, 128, 128, 2048, 256, orc.F16),             # 128 rows: one 128-token tile per head
    (5, 20, 13, 4096, 128, orc.BF16),              # 93 rows of which 65 live
]


@pytest.mark.parametrize("interval,pitch,batch,k,n,dtype", ADD_CASES)
def test_matmul_add_against_the_oracle(interval, pitch, batch, k, n, dtype):
    import torch

    import ellm_amd

    a = rand_storage((interval, pitch, k), 51, dtype)
    w = rand_storage((n, k), 52, dtype, scale=k ** -0.5)
    r = rand_storage((interval, pitch, n), 53, dtype)
    da, dw, dr = to_dev(a, dtype), to_dev(w, dtype), to_dev(r, dtype)
    out = torch.zeros_like(dr)
    op = ellm_amd.MatMulAdd(da, dw, dr, out)
    op.run(0, interval, batch)
    torch.cuda.synchronize()
    got = to_host(out, dtype)
    want = orc.from_storage(orc.matmul_add(a, w, r, dtype, batch_size=batch), dtype)
    res = compare_ulps(got, want, dtype)
    assert res["ok"], res
    assert not got[:, batch:].any()
    op.close()
    # in place: the output may be the residual buffer
    op = ellm_amd.MatMulAdd(da, dw, dr, dr)
    op.run(0, interval, batch)
    torch.cuda.synchronize()
    got2 = to_host(dr, dtype)
    assert np.array_equal(got2[:, :batch], got[:, :batch])
    op.close()


def test_matmul3_full_size_properties():
    """The benchmark shape (32768 tokens x 2048 -> 40 heads): properties that do not need the
    oracle on all of it (unit RMS of every normalised head row, value rows against a library
    product) plus the oracle on 24 rows spread over the token range."""
    import torch

    import ellm_amd

    dtype = orc.F16
    tokens, k, hq, hkv = 32768, 2048, 32, 4
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    x = torch.randn((tokens, 1, k), generator=g, device="cuda").to(torch.float16)
    wq = (torch.randn((hq * D, k), generator=g, device="cuda") * k ** -0.5).to(torch.float16)
    wk = (torch.randn((hkv * D, k), generator=g, device="cuda") * k ** -0.5).to(torch.float16)
    wv = (torch.randn((hkv * D, k), generator=g, device="cuda") * k ** -0.5).to(torch.float16)
    rope_np = _rope_table(tokens, dtype)
    rope = to_dev(rope_np, dtype)
    q = torch.zeros((tokens, 1, hq, D), dtype=torch.float16, device="cuda")
    cache = ellm_amd.KVCache(1, 1, hkv, tokens, ellm_amd.DTYPE_F16)
    kt, vt = cache.layer_tensors(0, torch.float16)
    _, _, strides = cache.layer(0)
    op = ellm_amd.MatMul3(x, wq, q, wk, kt, wv, vt, rope, D, 1, hq, hkv, strides, tokens)
    op.run(0, tokens, 1)
    torch.cuda.synchronize()
    # rotations keep the norm of every pair: each stored head row has unit RMS up to rounding
    for t in (q.float(), kt.float()):
        rms = t.pow(2).mean(-1).sqrt()
        assert float((rms - 1).abs().max()) < 2e-3
    # value rows: plain products (library GEMM in binary32 as the second opinion)
    v_lib = (x[:, 0].float() @ wv.float().T).view(tokens, hkv, D).permute(1, 0, 2)
    assert float((vt[0].float() - v_lib).abs().max()) < 4e-3          # 1 ulp of binary16 below 4, values reach ~4
    # oracle on selected rows: the rows become sequences of a one-token call at their positions
    rows = np.unique(np.concatenate((np.arange(0, tokens, 1489), [255, 256, 32767]))).astype(np.uint32)
    hid = np.ascontiguousarray(x[torch.from_numpy(rows.astype(np.int64)).cuda(), 0].view(torch.int16).cpu().numpy().view(np.uint16))[None]
    host = [t.view(torch.int16).cpu().numpy().view(np.uint16) for t in (wq, wk, wv)]
    n = len(rows)
    oq = np.zeros((1, n, hq, D), dtype=np.uint16)
    okc = np.zeros((n, hkv, tokens, D), dtype=np.uint16)
    ovc = np.zeros_like(okc)
    assert orc.matmul3(hid, *host, oq, okc, ovc, rope_np, (hkv * tokens * D, tokens * D, D, 1), tokens, 0, 1,
                       dtype, positions=rows) == 0
    gq = to_host(q, dtype)[rows, 0]
    gk = to_host(kt, dtype)[0][:, rows]
    gv = to_host(vt, dtype)[0][:, rows]
    wq_rows = orc.from_storage(oq, dtype)[0]
    wk_rows = np.stack([orc.from_storage(okc[i, :, rows[i]], dtype) for i in range(n)], axis=1)
    wv_rows = np.stack([orc.from_storage(ovc[i, :, rows[i]], dtype) for i in range(n)], axis=1)
    assert compare_ulps(gq, wq_rows, dtype)["ok"]
    assert compare_ulps(gk, wk_rows, dtype)["ok"]
    assert compare_ulps(gv, wv_rows, dtype)["ok"]
    op.close()
    cache.close()


def test_matmul3_and_matmul_add_random_shapes():
    """A seeded sweep over shapes that cross the dispatch boundaries (few rows / passes / small
    tiles, K a multiple of 64 or of 256, one or two column blocks, odd head counts, partial
    batches, ragged positions)."""
    import torch

    import ellm_amd

    rng = np.random.default_rng(2024)
    for case in range(24):
        dtype = orc.F16 if case % 3 else orc.BF16
        k = int(rng.choice([64, 192, 256, 512, 1024, 1280, 2048]))
        hq = int(rng.integers(1, 7))
        hkv = int(rng.integers(1, 4))
        if case % 6 == 0:
            hq, hkv = 30, 2                      # wide output: two column blocks in the few-rows kernel
        pitch = int(rng.integers(1, 20))
        batch = int(rng.integers(1, pitch + 1))
        interval = int(rng.choice([1, 1, 2, 7, 40, 150])) if k <= 1024 else int(rng.choice([1, 1, 3, 30]))
        cap = 64 if interval <= 64 else 256
        p0 = int(rng.integers(0, cap - interval + 1))
        ragged = interval == 1 and case % 2 == 0
        hidden = rand_storage((interval, pitch, k), 1000 + case, dtype)
        wq, wk, wv = _weights(k, hq, hkv, dtype, 2000 + 3 * case)
        rope = _rope_table(cap, dtype)
        positions = rng.integers(0, cap, size=pitch).astype(np.uint32) if ragged else None
        got, want = _run_matmul3(hidden, wq, wk, wv, rope, dtype, pitch, hq, hkv, cap, 0 if ragged else p0,
                                 interval, batch, positions=positions)
        for name, g, w in zip("qkv", got, want):
            r = compare_ulps(g, w, dtype)
            assert r["ok"], (case, name, dict(k=k, hq=hq, hkv=hkv, pitch=pitch, batch=batch, interval=interval), r)
        # output projection on the same activations: k -> n
        n = 128 * int(rng.integers(1, 5))
        w = rand_storage((n, k), 3000 + case, dtype, scale=k ** -0.5)
        res = rand_storage((interval, pitch, n), 4000 + case, dtype)
        da, dw, dr = to_dev(hidden, dtype), to_dev(w, dtype), to_dev(res, dtype)
        out = torch.zeros_like(dr)
        op = ellm_amd.MatMulAdd(da, dw, dr, out)
        op.run(0, interval, batch)
        torch.cuda.synchronize()
        g = to_host(out, dtype)
        wnt = orc.from_storage(orc.matmul_add(hidden, w, res, dtype, batch_size=batch), dtype)
        r = compare_ulps(g, wnt, dtype)
        assert r["ok"], (case, "add", dict(k=k, n=n, pitch=pitch, batch=batch, interval=interval), r)
        assert not g[:, batch:].any()
        op.close()
