"""The benchmark configurations at their full sizes: parity with the CPU oracle (all rows
where the oracle finishes in seconds, a seeded sample of rows otherwise) and
size-independent properties."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, LSE_TOL, compare, rand_storage, to_dev, to_host, torch_dtype

pytestmark = pytest.mark.gpu


def _device_normal(shape, seed, dtype, scale=None):
    """Seeded N(0,1) generated on the device (fast for 10^8 values), optionally scaled
    per head; returned as a device tensor in the storage type."""
    import torch

    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    x = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32)
    if scale is not None:
        x = x * scale
    return x.to(torch_dtype(dtype))


def _host(t, dtype):
    """Device tensor -> numpy storage array (float16, or uint16 bit patterns for bfloat16)."""
    import torch

    a = t.contiguous().view(torch.int16).cpu().numpy()
    return a.view(np.float16) if dtype == orc.F16 else a.view(np.uint16)


def _make_op(dq, dk, dv, bcap, hq, hkv, cap, scale, interval):
    import torch

    import ellm_amd

    dout = torch.full_like(dq, float("nan"))
    dlse = torch.full((dq.shape[0], bcap, hq), float("nan"), dtype=torch.float32, device="cuda")
    op = ellm_amd.Attention(dq, dk, dv, dout, bcap, hq, hkv, D, [hkv * cap * D, cap * D, D, 1],
                            scale, lse=dlse, sequence_capacity=cap, max_position_interval=interval)
    return op, dout, dlse


def _check_rows(op_or, rows, p0, dout, dlse, dtype, n_threads=8):
    want, want_lse, _ = op_or.run_rows(p0, rows, n_threads)
    got = to_host(dout, dtype)[rows[:, 0], rows[:, 1], rows[:, 2]]
    got_lse = dlse.cpu().numpy()[rows[:, 0], rows[:, 1], rows[:, 2]]
    res = compare(got, orc.from_storage(want, dtype), dtype)
    lse_err = float(np.abs(got_lse - want_lse).max())
    print(res, f"lse_err={lse_err:.2e}", flush=True)
    assert res["ok"], res
    assert lse_err <= LSE_TOL, lse_err


def test_config0_prefill_512_mha_in_a_4096_cache():
    """Batch 1, 512 tokens, 32 query = 32 KV heads, binary16, inputs N(0,1)/sqrt(128), cache
    preallocated at 4096 positions and filled from position 0 through the append entry
    point.  Plumbing is bit-for-bit (cache contents, untouched positions), values to tolerance."""
    import torch

    import ellm_amd

    dtype, s, h, cap = orc.F16, 512, 32, 4096
    sc = 1.0 / np.sqrt(D)
    q = rand_storage((s, 1, h, D), 101, dtype, scale=sc)
    ksrc = rand_storage((s, 1, h, D), 102, dtype, scale=sc)      # [token][seq][kv_head][D]
    vsrc = rand_storage((s, 1, h, D), 103, dtype, scale=sc)
    cache = ellm_amd.KVCache(1, 1, h, cap, ellm_amd.DTYPE_F16)
    cache.append(0, 0, to_dev(ksrc, dtype), to_dev(vsrc, dtype))
    kt, vt = cache.layer_tensors(0, torch.float16)
    torch.cuda.synchronize()
    k = np.zeros((1, h, cap, D), dtype=np.float16)
    v = np.zeros_like(k)
    k[:, :, :s] = ksrc.transpose(1, 2, 0, 3)
    v[:, :, :s] = vsrc.transpose(1, 2, 0, 3)
    assert np.array_equal(_host(kt, dtype), k) and np.array_equal(_host(vt, dtype), v)
    dq = to_dev(q, dtype)
    op, dout, dlse = _make_op(dq, kt, vt, 1, h, h, cap, sc, s)
    op.run(0, s, 1)
    torch.cuda.synchronize()
    want, want_lse = orc.attention(q, k, v, sc, dtype, position_index=0)
    res = compare(to_host(dout, dtype), orc.from_storage(want, dtype), dtype)
    lse_err = float(np.abs(dlse.cpu().numpy() - want_lse).max())
    print(res, f"lse_err={lse_err:.2e}", flush=True)
    assert res["ok"] and lse_err <= LSE_TOL
    # token 0 sees one key: its output is that value row, exactly
    assert np.array_equal(to_host(dout, dtype)[0, 0], orc.from_storage(v, dtype)[0, :, 0])
    op.close()
    cache.close()


def test_config1_decode_16_sequences_8192_tokens():
    """32 query / 4 KV heads, 16 independent sequences, 8192 cached tokens each, binary16,
    K/V/q ~ N(0,1): every output row against the oracle."""
    import torch

    dtype, b, hq, hkv, length = orc.F16, 16, 32, 4, 8192
    sc = 1.0 / np.sqrt(D)
    dq = _device_normal((1, b, hq, D), 111, dtype)
    dk = _device_normal((b, hkv, length, D), 112, dtype)
    dv = _device_normal((b, hkv, length, D), 113, dtype)
    op, dout, dlse = _make_op(dq, dk, dv, b, hq, hkv, length, sc, 1)
    op.run(length - 1, 1, b)
    torch.cuda.synchronize()
    q, k, v = _host(dq, dtype), _host(dk, dtype), _host(dv, dtype)
    want, want_lse = orc.attention(q, k, v, sc, dtype, position_index=length - 1)
    res = compare(to_host(dout, dtype), orc.from_storage(want, dtype), dtype)
    lse_err = float(np.abs(dlse.cpu().numpy() - want_lse).max())
    print(res, f"lse_err={lse_err:.2e}", flush=True)
    assert res["ok"] and lse_err <= LSE_TOL
    op.close()


def test_decode_one_sequence_131072_tokens():
    """The headline single-token case: one sequence with a 128k-token cache."""
    import torch

    dtype, hq, hkv, length = orc.F16, 32, 4, 131072
    sc = 1.0 / np.sqrt(D)
    dq = _device_normal((1, 1, hq, D), 121, dtype)
    dk = _device_normal((1, hkv, length, D), 122, dtype)
    dv = _device_normal((1, hkv, length, D), 123, dtype)
    op, dout, dlse = _make_op(dq, dk, dv, 1, hq, hkv, length, sc, 1)
    op.run(length - 1, 1, 1)
    torch.cuda.synchronize()
    want, want_lse = orc.attention(_host(dq, dtype), _host(dk, dtype), _host(dv, dtype), sc, dtype,
                                   position_index=length - 1)
    res = compare(to_host(dout, dtype), orc.from_storage(want, dtype), dtype)
    lse_err = float(np.abs(dlse.cpu().numpy() - want_lse).max())
    print(res, f"lse_err={lse_err:.2e}", flush=True)
    assert res["ok"] and lse_err <= LSE_TOL
    op.close()


def test_config2_prefill_32768_tokens():
    """Batch 1, 32 query / 4 KV heads, 32768 tokens in one pass, binary16, N(0,1) with a
    per-head scale ~ U[0.5, 2].  The oracle checks a seeded sample of (token, head) rows
    (the full problem is 4.4e12 MACs); constant-V and chunk invariance cover every row."""
    import torch

    dtype, s, hq, hkv = orc.F16, 32768, 32, 4
    sc = 1.0 / np.sqrt(D)
    g = torch.Generator(device="cuda")
    g.manual_seed(130)
    qs = torch.rand((1, 1, hq, 1), generator=g, device="cuda") * 1.5 + 0.5
    ks = torch.rand((1, hkv, 1, 1), generator=g, device="cuda") * 1.5 + 0.5
    vs = torch.rand((1, hkv, 1, 1), generator=g, device="cuda") * 1.5 + 0.5
    dq = _device_normal((s, 1, hq, D), 131, dtype, scale=qs)
    dk = _device_normal((1, hkv, s, D), 132, dtype, scale=ks)
    dv = _device_normal((1, hkv, s, D), 133, dtype, scale=vs)
    op, dout, dlse = _make_op(dq, dk, dv, 1, hq, hkv, s, sc, s)
    op.run(0, s, 1)
    torch.cuda.synchronize()
    q, k, v = _host(dq, dtype), _host(dk, dtype), _host(dv, dtype)
    rng = np.random.default_rng(134)
    toks = np.concatenate([[0, 1, 31, 32, 63, 64, 65, 127, 128, s - 1, s - 32, s - 33],
                           rng.integers(0, s, 116)])
    rows = np.stack([toks, np.zeros_like(toks), rng.integers(0, hq, toks.size)], 1).astype(np.uint32)
    ref_op = orc.Operator(q, k, v, np.zeros((1,), np.float16), None, 1, hq, hkv, D,
                          [hkv * s * D, s * D, D, 1], sc, dtype)
    _check_rows(ref_op, rows, 0, dout, dlse, dtype)

    # chunk invariance at full size: two passes of 16384 tokens give the same rows
    whole = dout.clone()
    whole_lse = dlse.clone()
    dout.fill_(float("nan"))
    half = s // 2
    import ellm_amd
    op2 = ellm_amd.Attention(dq[half:], dk, dv, dout[half:], 1, hq, hkv, D,
                             [hkv * s * D, s * D, D, 1], sc, lse=dlse[half:],
                             sequence_capacity=s, max_position_interval=half)
    op.run(0, half, 1)
    op2.run(half, half, 1)
    torch.cuda.synchronize()
    res = compare(to_host(dout, dtype), to_host(whole, dtype), dtype)
    print("two chunks vs one pass:", res, flush=True)
    assert res["ok"]
    assert float((dlse - whole_lse).abs().max()) <= LSE_TOL

    # constant V: every output element equals the constant, whatever the weights are
    dv.fill_(0.75)
    op.run(0, s, 1)
    torch.cuda.synchronize()
    assert float((dout.float() - 0.75).abs().max()) <= 2.0 ** -11
    op.close()
    op2.close()


def test_config3_chunk_of_8192_on_a_120000_token_cache_bf16():
    """64 query / 8 KV heads, bfloat16, cache pre-filled with 120000 tokens, a chunk of 8192
    new tokens attends causally to all 128192 positions; compared with the oracle on a
    seeded subset of 4 heads."""
    import torch

    dtype, hq, hkv, p0, s = orc.BF16, 64, 8, 120000, 8192
    cap = p0 + s
    sc = 1.0 / np.sqrt(D)
    dq = _device_normal((s, 1, hq, D), 141, dtype)
    dk = _device_normal((1, hkv, cap, D), 142, dtype)
    dv = _device_normal((1, hkv, cap, D), 143, dtype)
    op, dout, dlse = _make_op(dq, dk, dv, 1, hq, hkv, cap, sc, s)
    op.run(p0, s, 1)
    torch.cuda.synchronize()
    q, k, v = _host(dq, dtype), _host(dk, dtype), _host(dv, dtype)
    rng = np.random.default_rng(144)
    heads = rng.choice(hq, 4, replace=False)
    toks = np.concatenate([[0, 31, 32, s - 1], rng.integers(0, s, 8)])
    rows = np.array([[t, 0, h] for h in heads for t in toks], dtype=np.uint32)
    ref_op = orc.Operator(q, k, v, np.zeros((1,), np.uint16), None, 1, hq, hkv, D,
                          [hkv * cap * D, cap * D, D, 1], sc, dtype)
    _check_rows(ref_op, rows, p0, dout, dlse, dtype)
    # with ~124k keys per row the outputs are small: they also meet the binary16 bound
    want, _, _ = ref_op.run_rows(p0, rows, 8)
    got = to_host(dout, dtype)[rows[:, 0], rows[:, 1], rows[:, 2]]
    assert np.abs(got - orc.from_storage(want, dtype)).max() <= 2e-3
    op.close()


def test_config4_mixed_step_over_layers_reduced():
    """One step at the graph level, attention only: per layer, one sequence prefills a chunk
    while the other sequences decode one token against caches of different lengths.  Full
    size (48 layers, 16384-token prefill, 32 decoding sequences up to 131072 tokens) needs
    208 GB of cache; this runs 2 layers, a 4096-token prefill and 6 decoding sequences with
    lengths drawn from [1024, 32768], through one [layer][sequence][kv_head][position][128]
    cache object, and checks sampled rows of both kinds in both layers."""
    import torch

    import ellm_amd

    dtype, hq, hkv = orc.F16, 32, 4
    layers, n_dec, s_pf, cap = 2, 6, 4096, 32768
    sc = 1.0 / np.sqrt(D)
    rng = np.random.default_rng(150)
    lengths = rng.integers(1024, cap + 1, n_dec)
    cache = ellm_amd.KVCache(layers, 1 + n_dec, hkv, cap, ellm_amd.DTYPE_F16)
    stream = torch.cuda.current_stream()
    ops, bufs = [], []
    for layer in range(layers):
        kt, vt = cache.layer_tensors(layer, torch.float16)
        kt.copy_(_device_normal(tuple(kt.shape), 151 + layer, dtype))
        vt.copy_(_device_normal(tuple(vt.shape), 161 + layer, dtype))
        q_pf = _device_normal((s_pf, 1, hq, D), 171 + layer, dtype)
        q_dec = _device_normal((1, n_dec, hq, D), 181 + layer, dtype)
        _, _, strides = cache.layer(layer)
        op_pf, out_pf, lse_pf = _make_op(q_pf, kt, vt, 1, hq, hkv, cap, sc, s_pf)
        # the decoding sequences are slots 1.. of the same cache: base pointer of slot 1
        op_dec, out_dec, lse_dec = _make_op(q_dec, kt[1:], vt[1:], n_dec, hq, hkv, cap, sc, 1)
        ops.append((op_pf, op_dec))
        bufs.append((kt, vt, q_pf, q_dec, out_pf, lse_pf, out_dec, lse_dec))
    dpos = torch.from_numpy((lengths - 1).astype(np.int32)).cuda()
    for op_pf, op_dec in ops:          # one stream, launches in graph order
        op_pf.run(0, s_pf, 1, stream=stream)
        op_dec.run_ragged(dpos, int(lengths.max() - 1), n_dec, stream=stream)
    torch.cuda.synchronize()
    for layer in range(layers):
        kt, vt, q_pf, q_dec, out_pf, lse_pf, out_dec, lse_dec = bufs[layer]
        k, v = _host(kt, dtype), _host(vt, dtype)
        strides = [hkv * cap * D, cap * D, D, 1]
        ref_pf = orc.Operator(_host(q_pf, dtype), k, v, np.zeros((1,), np.float16), None, 1, hq,
                              hkv, D, strides, sc, dtype)
        toks = np.concatenate([[0, 63, s_pf - 1], rng.integers(0, s_pf, 13)])
        rows = np.stack([toks, np.zeros_like(toks), rng.integers(0, hq, toks.size)], 1)
        _check_rows(ref_pf, rows.astype(np.uint32), 0, out_pf, lse_pf, dtype)
        want, want_lse = orc.attention(_host(q_dec, dtype), k[1:], v[1:], sc, dtype,
                                       positions=(lengths - 1).astype(np.uint32))
        res = compare(to_host(out_dec, dtype), orc.from_storage(want, dtype), dtype)
        print("decode part:", res, flush=True)
        assert res["ok"]
        assert np.abs(lse_dec.cpu().numpy() - want_lse).max() <= LSE_TOL
    for op_pf, op_dec in ops:
        op_pf.close()
        op_dec.close()
    cache.close()


def test_config4_one_layer_at_its_real_shape_ragged_cache():
    """One layer of the mixed step at full size, projection -> cache -> attention: sequence 0
    prefills 16384 tokens while 32 sequences decode one token each against caches of lengths
    U{1024..131072} (seed 7, as bench.py draws them), all 33 in ONE cache object whose sequences
    have their own capacities (2.27 M positions: 2.3 GB each for K and V).  Q/K/V come from the
    fused projection with random-init binary16 weights; sampled prefill rows and every
    single-token row are checked against the oracle run on what the device holds, the
    projection's own rows against the oracle's projection within one unit in the last place."""
    import torch

    import ellm_amd

    dtype, hq, hkv, hidden_size, s_pf, n_dec = orc.F16, 32, 4, 2048, 16384, 32
    td = torch.float16
    sc = 1.0 / np.sqrt(D)
    lengths = np.random.default_rng(7).integers(1024, 131072 + 1, size=n_dec)
    caps = [s_pf] + [int((n + 63) // 64 * 64) for n in lengths]
    total = sum(caps)
    cache = ellm_amd.KVCache.ragged(1, caps, hkv, ellm_amd.DTYPE_F16)
    kt, vt = cache.layer_flat_tensors(0, td)              # [hkv, total, 128]
    for h in range(hkv):                                   # the caches already hold their tokens
        kt[h].copy_(_device_normal((total, D), 200 + h, dtype))
        vt[h].copy_(_device_normal((total, D), 210 + h, dtype))
    w = [_device_normal((heads * D, hidden_size), 220 + i, dtype) * hidden_size ** -0.5
         for i, heads in enumerate((hq, hkv, hkv))]
    w = [x.to(td) for x in w]
    jj = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(max(caps), dtype=np.float64)[:, None] * (1.0e6 ** (-2.0 * jj / D))[None, :]
    rope_h = np.empty((max(caps), D), dtype=np.float32)
    rope_h[:, 0::2], rope_h[:, 1::2] = np.cos(ang), np.sin(ang)
    rope_h = orc.to_storage(rope_h, dtype)
    rope = to_dev(rope_h, dtype)
    x_pf = _device_normal((s_pf, 1, hidden_size), 230, dtype)
    x_dec = _device_normal((1, n_dec, hidden_size), 231, dtype)
    q_pf = torch.zeros((s_pf, 1, hq, D), dtype=td, device="cuda")
    q_dec = torch.zeros((1, n_dec, hq, D), dtype=td, device="cuda")
    out_pf, out_dec = torch.full_like(q_pf, float("nan")), torch.full_like(q_dec, float("nan"))
    lse_pf = torch.zeros((s_pf, 1, hq), dtype=torch.float32, device="cuda")
    lse_dec = torch.zeros((1, n_dec, hq), dtype=torch.float32, device="cuda")
    v0, v1 = cache.layer_ragged(0, 0), cache.layer_ragged(0, 1)
    assert v1.capacities == caps[1:]
    proj_pf = ellm_amd.MatMul3(x_pf, w[0], q_pf, w[1], kt, w[2], vt, rope, D, 1, hq, hkv, v0.strides, 0,
                               seq_table=v0)
    proj_dec = ellm_amd.MatMul3(x_dec, w[0], q_dec, w[1], kt, w[2], vt, rope, D, n_dec, hq, hkv, v1.strides, 0,
                                seq_table=v1)
    att_pf = ellm_amd.Attention(q_pf, kt, vt, out_pf, 1, hq, hkv, D, v0.strides, sc, lse=lse_pf,
                                max_position_interval=s_pf, seq_table=v0)
    att_dec = ellm_amd.Attention(q_dec, kt, vt, out_dec, n_dec, hq, hkv, D, v1.strides, sc, lse=lse_dec,
                                 max_position_interval=1, seq_table=v1)
    pos = (lengths - 1).astype(np.int32)
    dpos = torch.from_numpy(pos).cuda()
    max_pos = int(pos.max())
    proj_pf.run(0, s_pf, 1)
    att_pf.run(0, s_pf, 1)
    proj_dec.run_ragged(dpos, max_pos, n_dec)
    att_dec.run_ragged(dpos, max_pos, n_dec)
    torch.cuda.synchronize()

    k_h, v_h = _host(kt, dtype), _host(vt, dtype)          # [hkv, total, 128]
    strides = [0, total * D, D, 1]
    offs = np.concatenate([[0], np.cumsum(caps)[:-1]])
    rng = np.random.default_rng(240)

    # projection rows: four windows of 16 prefill tokens and all 32 single tokens, 1 ulp
    wh = [_host(x, dtype) for x in w]
    xh_pf, xh_dec = _host(x_pf, dtype), _host(x_dec, dtype)
    qh_pf, qh_dec = _host(q_pf, dtype), _host(q_dec, dtype)

    def ulps(got, want):
        got, want = orc.from_storage(got, dtype), orc.from_storage(want, dtype)
        return float((np.abs(got - want) / storage_ulp_at(want)).max())

    def storage_ulp_at(want):
        return 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 0.125))) - 10)

    for t0 in (0, 5000, 12345, s_pf - 16):
        oq = np.zeros((16, 1, hq, D), dtype=np.float16)
        ok = np.zeros((1, hkv, s_pf, D), dtype=np.float16)
        ov = np.zeros_like(ok)
        assert orc.matmul3(np.ascontiguousarray(xh_pf[t0:t0 + 16]), wh[0], wh[1], wh[2], oq, ok, ov, rope_h,
                           [hkv * s_pf * D, s_pf * D, D, 1], s_pf, t0, 16, dtype) == 0
        worst = max(ulps(qh_pf[t0:t0 + 16], oq), ulps(k_h[:, t0:t0 + 16], ok[0, :, t0:t0 + 16]),
                    ulps(v_h[:, t0:t0 + 16], ov[0, :, t0:t0 + 16]))
        print(f"projection, prefill tokens {t0}..{t0 + 15}: worst {worst:.2f} ulp", flush=True)
        assert worst <= 1.0
    capmax = max(caps[1:])
    oq = np.zeros((1, n_dec, hq, D), dtype=np.float16)
    ok = np.zeros((n_dec, hkv, capmax, D), dtype=np.float16)
    ov = np.zeros_like(ok)
    assert orc.matmul3(xh_dec, wh[0], wh[1], wh[2], oq, ok, ov, rope_h, [hkv * capmax * D, capmax * D, D, 1],
                       capmax, 0, 1, dtype, positions=pos.astype(np.uint32)) == 0
    worst = ulps(qh_dec, oq)
    for i in range(n_dec):
        row = offs[1 + i] + pos[i]
        worst = max(worst, ulps(k_h[:, row], ok[i, :, pos[i]]), ulps(v_h[:, row], ov[i, :, pos[i]]))
    print(f"projection, single tokens: worst {worst:.2f} ulp", flush=True)
    assert worst <= 1.0
    del ok, ov

    # attention, prefill side: sampled (token, head) rows on the device's own Q/K/V
    ref_pf = orc.Operator(qh_pf, k_h, v_h, np.zeros((1,), np.float16), None, 1, hq, hkv, D, strides, sc, dtype)
    toks = np.concatenate([[0, 31, 63, 64, s_pf - 1], rng.integers(0, s_pf, 27)])
    rows = np.stack([toks, np.zeros_like(toks), rng.integers(0, hq, toks.size)], 1).astype(np.uint32)
    _check_rows(ref_pf, rows, 0, out_pf, lse_pf, dtype)
    # attention, single-token side: every (sequence, head) row
    got_dec, got_lse = to_host(out_dec, dtype), lse_dec.cpu().numpy()
    all_heads = np.array([[0, 0, h] for h in range(hq)], dtype=np.uint32)
    worst_abs = worst_lse = 0.0
    for i in range(n_dec):
        o = offs[1 + i]
        ref = orc.Operator(np.ascontiguousarray(qh_dec[:, i:i + 1]), k_h[:, o:], v_h[:, o:],
                           np.zeros((1,), np.float16), None, 1, hq, hkv, D, strides, sc, dtype)
        want, want_lse, _ = ref.run_rows(int(pos[i]), all_heads, 8)
        res = compare(got_dec[0, i], orc.from_storage(want, dtype), dtype)
        assert res["ok"], (i, int(lengths[i]), res)
        worst_abs = max(worst_abs, res["max_abs"])
        worst_lse = max(worst_lse, float(np.abs(got_lse[0, i] - want_lse).max()))
    print(f"single-token rows of 32 sequences ({int(lengths.sum())} cached tokens): max_abs {worst_abs:.2e} "
          f"lse_err {worst_lse:.2e}", flush=True)
    assert worst_lse <= LSE_TOL
    for op in (proj_pf, proj_dec, att_pf, att_dec):
        op.close()
    cache.close()


def test_config4_all_48_layers_first_middle_and_last_checked():
    """The mixed step of configs[4] as bench.py runs it (`mixed48`): 48 layers, each with its own
    random-init projection weights and its own K/V in one cache object with per-sequence capacities
    (223.6 GB resident), a 16384-token prefill of sequence 0 and one new token of 32 sequences with
    cache lengths U{1024..131072} (seed 7), projections writing K/V into the caches.  All 192 launches
    run in the benchmark's order on one stream; the outputs of layers 0, 23 and 47 are kept as they
    leave their layer and checked against the oracle on what the device holds for that layer: sampled
    prefill rows, every head of four of the 32 single-token sequences, and the projection's own rows
    of those within one unit in the last place."""
    import torch

    import ellm_amd

    dtype, hq, hkv, hidden, s_pf, n_dec, layers = orc.F16, 32, 4, 2048, 16384, 32, 48
    td = torch.float16
    sc = 1.0 / np.sqrt(D)
    lengths = np.random.default_rng(7).integers(1024, 131072 + 1, size=n_dec)
    caps = [s_pf] + [int((n + 63) // 64 * 64) for n in lengths]
    need = 2 * layers * hkv * sum(caps) * D * 2
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    if free < need + 8 * 2 ** 30:
        pytest.skip(f"needs {need / 2 ** 30:.0f} GiB of device memory for the 48 caches, {free / 2 ** 30:.0f} free")
    cache = ellm_amd.KVCache.ragged(layers, caps, hkv, ellm_amd.DTYPE_F16)
    total = sum(caps)
    offs = np.concatenate([[0], np.cumsum(caps)[:-1]])
    jj = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(max(caps), dtype=np.float64)[:, None] * (1.0e6 ** (-2.0 * jj / D))[None, :]
    rope_h = np.empty((max(caps), D), dtype=np.float32)
    rope_h[:, 0::2], rope_h[:, 1::2] = np.cos(ang), np.sin(ang)
    rope_h = orc.to_storage(rope_h, dtype)
    rope = to_dev(rope_h, dtype)
    x_pf = _device_normal((s_pf, 1, hidden), 310, dtype)
    x_dec = _device_normal((1, n_dec, hidden), 300, dtype)
    q_pf = torch.zeros((s_pf, 1, hq, D), dtype=td, device="cuda")
    q_dec = torch.zeros((1, n_dec, hq, D), dtype=td, device="cuda")
    out_pf, out_dec = torch.zeros_like(q_pf), torch.zeros_like(q_dec)
    lse_pf = torch.zeros((s_pf, 1, hq), dtype=torch.float32, device="cuda")
    lse_dec = torch.zeros((1, n_dec, hq), dtype=torch.float32, device="cuda")
    pos = (lengths - 1).astype(np.int32)
    dpos = torch.from_numpy(pos).cuda()
    max_pos = int(pos.max())
    ops, weights = [], []
    for layer in range(layers):
        kt, vt = cache.layer_flat_tensors(layer, td)
        kt.normal_()              # the sequences' caches already hold their tokens
        vt.normal_()
        v0, v1 = cache.layer_ragged(layer, 0), cache.layer_ragged(layer, 1)
        w = [(_device_normal((h * D, hidden), 700 + 3 * layer + i, dtype).float() * hidden ** -0.5).to(td)
             for i, h in enumerate((hq, hkv, hkv))]
        weights.append(w)
        ops.append((ellm_amd.MatMul3(x_pf, w[0], q_pf, w[1], kt, w[2], vt, rope, D, 1, hq, hkv, v0.strides, 0, seq_table=v0),
                    ellm_amd.Attention(q_pf, kt, vt, out_pf, 1, hq, hkv, D, v0.strides, sc, lse=lse_pf,
                                       max_position_interval=s_pf, seq_table=v0),
                    ellm_amd.MatMul3(x_dec, w[0], q_dec, w[1], kt, w[2], vt, rope, D, n_dec, hq, hkv, v1.strides, 0,
                                     seq_table=v1),
                    ellm_amd.Attention(q_dec, kt, vt, out_dec, n_dec, hq, hkv, D, v1.strides, sc, lse=lse_dec,
                                       max_position_interval=1, seq_table=v1)))
    checked = (0, layers // 2 - 1, layers - 1)
    kept = {}
    torch.cuda.synchronize()
    for layer, (qkv_pre, att_pre, qkv_dec, att_dec) in enumerate(ops):      # the benchmark's order
        qkv_pre.run(0, s_pf, 1)
        att_pre.run(0, s_pf, 1)
        qkv_dec.run_ragged(dpos, max_pos, n_dec)
        att_dec.run_ragged(dpos, max_pos, n_dec)
        if layer in checked:      # the activations are layer-shared scratch: keep this layer's
            kept[layer] = tuple(t.clone() for t in (q_pf, out_pf, lse_pf, q_dec, out_dec, lse_dec))
    torch.cuda.synchronize()

    rng = np.random.default_rng(241)
    xh_dec = _host(x_dec, dtype)
    xh_pf = _host(x_pf, dtype)
    picks = sorted({int(np.argmin(lengths)), int(np.argmax(lengths)), 5, 20})
    all_heads = np.array([[0, 0, h] for h in range(hq)], dtype=np.uint32)

    def ulps(got, want):
        got, want = orc.from_storage(got, dtype), orc.from_storage(want, dtype)
        return float((np.abs(got - want) / 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 0.125))) - 10)).max())

    for layer in checked:
        kt, vt = cache.layer_flat_tensors(layer, td)
        wh = [_host(x, dtype) for x in weights[layer]]
        g_q_pf, g_out_pf, g_lse_pf, g_q_dec, g_out_dec, g_lse_dec = kept[layer]
        # prefill side: the plane of sequence 0 and sampled (token, head) rows
        k0, v0h = _host(kt[:, :s_pf], dtype), _host(vt[:, :s_pf], dtype)          # [hkv, 16384, 128]
        ref = orc.Operator(_host(g_q_pf, dtype), k0, v0h, np.zeros((1,), np.float16), None, 1, hq, hkv, D,
                           [0, s_pf * D, D, 1], sc, dtype)
        toks = np.concatenate([[0, 63, s_pf - 1], rng.integers(0, s_pf, 9)])
        rows = np.stack([toks, np.zeros_like(toks), rng.integers(0, hq, toks.size)], 1).astype(np.uint32)
        _check_rows(ref, rows, 0, g_out_pf, g_lse_pf, dtype)
        # ... and a window of its projection
        t0 = int(rng.integers(0, s_pf - 16))
        oq = np.zeros((16, 1, hq, D), dtype=np.float16)
        ok = np.zeros((1, hkv, s_pf, D), dtype=np.float16)
        ov = np.zeros_like(ok)
        assert orc.matmul3(np.ascontiguousarray(xh_pf[t0:t0 + 16]), wh[0], wh[1], wh[2], oq, ok, ov, rope_h,
                           [hkv * s_pf * D, s_pf * D, D, 1], s_pf, t0, 16, dtype) == 0
        worst = max(ulps(_host(g_q_pf, dtype)[t0:t0 + 16], oq), ulps(k0[:, t0:t0 + 16], ok[0, :, t0:t0 + 16]),
                    ulps(v0h[:, t0:t0 + 16], ov[0, :, t0:t0 + 16]))
        assert worst <= 1.0, (layer, "prefill projection", worst)
        # single-token side: every head of four sequences, and their projection rows
        got_dec, got_lse = to_host(g_out_dec, dtype), g_lse_dec.cpu().numpy()
        qh_dec = _host(g_q_dec, dtype)
        for i in picks:
            o, cap_i = int(offs[1 + i]), caps[1 + i]
            ki, vi = _host(kt[:, o:o + cap_i], dtype), _host(vt[:, o:o + cap_i], dtype)
            ref = orc.Operator(np.ascontiguousarray(qh_dec[:, i:i + 1]), ki, vi, np.zeros((1,), np.float16), None, 1,
                               hq, hkv, D, [0, cap_i * D, D, 1], sc, dtype)
            want, want_lse, _ = ref.run_rows(int(pos[i]), all_heads, 8)
            res = compare(got_dec[0, i], orc.from_storage(want, dtype), dtype)
            assert res["ok"], (layer, i, int(lengths[i]), res)
            assert np.abs(got_lse[0, i] - want_lse).max() <= LSE_TOL, (layer, i)
            oq = np.zeros((1, 1, hq, D), dtype=np.float16)
            ok = np.zeros((1, hkv, cap_i, D), dtype=np.float16)
            ov = np.zeros_like(ok)
            assert orc.matmul3(np.ascontiguousarray(xh_dec[:, i:i + 1]), wh[0], wh[1], wh[2], oq, ok, ov, rope_h,
                               [hkv * cap_i * D, cap_i * D, D, 1], cap_i, int(pos[i]), 1, dtype) == 0
            worst = max(ulps(qh_dec[:, i:i + 1], oq), ulps(ki[:, pos[i]], ok[0, :, pos[i]]),
                        ulps(vi[:, pos[i]], ov[0, :, pos[i]]))
            assert worst <= 1.0, (layer, i, "single-token projection", worst)
        print(f"layer {layer}: prefill rows, 4 x 32 single-token rows and their projection rows match the oracle", flush=True)
    for group in ops:
        for op in group:
            op.close()
    cache.close()
