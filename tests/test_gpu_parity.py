"""HIP path against the CPU oracle on the same seeded inputs, through the C ABI."""
import ctypes

import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import (D, LSE_TOL, compare, gpu_attention, rand_storage, to_dev, to_host,
                      torch_dtype)

pytestmark = pytest.mark.gpu


def _check(name, q, k, v, scale, dtype, p0=0, batch=None, positions=None):
    want, want_lse = orc.attention(q, k, v, scale, dtype, position_index=p0, positions=positions,
                                   batch=batch)
    got, got_lse = gpu_attention(q, k, v, scale, dtype, position_index=p0, batch=batch,
                                 positions=positions)
    b = q.shape[1] if batch is None else batch
    res = compare(got[:, :b], orc.from_storage(want, dtype)[:, :b], dtype)
    lse_err = float(np.abs(got_lse[:, :b] - want_lse[:, :b]).max())
    print(f"{name}: {res} lse_err={lse_err:.2e}", flush=True)
    assert res["ok"], (name, res)
    assert lse_err <= LSE_TOL, (name, lse_err)
    if b < q.shape[1]:   # rows of sequences beyond the live batch are never written
        assert np.isnan(got[:, b:]).all()
    return got, got_lse


# (name, batch capacity, batch, q heads, kv heads, capacity, position_index, interval)
PREFILL = [
    ("one_token_block", 1, 1, 8, 1, 64, 0, 32),
    ("ragged_tail_g8", 1, 1, 8, 1, 256, 0, 200),
    ("mha_two_seq", 2, 2, 4, 4, 128, 0, 96),
    ("chunk_on_cache", 1, 1, 8, 2, 256, 100, 70),
    ("batch_below_capacity_g4", 3, 2, 8, 2, 512, 0, 300),
    ("g2", 1, 1, 4, 2, 320, 5, 257),
    ("g3_odd_group", 1, 1, 6, 2, 200, 0, 150),
    ("g16", 1, 1, 16, 1, 160, 3, 100),
    ("interval_2", 2, 2, 8, 2, 64, 61, 2),
    ("tile_edge_63_64_65", 1, 1, 8, 1, 256, 63, 66),
    ("qwen3_heads_2k", 1, 1, 32, 4, 2048, 0, 2048),
    # few row blocks on a long cache: the key range is split over workgroups and merged
    ("split_chunk_on_long_cache", 1, 1, 8, 1, 2304, 2000, 70),
    ("split_batch_below_capacity_g4", 3, 2, 8, 2, 1600, 1500, 40),
    ("split_interval_2", 2, 2, 8, 2, 4200, 4100, 2),
    ("split_from_zero_later_splits_empty_for_early_rows", 1, 1, 8, 1, 1152, 0, 1100),
    ("split_qwen3_chunk_64_on_8k", 1, 1, 32, 4, 8320, 8192, 64),
    ("split_three_tokens_on_20k_forty_splits", 1, 1, 8, 1, 20480, 20000, 3),
    # at most 128 query rows per K/V plane on a cache of 512 keys or more: the streaming chunk
    # kernel (one workgroup holds all (token, head) rows of a GQA group, keys split over workgroups);
    # the short last chunk of a prompt in the reference's serving loop, 24 sequences
    ("stream_2tok_b24_on_tile_edge", 24, 24, 32, 4, 1200, 1024, 2),
    ("stream_3tok_b24_off_edge", 24, 24, 32, 4, 1200, 1000, 3),
    ("stream_16tok_b24_across_chunk_edge", 24, 24, 32, 4, 1200, 1087, 16),
    ("stream_16tok_b24_on_chunk_edge", 24, 24, 32, 4, 1216, 1088, 16),
    # 129-256 and 257-384 rows a plane: the same kernel with eight and twelve waves
    ("stream_17tok_b24_eight_waves", 24, 24, 32, 4, 1200, 1001, 17),
    ("stream_32tok_b24_eight_waves_full", 24, 24, 32, 4, 1200, 1056, 32),
    ("stream_33tok_b24_twelve_waves", 24, 24, 32, 4, 1200, 1001, 33),
    ("stream_48tok_b6_twelve_waves_full", 6, 6, 32, 4, 1200, 1087, 48),
    ("stream_g16_20tok_twelve_waves_below_capacity", 3, 2, 16, 1, 900, 700, 20),
    ("stream_g3_50tok_eight_waves_odd_group", 2, 2, 6, 2, 800, 600, 50),
    ("pingpong_49tok_b24", 24, 24, 32, 4, 1200, 1001, 49),           # 392 rows a plane: the tile kernel
    # up to the reference's full chunk (sequence_chunk_size = 64, src/serving/start copy.rs:30) x 24 sequences
    ("chunk_56tok_b24_off_tile_edge", 24, 24, 32, 4, 1200, 1001, 56),
    ("chunk_63tok_b24_across_tile_edge", 24, 24, 32, 4, 1200, 1087, 63),
    ("chunk_64tok_b24_on_tile_edge", 24, 24, 32, 4, 1216, 1088, 64),
    ("stream_batch_below_capacity_9tok", 5, 3, 8, 2, 900, 700, 9),    # 36 rows: a part-filled second wave
    ("stream_g16_8tok_full_workgroup", 1, 1, 16, 1, 3000, 2900, 8),   # 128 rows exactly
    ("stream_first_split_only_for_early_rows", 2, 2, 8, 2, 700, 500, 5),
    ("stream_unsplit_many_sequences", 160, 160, 32, 4, 600, 560, 16),  # no room for partial rows: one split
]


@pytest.mark.parametrize("case", PREFILL, ids=[c[0] for c in PREFILL])
@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16], ids=["f16", "bf16"])
def test_prefill_matches_oracle(case, dtype):
    name, bcap, b, hq, hkv, cap, p0, s = case
    print("case", name, flush=True)
    q = rand_storage((s, bcap, hq, D), 1, dtype)
    k = rand_storage((bcap, hkv, cap, D), 2, dtype)
    v = rand_storage((bcap, hkv, cap, D), 3, dtype)
    _check(name, q, k, v, 1.0 / np.sqrt(D), dtype, p0=p0, batch=b)


DECODE = [
    ("first_token", 1, 1, 8, 1, 64, 0),
    ("short", 1, 1, 8, 1, 64, 4),
    ("two_splits", 2, 2, 8, 2, 512, 299),
    ("mha", 2, 2, 4, 4, 1024, 700),
    ("batch_below_capacity", 5, 3, 8, 2, 640, 600),
    ("g32_two_head_groups", 1, 1, 32, 1, 4096, 4000),
    ("g3_odd_group", 2, 2, 6, 2, 300, 257),
    ("qwen3_b16_1k", 16, 16, 32, 4, 1024, 1023),
    ("long_b1_two_merge_levels", 1, 1, 8, 1, 65536, 65535),
]


@pytest.mark.parametrize("case", DECODE, ids=[c[0] for c in DECODE])
@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16], ids=["f16", "bf16"])
def test_decode_matches_oracle(case, dtype):
    name, bcap, b, hq, hkv, cap, pos = case
    print("case", name, flush=True)
    q = rand_storage((1, bcap, hq, D), 4, dtype)
    k = rand_storage((bcap, hkv, cap, D), 5, dtype)
    v = rand_storage((bcap, hkv, cap, D), 6, dtype)
    _check(name, q, k, v, 1.0 / np.sqrt(D), dtype, p0=pos, batch=b)


def test_decode_ragged_positions():
    dtype = orc.F16
    pos = np.array([5, 2047, 300, 1000, 0, 64, 63, 1535], dtype=np.uint32)
    q = rand_storage((1, 8, 16, D), 7, dtype)
    k = rand_storage((8, 2, 2048, D), 8, dtype)
    v = rand_storage((8, 2, 2048, D), 9, dtype)
    _check("ragged", q, k, v, 1.0 / np.sqrt(D), dtype, positions=pos)


def test_decode_repeated_launches_reuse_the_counters():
    """The arrival counters of the split merge must be back at zero after every launch."""
    import torch

    import ellm_amd

    dtype = orc.F16
    b, hq, hkv, cap = 4, 16, 2, 4096
    q = rand_storage((1, b, hq, D), 10, dtype)
    k = rand_storage((b, hkv, cap, D), 11, dtype)
    v = rand_storage((b, hkv, cap, D), 12, dtype)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    dout = torch.zeros_like(dq)
    op = ellm_amd.Attention(dq, dk, dv, dout, b, hq, hkv, D, [hkv * cap * D, cap * D, D, 1],
                            1.0 / np.sqrt(D), sequence_capacity=cap, max_position_interval=1)
    first = None
    for n, pos in enumerate((4095, 1000, 4095, 77, 4095, 4095)):
        if n == 4:
            op.reset()    # the counters are at zero already: the reset must be harmless
        op.run(pos, 1, b)
        torch.cuda.synchronize()
        if pos == 4095:
            got = dout.clone()
            if first is None:
                first = got
                want, _ = orc.attention(q, k, v, 1.0 / np.sqrt(D), dtype, position_index=pos)
                assert compare(to_host(got, dtype), orc.from_storage(want, dtype), dtype)["ok"]
            else:
                assert torch.equal(got, first)   # same launch, same bits
    op.close()


def test_reference_kv_layout_strides():
    """K/V handed over as the reference's permuted view of [position][sequence][kv_head][D]
    (src/qwen3_moe/attention.rs:149-166): kv_strides = [Hkv*D, D, B*Hkv*D, 1]."""
    dtype = orc.F16
    s, b, hq, hkv, cap, p0 = 40, 2, 8, 2, 128, 50
    q = rand_storage((s, b, hq, D), 13, dtype)
    kphys = rand_storage((cap, b, hkv, D), 14, dtype)
    vphys = rand_storage((cap, b, hkv, D), 15, dtype)
    strides = [hkv * D, D, b * hkv * D, 1]
    k = np.ascontiguousarray(kphys.transpose(1, 2, 0, 3))
    v = np.ascontiguousarray(vphys.transpose(1, 2, 0, 3))
    want, want_lse = orc.attention(q, k, v, 0.09, dtype, position_index=p0)
    got, lse = gpu_attention(q, kphys, vphys, 0.09, dtype, position_index=p0, kv_strides=strides,
                             cap=cap, kv_heads=hkv)
    assert compare(got, orc.from_storage(want, dtype), dtype)["ok"]
    assert np.abs(lse - want_lse).max() <= LSE_TOL
    # and a single-token step on the same layout
    q1 = q[:1]
    want1, _ = orc.attention(q1, k, v, 0.09, dtype, position_index=cap - 1)
    got1, _ = gpu_attention(q1, kphys, vphys, 0.09, dtype, position_index=cap - 1,
                            kv_strides=strides, cap=cap, kv_heads=hkv)
    assert compare(got1, orc.from_storage(want1, dtype), dtype)["ok"]


@pytest.mark.parametrize("scale", [-0.07, 0.0, 1.0, 1e-3])
def test_unusual_scales(scale):
    dtype = orc.F16
    q = rand_storage((50, 1, 8, D), 16, dtype)
    k = rand_storage((1, 2, 128, D), 17, dtype, scale=0.3)
    v = rand_storage((1, 2, 128, D), 18, dtype)
    _check(f"scale {scale} prefill", q, k, v, scale, dtype, p0=30)
    _check(f"scale {scale} decode", q[:1], k, v, scale, dtype, p0=127)
    # the same through the split chunk path (few rows on a long cache) and its merge
    k2 = rand_storage((1, 2, 1600, D), 27, dtype, scale=0.3)
    v2 = rand_storage((1, 2, 1600, D), 28, dtype)
    _check(f"scale {scale} split chunk", q, k2, v2, scale, dtype, p0=1500)


def test_garbage_beyond_the_position_does_not_leak():
    """Cache rows after the last visible position hold NaN / Inf / huge values, and so
    does the output buffer before the call; none of it may reach the result."""
    dtype = orc.F16
    s, p0, cap = 70, 20, 256
    q = rand_storage((s, 1, 8, D), 19, dtype)
    k = rand_storage((1, 2, cap, D), 20, dtype)
    v = rand_storage((1, 2, cap, D), 21, dtype)
    clean, clean_lse = gpu_attention(q, k, v, 0.09, dtype, position_index=p0)
    k2, v2 = k.copy(), v.copy()
    k2[:, :, p0 + s:], v2[:, :, p0 + s:] = np.nan, np.inf
    k2[:, :, p0 + s + 3], v2[:, :, p0 + s + 3] = 60000.0, -60000.0
    dirty, dirty_lse = gpu_attention(q, k2, v2, 0.09, dtype, position_index=p0, out_fill=float("inf"))
    assert np.array_equal(clean, dirty) and np.array_equal(clean_lse, dirty_lse)
    c1, _ = gpu_attention(q[:1], k, v, 0.09, dtype, position_index=p0 + s - 1)
    d1, _ = gpu_attention(q[:1], k2, v2, 0.09, dtype, position_index=p0 + s - 1)
    assert np.array_equal(c1, d1)


def test_garbage_beyond_the_position_does_not_leak_into_split_chunks():
    """The split chunk path: workgroups of later key ranges see rows whose every key is masked,
    and the cache beyond the last position holds NaN / Inf."""
    dtype = orc.F16
    s, p0, cap = 40, 1400, 2048
    q = rand_storage((s, 1, 8, D), 22, dtype)
    k = rand_storage((1, 2, cap, D), 23, dtype)
    v = rand_storage((1, 2, cap, D), 24, dtype)
    clean, clean_lse = gpu_attention(q, k, v, 0.09, dtype, position_index=p0)
    k2, v2 = k.copy(), v.copy()
    bad = np.array([0x7e00, 0x7c00, 0xfc00, 0x7bff], dtype=np.uint16)      # NaN, +Inf, -Inf, 65504
    k2[:, :, p0 + s:] = bad[np.arange(k2[:, :, p0 + s:].size) % 4].reshape(k2[:, :, p0 + s:].shape)
    v2[:, :, p0 + s:] = bad[(np.arange(v2[:, :, p0 + s:].size) + 1) % 4].reshape(v2[:, :, p0 + s:].shape)
    dirty, dirty_lse = gpu_attention(q, k2, v2, 0.09, dtype, position_index=p0)
    assert np.array_equal(clean, dirty) and np.array_equal(clean_lse, dirty_lse)
    want, want_lse = orc.attention(q, k, v, 0.09, dtype, position_index=p0)
    assert compare(clean, orc.from_storage(want, dtype), dtype)["ok"]


def test_causality_rows_ignore_later_keys():
    dtype = orc.F16
    s, cap = 130, 192
    q = rand_storage((s, 1, 8, D), 22, dtype)
    k = rand_storage((1, 1, cap, D), 23, dtype)
    v = rand_storage((1, 1, cap, D), 24, dtype)
    base, _ = gpu_attention(q, k, v, 0.09, dtype, position_index=0)
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 100:] = rand_storage((1, 1, cap - 100, D), 25, dtype)
    v2[:, :, 100:] = rand_storage((1, 1, cap - 100, D), 26, dtype)
    pert, _ = gpu_attention(q, k2, v2, 0.09, dtype, position_index=0)
    assert np.array_equal(base[:100], pert[:100])        # rows 0..99 never see keys >= 100
    assert not np.array_equal(base[100:], pert[100:])


@pytest.mark.parametrize("shape", [("tile", 130, 60, 256, 8, 1), ("stream", 24, 900, 1024, 8, 2)],
                         ids=lambda sh: sh[0])
def test_value_rows_rule_at_the_boundary_the_header_states(shape):
    """ellm_attn_run's rule for K/V contents, pinned where it bites, in the tile kernel and in the
    streaming chunk kernel: (1) rows of the call's own later tokens are read by earlier query rows
    with a probability of exactly 0, so while they are FINITE (whatever their values) the earlier
    rows' bits do not depend on them; (2) rows strictly beyond the call's last position are never
    read: NaN / Inf there change nothing.  (The reference reads neither: flash_attention.rs:57-58.)"""
    _, s, p0, cap, hq, hkv = shape
    dtype = orc.F16
    q = rand_storage((s, 1, hq, D), 91, dtype)
    k = rand_storage((1, hkv, cap, D), 92, dtype)
    v = rand_storage((1, hkv, cap, D), 93, dtype)
    base, base_lse = gpu_attention(q, k, v, 0.09, dtype, position_index=p0)
    cut = s // 2                                         # tokens cut.. of the chunk are "later" for rows < cut
    k2, v2 = k.copy(), v.copy()
    k2.view(np.float16)[:, :, p0 + cut:p0 + s] = 60000.0    # finite, huge
    v2.view(np.float16)[:, :, p0 + cut:p0 + s] = -65504.0
    k2.view(np.uint16)[:, :, p0 + s:] = 0x7e00              # NaN beyond the call's last position
    v2.view(np.uint16)[:, :, p0 + s:] = 0x7c00              # +Inf
    pert, pert_lse = gpu_attention(q, k2, v2, 0.09, dtype, position_index=p0)
    assert np.array_equal(base[:cut], pert[:cut]) and np.array_equal(base_lse[:cut], pert_lse[:cut])
    assert np.isfinite(pert[:cut]).all()
    want, _ = orc.attention(q, k, v, 0.09, dtype, position_index=p0)
    assert compare(base, orc.from_storage(want, dtype), dtype)["ok"]


def test_chunked_prefill_and_decode_agree_with_one_pass():
    """The position loop of the serving layer (src/serving/'start copy.rs':86-111): full
    chunks, a partial chunk, then single-token steps give the rows of one pass."""
    dtype = orc.F16
    s, cap = 200, 256
    q = rand_storage((s, 1, 8, D), 27, dtype)
    k = rand_storage((1, 2, cap, D), 28, dtype)
    v = rand_storage((1, 2, cap, D), 29, dtype)
    whole, whole_lse = gpu_attention(q, k, v, 0.09, dtype, position_index=0)
    rows, lses = [], []
    for t0, n in ((0, 64), (64, 64), (128, 37)):
        o, l = gpu_attention(q[t0:t0 + n], k, v, 0.09, dtype, position_index=t0)
        rows.append(o)
        lses.append(l)
    for t in range(165, s):
        o, l = gpu_attention(q[t:t + 1], k, v, 0.09, dtype, position_index=t)
        rows.append(o)
        lses.append(l)
    got, got_lse = np.concatenate(rows), np.concatenate(lses)
    # different tilings round differently: same tolerance as against the oracle
    assert compare(got, whole, dtype)["ok"]
    assert np.abs(got_lse - whole_lse).max() <= LSE_TOL


def test_gqa_group_with_identical_queries_gives_identical_rows():
    dtype = orc.F16
    q = rand_storage((40, 1, 8, D), 30, dtype)
    q[:, :, 1:4] = q[:, :, 0:1]
    k = rand_storage((1, 2, 64, D), 31, dtype)
    v = rand_storage((1, 2, 64, D), 32, dtype)
    out, _ = gpu_attention(q, k, v, 0.09, dtype, position_index=10)
    for h in range(1, 4):
        assert np.array_equal(out[:, :, h], out[:, :, 0])
    assert not np.array_equal(out[:, :, 4], out[:, :, 0])


def test_run_rejects_out_of_range_arguments():
    import torch

    import ellm_amd

    b, hq, hkv, cap = 2, 8, 2, 64
    t = torch.zeros((4, b, hq, D), dtype=torch.float16, device="cuda")
    kv = torch.zeros((b, hkv, cap, D), dtype=torch.float16, device="cuda")
    op = ellm_amd.Attention(t, kv, kv, torch.zeros_like(t), b, hq, hkv, D,
                            [hkv * cap * D, cap * D, D, 1], 0.1, sequence_capacity=cap,
                            max_position_interval=4)
    for args in ((cap, 1, b), (cap - 2, 4, b), (0, 5, b), (0, 1, b + 1)):
        with pytest.raises(ellm_amd.EllmError) as e:
            op.run(*args)
        assert e.value.status == 3
    op.run(0, 0, b)      # empty work is fine
    op.run(0, 1, 0)
    with pytest.raises(ellm_amd.EllmError):
        op.run_ragged(torch.zeros(b, dtype=torch.int32, device="cuda"), cap, b)
    torch.cuda.synchronize()
    op.close()


def test_kv_cache_append_in_place():
    """[token][sequence][kv_head][D] rows land at their token coordinates of
    [layer][sequence][kv_head][position][D]; attention over the cache then equals the
    oracle over the same rows."""
    import torch

    import ellm_amd

    dtype = orc.F16
    layers, bcap, b, hkv, hq, cap = 2, 3, 2, 2, 8, 96
    cache = ellm_amd.KVCache(layers, bcap, hkv, cap, ellm_amd.DTYPE_F16)
    ksrc = rand_storage((80, bcap, hkv, D), 33, dtype)
    vsrc = rand_storage((80, bcap, hkv, D), 34, dtype)
    dks, dvs = to_dev(ksrc, dtype), to_dev(vsrc, dtype)
    layer = 1
    cache.append(layer, 0, dks[:50], dvs[:50], batch_size=b)          # a 50-token chunk
    for t in range(50, 80):                                            # then token by token
        cache.append(layer, t, dks[t:t + 1], dvs[t:t + 1], batch_size=b)
    kt, vt = cache.layer_tensors(layer, torch_dtype(dtype))
    torch.cuda.synchronize()
    kh = to_host(kt, dtype)
    assert np.array_equal(kh[:b, :, :80], orc.from_storage(ksrc, dtype)[:, :b].transpose(1, 2, 0, 3))
    assert not kh[b:].any() and not kh[:, :, 80:].any()                # zero-filled elsewhere
    k0, _ = cache.layer_tensors(0, torch_dtype(dtype))
    assert not to_host(k0, dtype).any()                                # other layer untouched
    kptr, vptr, strides = cache.layer(layer)
    assert strides == [hkv * cap * D, cap * D, D, 1]
    q = rand_storage((30, bcap, hq, D), 35, dtype)
    dq = to_dev(q, dtype)
    dout = torch.zeros_like(dq)
    op = ellm_amd.Attention(dq, kt, vt, dout, bcap, hq, hkv, D, strides, 0.09,
                            sequence_capacity=cap, max_position_interval=30)
    op.run(50, 30, b)
    torch.cuda.synchronize()
    kfull = np.zeros((bcap, hkv, cap, D), dtype=np.float16)
    vfull = np.zeros_like(kfull)
    kfull[:, :, :80] = ksrc.transpose(1, 2, 0, 3)
    vfull[:, :, :80] = vsrc.transpose(1, 2, 0, 3)
    want, _ = orc.attention(q, kfull, vfull, 0.09, dtype, position_index=50, batch=b)
    assert compare(to_host(dout, dtype)[:, :b], orc.from_storage(want, dtype)[:, :b], dtype)["ok"]
    with pytest.raises(ellm_amd.EllmError):
        cache.append(layer, cap - 10, dks[:50], dvs[:50], batch_size=b)
    with pytest.raises(ellm_amd.EllmError):
        cache.append(layers, 0, dks[:1], dvs[:1], batch_size=b)
    op.close()
    cache.close()


def test_host_mirror_thread_convention():
    """All worker threads call run(); only thread 0 launches (src/serving/start.rs:69-73)."""
    import torch

    import ellm_amd

    dtype = orc.F16
    q = rand_storage((1, 1, 8, D), 36, dtype)
    k = rand_storage((1, 1, 64, D), 37, dtype)
    v = rand_storage((1, 1, 64, D), 38, dtype)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    dout = torch.zeros_like(dq)
    op = ellm_amd.Attention.new(dq, dk, dv, dout, 1, 8, 1, D, [64 * D, 64 * D, D, 1], 0.09)
    for tid in range(1, 8):
        op.run(63, 1, 1, cpu_num=8, thread_id=tid)
    torch.cuda.synchronize()
    assert not dout.any()
    op.run(63, 1, 1, cpu_num=8, thread_id=0)
    torch.cuda.synchronize()
    want, _ = orc.attention(q, k, v, 0.09, dtype, position_index=63)
    assert compare(to_host(dout, dtype), orc.from_storage(want, dtype), dtype)["ok"]
    op.close()


@pytest.mark.gpu
def test_host_mirror_refuses_short_or_mistyped_buffers():
    """Extents are checked against what the operator will address (the C ABI sees addresses
    only): a cache shorter than capacity x stride, an output of another type, 64-bit positions."""
    import torch

    import ellm_amd

    hq, hkv, cap = 8, 2, 64
    q = torch.zeros((1, 2, hq, 128), dtype=torch.float16, device="cuda")
    out = torch.zeros_like(q)
    k = torch.zeros((2, hkv, cap, 128), dtype=torch.float16, device="cuda")
    strides = [hkv * cap * 128, cap * 128, 128, 1]
    with pytest.raises(ValueError, match="addresses"):
        ellm_amd.Attention(q, k[:, :, : cap // 2].contiguous(), k, out, 2, hq, hkv, 128, strides, 0.1,
                           sequence_capacity=cap)
    with pytest.raises(TypeError, match="expected"):
        ellm_amd.Attention(q, k, k, out.to(torch.bfloat16), 2, hq, hkv, 128, strides, 0.1)
    with pytest.raises(ValueError, match="addresses"):
        ellm_amd.Attention(q, k, k, out, 3, hq, hkv, 128, strides, 0.1)   # batch capacity 3, buffers for 2
    op = ellm_amd.Attention(q, k, k, out, 2, hq, hkv, 128, strides, 0.1)
    with pytest.raises(TypeError, match="32-bit"):
        op.run_ragged(torch.zeros(2, dtype=torch.int64, device="cuda"), 3, 2)
    with pytest.raises(ValueError, match="addresses"):
        op.run_ragged(torch.zeros(1, dtype=torch.int32, device="cuda"), 3, 2)
    op.close()
