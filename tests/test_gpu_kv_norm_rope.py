"""Key rows normalised and rotated on the way into the cache (ellm_kv_append_norm_rope)
against the CPU oracle, through the C ABI.  The kernel keeps the oracle's operation
order in binary32 (sequential sum of squares, one rounding per operation), so rows are
compared bit for bit."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, compare, rand_storage, to_dev, to_host, torch_dtype

pytestmark = pytest.mark.gpu


def _rope_table(positions, dtype, theta=1.0e6):
    """(cos, sin) interleaved, angle = position * theta^(-2j / D): the usual rotary table."""
    j = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(positions, dtype=np.float64)[:, None] * theta ** (-2.0 * j / D)[None, :]
    t = np.empty((positions, D), dtype=np.float32)
    t[:, 0::2], t[:, 1::2] = np.cos(ang), np.sin(ang)
    return orc.to_storage(t, dtype)


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def _dev_bits(t):
    import torch

    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


CASES = [
    # (sequences in cache, batch, src pitch, kv heads, capacity, first position, tokens)
    (2, 2, 2, 2, 64, 0, 64),       # a whole chunk from position 0
    (3, 2, 5, 4, 200, 131, 37),    # pitch > batch, odd sizes, offset start
    (16, 16, 16, 4, 128, 100, 1),  # one token for 16 sequences
    (1, 1, 1, 1, 40, 39, 1),       # the last position of a plane
]


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
@pytest.mark.parametrize("case", CASES)
def test_rows_match_the_oracle_bit_for_bit(case, dtype):
    import torch

    import ellm_amd

    seqs, b, pitch, hkv, cap, p0, n_tok = case
    code = ellm_amd.DTYPE_F16 if dtype == orc.F16 else ellm_amd.DTYPE_BF16
    cache = ellm_amd.KVCache(2, seqs, hkv, cap, code)
    k_src = rand_storage((n_tok, pitch, hkv, D), 41, dtype, scale=3.0)
    v_src = rand_storage((n_tok, pitch, hkv, D), 42, dtype)
    k_src[0, 0, 0, :] = 0                      # a zero row must come out as zeros, not NaN
    rope = _rope_table(cap, dtype)
    layer = 1
    cache.append_norm_rope(layer, p0, to_dev(k_src, dtype), to_dev(v_src, dtype),
                           to_dev(rope, dtype), eps=1e-6, batch_size=b)
    torch.cuda.synchronize()
    kt, vt = cache.layer_tensors(layer, torch_dtype(dtype))
    want_k = np.zeros((seqs, hkv, cap, D), dtype=k_src.dtype)
    want_v = np.zeros_like(want_k)
    assert orc.kv_append_norm_rope(want_k, want_v, p0, k_src, v_src, rope, 1e-6, dtype,
                                   batch_size=b) == 0
    assert np.array_equal(_dev_bits(kt), _bits(want_k))
    assert np.array_equal(_dev_bits(vt), _bits(want_v))
    assert not np.isnan(to_host(kt, dtype)).any()
    k0, v0 = cache.layer_tensors(0, torch_dtype(dtype))
    assert not _dev_bits(k0).any() and not _dev_bits(v0).any()      # other layer untouched
    cache.close()


def test_per_sequence_positions():
    import torch

    import ellm_amd

    dtype = orc.F16
    seqs, hkv, cap = 5, 2, 300
    cache = ellm_amd.KVCache(1, seqs, hkv, cap, ellm_amd.DTYPE_F16)
    k_src = rand_storage((1, seqs, hkv, D), 43, dtype)
    v_src = rand_storage((1, seqs, hkv, D), 44, dtype)
    rope = _rope_table(cap, dtype)
    positions = np.array([0, 17, 299, 128, 5], dtype=np.int32)
    dpos = torch.from_numpy(positions).cuda()
    cache.append_norm_rope(0, 12345, to_dev(k_src, dtype), to_dev(v_src, dtype), to_dev(rope, dtype),
                           positions=dpos, max_position=299)
    torch.cuda.synchronize()
    kt, vt = cache.layer_tensors(0, torch_dtype(dtype))
    want_k = np.zeros((seqs, hkv, cap, D), dtype=np.float16)
    want_v = np.zeros_like(want_k)
    assert orc.kv_append_norm_rope(want_k, want_v, 0, k_src, v_src, rope, 1e-6, dtype,
                                   positions=positions) == 0
    assert np.array_equal(_dev_bits(kt), _bits(want_k))
    assert np.array_equal(_dev_bits(vt), _bits(want_v))
    cache.close()


def test_attention_over_rotated_keys_matches_the_oracle_pipeline():
    """Chunk, then token by token, through the fused write; attention over the cache then
    equals the oracle's attention over the oracle's rotated keys."""
    import torch

    import ellm_amd

    dtype = orc.F16
    bcap, b, hkv, hq, cap, total = 2, 2, 2, 8, 96, 70
    cache = ellm_amd.KVCache(1, bcap, hkv, cap, ellm_amd.DTYPE_F16)
    k_src = rand_storage((total, bcap, hkv, D), 45, dtype, scale=2.0)
    v_src = rand_storage((total, bcap, hkv, D), 46, dtype)
    rope = _rope_table(cap, dtype)
    dk, dv, dr = to_dev(k_src, dtype), to_dev(v_src, dtype), to_dev(rope, dtype)
    cache.append_norm_rope(0, 0, dk[:48], dv[:48], dr, batch_size=b)
    for t in range(48, total):
        cache.append_norm_rope(0, t, dk[t:t + 1], dv[t:t + 1], dr, batch_size=b)
    kt, vt = cache.layer_tensors(0, torch_dtype(dtype))
    _, _, strides = cache.layer(0)
    q = rand_storage((20, bcap, hq, D), 47, dtype)
    dq = to_dev(q, dtype)
    dout = torch.zeros_like(dq)
    op = ellm_amd.Attention(dq, kt, vt, dout, bcap, hq, hkv, D, strides, 0.3,
                            sequence_capacity=cap, max_position_interval=20)
    op.run(50, 20, b)
    torch.cuda.synchronize()
    want_k = np.zeros((bcap, hkv, cap, D), dtype=np.float16)
    want_v = np.zeros_like(want_k)
    assert orc.kv_append_norm_rope(want_k, want_v, 0, k_src, v_src, rope, 1e-6, dtype,
                                   batch_size=b) == 0
    want, _ = orc.attention(q, want_k, want_v, 0.3, dtype, position_index=50, batch=b)
    assert compare(to_host(dout, dtype)[:, :b], orc.from_storage(want, dtype)[:, :b], dtype)["ok"]
    op.close()
    cache.close()


def test_rejects_positions_outside_the_cache_or_the_table():
    import torch

    import ellm_amd

    dtype = orc.F16
    cache = ellm_amd.KVCache(1, 2, 1, 32, ellm_amd.DTYPE_F16)
    k = to_dev(rand_storage((4, 2, 1, D), 48, dtype), dtype)
    rope_full = to_dev(_rope_table(32, dtype), dtype)
    rope_short = to_dev(_rope_table(16, dtype), dtype)
    with pytest.raises(ellm_amd.EllmError):
        cache.append_norm_rope(0, 30, k, k, rope_full)                 # 30..33 of 32
    with pytest.raises(ellm_amd.EllmError):
        cache.append_norm_rope(0, 14, k, k, rope_short)                # table has 16 rows
    with pytest.raises(ellm_amd.EllmError):
        cache.append_norm_rope(1, 0, k, k, rope_full)                  # no such layer
    with pytest.raises(ellm_amd.EllmError):
        cache.append_norm_rope(0, 0, k, k, rope_full, eps=-1.0)
    pos = torch.zeros(2, dtype=torch.int32, device="cuda")
    with pytest.raises(ellm_amd.EllmError):
        cache.append_norm_rope(0, 0, k, k, rope_full, positions=pos, max_position=29)
    cache.append_norm_rope(0, 28, k, k, rope_full)                     # exactly fits
    torch.cuda.synchronize()
    cache.close()
