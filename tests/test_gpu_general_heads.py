"""Attention for head sizes other than 128 and for binary32 storage (the library's plain
kernel, attn_general.hip) against the oracle, through the C ABI.  The reference's generic leaf
takes any `length` and element type (src/kernel/generic/flash_attention.rs:60-89) and its
operator test runs in f32 on all-ones tensors (src/compiler/mul/attention.rs:262-330); the
first test below is that test.  Both sides work in binary32 throughout, so 16-bit results may
differ by the one rounding to storage and binary32 results by the order of the sums."""
import ctypes

import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import LSE_TOL, compare_ulps

pytestmark = pytest.mark.gpu


def _torch_dtype(dtype):
    import torch

    return {orc.F16: torch.float16, orc.BF16: torch.bfloat16, orc.F32: torch.float32}[dtype]


def _to_dev(a, dtype):
    import torch

    if dtype == orc.F32:
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(_torch_dtype(dtype))


def _to_host(t, dtype):
    import torch

    if dtype == orc.F32:
        return t.cpu().numpy()
    return orc.from_storage(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16), dtype)


def _rand(shape, seed, dtype):
    rng = np.random.default_rng(seed)
    return orc.to_storage(rng.standard_normal(shape, dtype=np.float32), dtype)


def _run(q, k, v, scale, dtype, p0=0, batch=None, positions=None, kv_strides=None, cap=None, kv_heads=None):
    import torch

    import ellm_amd

    S, bcap, hq, hs = q.shape
    if kv_strides is None:
        hkv, cap = k.shape[1], k.shape[2]
        kv_strides = [hkv * cap * hs, cap * hs, hs, 1]
    else:
        hkv = kv_heads
    dq, dk, dv = (_to_dev(a, dtype) for a in (q, k, v))
    dout = torch.full_like(dq, float("nan"))
    dlse = torch.full((S, bcap, hq), float("nan"), dtype=torch.float32, device="cuda")
    op = ellm_amd.Attention(dq, dk, dv, dout, bcap, hq, hkv, hs, kv_strides, scale, lse=dlse,
                            sequence_capacity=cap, max_position_interval=S)
    b = bcap if batch is None else batch
    try:
        assert op.ragged_path(cap - 1, b) == 0      # never the kernels built for 128-wide 16-bit heads
        if positions is None:
            op.run(p0, S, b)
        else:
            dpos = torch.from_numpy(np.asarray(positions, dtype=np.uint32).view(np.int32)).cuda()
            op.run_ragged(dpos, int(np.max(positions)), b)
        torch.cuda.synchronize()
        return _to_host(dout, dtype), dlse.cpu().numpy()
    finally:
        op.close()


def _check(name, got, lse, want, want_lse, dtype, batch):
    g, w = got[:, :batch], orc.from_storage(want, dtype)[:, :batch]
    assert not np.isnan(g).any(), name
    if dtype == orc.F32:
        err = np.abs(g - w)
        bound = 2e-5 + 1e-4 * np.abs(w)          # binary32 sums taken in a different order
        assert (err <= bound).all(), (name, float(err.max()))
    else:
        r = compare_ulps(g, w, dtype)
        assert r["ok"], (name, r)
    assert np.abs(lse[:, :batch] - want_lse[:, :batch]).max() <= LSE_TOL, name
    if batch < got.shape[1]:   # rows of sequences beyond the live batch are never written
        assert np.isnan(got[:, batch:]).all() and np.isnan(lse[:, batch:]).all(), name


def test_the_reference_operator_test_in_f32():
    """test_attention_f32 of src/compiler/mul/attention.rs:262-330: all-ones q, k, v in f32, chunk and
    cache of 256 positions, 16 sequences, 8 = 8 heads of 128, K/V as the permuted view of
    [position][sequence][kv_head][128]; every output element is 1."""
    s, b, h, hs = 256, 16, 8, 128
    q = np.ones((s, b, h, hs), dtype=np.float32)
    kv = np.ones((s, b, h, hs), dtype=np.float32)
    strides = [h * hs, hs, b * h * hs, 1]
    got, lse = _run(q, kv, kv, 1.0, orc.F32, p0=0, kv_strides=strides, cap=s, kv_heads=h)
    assert np.abs(got - 1.0).max() <= 1e-6
    # log-sum-exp of p + 1 equal scores of 128 each
    want_lse = 128.0 + np.log(np.arange(1, s + 1, dtype=np.float64))
    assert np.abs(lse - want_lse[:, None, None]).max() <= LSE_TOL


# (name, dtype, batch capacity, batch, q heads, kv heads, head size, capacity, position_index, interval)
CHUNKS = [
    ("f32_h128_chunk_on_cache", orc.F32, 2, 2, 8, 2, 128, 128, 50, 40),
    ("f16_h64_from_zero", orc.F16, 2, 2, 8, 2, 64, 200, 0, 150),
    ("bf16_h96_g3", orc.BF16, 1, 1, 6, 2, 96, 160, 3, 100),
    ("f16_h256", orc.F16, 1, 1, 4, 4, 256, 96, 10, 70),
    ("f16_h80_batch_below_capacity", orc.F16, 3, 2, 8, 2, 80, 128, 20, 33),
    ("f32_h19_odd", orc.F32, 2, 2, 4, 1, 19, 70, 0, 70),
    ("bf16_h8_interval_2", orc.BF16, 2, 2, 8, 8, 8, 64, 61, 2),
]


@pytest.mark.parametrize("case", CHUNKS, ids=[c[0] for c in CHUNKS])
def test_chunks_match_the_oracle(case):
    name, dtype, bcap, b, hq, hkv, hs, cap, p0, s = case
    print("case", name, flush=True)
    q, k, v = _rand((s, bcap, hq, hs), 1, dtype), _rand((bcap, hkv, cap, hs), 2, dtype), _rand((bcap, hkv, cap, hs), 3, dtype)
    scale = 1.0 / np.sqrt(hs)
    want, want_lse = orc.attention(q, k, v, scale, dtype, position_index=p0, batch=b)
    got, lse = _run(q, k, v, scale, dtype, p0=p0, batch=b)
    _check(name, got, lse, want, want_lse, dtype, b)


# (name, dtype, batch capacity, batch, q heads, kv heads, head size, capacity, position or per-sequence positions)
STEPS = [
    ("f16_h64_first_token", orc.F16, 1, 1, 8, 1, 64, 64, 0),
    ("f32_h128_long", orc.F32, 2, 2, 8, 2, 128, 3000, 2999),
    ("bf16_h192_g16", orc.BF16, 1, 1, 16, 1, 192, 700, 650),
    ("f16_h64_ragged_positions", orc.F16, 5, 4, 8, 2, 64, 640, [600, 0, 63, 301]),
    ("f32_h34_ragged_positions", orc.F32, 3, 3, 4, 2, 34, 200, [199, 5, 100]),
]


@pytest.mark.parametrize("case", STEPS, ids=[c[0] for c in STEPS])
def test_single_token_steps_match_the_oracle(case):
    name, dtype, bcap, b, hq, hkv, hs, cap, position = case
    print("case", name, flush=True)
    q, k, v = _rand((1, bcap, hq, hs), 4, dtype), _rand((bcap, hkv, cap, hs), 5, dtype), _rand((bcap, hkv, cap, hs), 6, dtype)
    scale = 1.0 / np.sqrt(hs)
    if np.isscalar(position):
        want, want_lse = orc.attention(q, k, v, scale, dtype, position_index=position, batch=b)
        got, lse = _run(q, k, v, scale, dtype, p0=position, batch=b)
    else:
        pos = np.zeros(bcap, dtype=np.uint32)
        pos[:b] = position
        want, want_lse = orc.attention(q, k, v, scale, dtype, positions=pos, batch=b)
        got, lse = _run(q, k, v, scale, dtype, batch=b, positions=position)
    _check(name, got, lse, want, want_lse, dtype, b)


def test_rows_beyond_the_position_are_never_read():
    """Garbage (NaN) in every K/V row past the call's last position, and for the chunk's earlier
    tokens in the rows of its later ones, changes nothing: this kernel reads keys 0..=p only."""
    dtype, s, b, hq, hkv, hs, cap, p0 = orc.F32, 5, 2, 4, 2, 64, 64, 20
    q, k, v = _rand((s, b, hq, hs), 7, dtype), _rand((b, hkv, cap, hs), 8, dtype), _rand((b, hkv, cap, hs), 9, dtype)
    scale = 0.11
    want, want_lse = orc.attention(q, k, v, scale, dtype, position_index=p0)
    k2, v2 = k.copy(), v.copy()
    k2[:, :, p0 + s:] = np.nan
    v2[:, :, p0 + s:] = np.nan
    got, lse = _run(q, k2, v2, scale, dtype, p0=p0)
    _check("garbage_beyond", got, lse, want, want_lse, dtype, b)
    # NaN from the first token's position + 1 on: the chunk's first token still comes out right
    # (unlike the MFMA kernels, whose rule is that rows up to the call's last position are finite)
    k3, v3 = k.copy(), v.copy()
    k3[:, :, p0 + 1:] = np.nan
    v3[:, :, p0 + 1:] = np.nan
    got3, lse3 = _run(q, k3, v3, scale, dtype, p0=p0)
    _check("garbage_after_own_position", got3[:1], lse3[:1], want[:1], want_lse[:1], dtype, b)
    assert np.isnan(got3[1:]).all()


def test_entry_points_for_128_wide_16_bit_heads_refuse_other_shapes():
    import torch

    import ellm_amd
    from ellm_amd import _lib

    lib = ellm_amd.load_library()
    b, hq, hkv, hs, cap = 2, 4, 2, 64, 128
    q = torch.zeros((1, b, hq, hs), dtype=torch.float16, device="cuda")
    k = torch.zeros((b, hkv, cap, hs), dtype=torch.float16, device="cuda")
    out = torch.zeros_like(q)
    op = ellm_amd.Attention(q, k, k, out, b, hq, hkv, hs, [hkv * cap * hs, cap * hs, hs, 1], 0.1,
                            sequence_capacity=cap, max_position_interval=1)
    try:
        rc = lib.ellm_attn_run_noalloc(ctypes.byref(op.desc), None, 5, b, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 2 and b"128-wide" in lib.ellm_last_error_string()
    finally:
        op.close()
    with pytest.raises(ellm_amd.EllmError) as e:     # the cache and the projections stay 16-bit, 128 wide
        ellm_amd.KVCache(1, 1, 1, 16, _lib.DTYPE_F32)
    assert e.value.status == 1
    with pytest.raises(ellm_amd.EllmError) as e:
        ellm_amd.KVCache(1, 1, 1, 16, _lib.DTYPE_F16, head_size=64)
    assert e.value.status == 2
    torch.cuda.synchronize()


def test_random_shapes_against_the_oracle():
    """Seeded sweep over head sizes 1..256, the three storage types, group sizes, batches below capacity,
    chunks and single-token steps with shared and per-sequence positions."""
    rng = np.random.default_rng(2024)
    for n in range(18):
        dtype = (orc.F16, orc.BF16, orc.F32)[n % 3]
        hs = int(rng.integers(1, 257))
        hkv = int(rng.integers(1, 4))
        hq = hkv * int(rng.integers(1, 5))
        bcap = int(rng.integers(1, 4))
        b = int(rng.integers(1, bcap + 1))
        cap = int(rng.integers(8, 300))
        q_seed = 100 + n
        scale = float(rng.uniform(0.02, 0.3))
        if n % 2 == 0:      # a chunk
            s = int(rng.integers(1, min(cap, 40) + 1))
            p0 = int(rng.integers(0, cap - s + 1))
            name = f"rand{n}_chunk_h{hs}_g{hq // hkv}_s{s}_p{p0}"
            print("case", name, flush=True)
            q, k, v = _rand((s, bcap, hq, hs), q_seed, dtype), _rand((bcap, hkv, cap, hs), q_seed + 50, dtype), _rand((bcap, hkv, cap, hs), q_seed + 90, dtype)
            want, want_lse = orc.attention(q, k, v, scale, dtype, position_index=p0, batch=b)
            got, lse = _run(q, k, v, scale, dtype, p0=p0, batch=b)
        else:               # one token per sequence at its own position
            positions = [int(x) for x in rng.integers(0, cap, size=b)]
            name = f"rand{n}_step_h{hs}_g{hq // hkv}_pos{positions}"
            print("case", name, flush=True)
            q, k, v = _rand((1, bcap, hq, hs), q_seed, dtype), _rand((bcap, hkv, cap, hs), q_seed + 50, dtype), _rand((bcap, hkv, cap, hs), q_seed + 90, dtype)
            pos = np.zeros(bcap, dtype=np.uint32)
            pos[:b] = positions
            want, want_lse = orc.attention(q, k, v, scale, dtype, positions=pos, batch=b)
            got, lse = _run(q, k, v, scale, dtype, batch=b, positions=positions)
        _check(name, got, lse, want, want_lse, dtype, b)
