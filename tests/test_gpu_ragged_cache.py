"""A cache whose sequences have different capacities (ellm_kv_create_ragged) against the
uniform cache (one capacity for all), through the C ABI.  Every kernel does the same
arithmetic on both and only the addresses differ, so cache contents and attention outputs
must be equal bit for bit; the uniform path itself is checked against the oracle elsewhere,
and once more here."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, compare, rand_storage, to_dev, to_host, torch_dtype

pytestmark = pytest.mark.gpu

CAPS = [320, 64, 1000, 129]
HQ, HKV, LAYERS, HIDDEN = 8, 2, 2, 256


def _code(dtype):
    import ellm_amd

    return ellm_amd.DTYPE_F16 if dtype == orc.F16 else ellm_amd.DTYPE_BF16


def _rope_table(positions, dtype, theta=1.0e6):
    jj = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(positions, dtype=np.float64)[:, None] * theta ** (-2.0 * jj / D)[None, :]
    t = np.empty((positions, D), dtype=np.float32)
    t[:, 0::2], t[:, 1::2] = np.cos(ang), np.sin(ang)
    return orc.to_storage(t, dtype)


def _bits(t):
    import torch

    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


class _Pair:
    """The same model state in a uniform cache (capacity max(CAPS)) and a ragged one."""

    def __init__(self, dtype):
        import ellm_amd

        self.dtype = dtype
        self.td = torch_dtype(dtype)
        self.uni = ellm_amd.KVCache(LAYERS, len(CAPS), HKV, max(CAPS), _code(dtype))
        self.rag = ellm_amd.KVCache.ragged(LAYERS, CAPS, HKV, _code(dtype))

    def planes_equal(self, layer):
        uk, uv = self.uni.layer_tensors(layer, self.td)
        rk, rv = self.rag.layer_flat_tensors(layer, self.td)
        off = 0
        for s, cap in enumerate(CAPS):
            for u, r in ((uk, rk), (uv, rv)):
                if not np.array_equal(_bits(u[s, :, :cap]), _bits(r[:, off:off + cap])):
                    return False
            off += cap
        return True

    def fill_random(self, layer, seed):
        import torch

        uk, uv = self.uni.layer_tensors(layer, self.td)
        rk, rv = self.rag.layer_flat_tensors(layer, self.td)
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        uk.copy_(torch.randn(uk.shape, generator=g, device="cuda").to(self.td))
        uv.copy_(torch.randn(uv.shape, generator=g, device="cuda").to(self.td))
        off = 0
        for s, cap in enumerate(CAPS):
            rk[:, off:off + cap] = uk[s, :, :cap]
            rv[:, off:off + cap] = uv[s, :, :cap]
            off += cap

    def close(self):
        self.uni.close()
        self.rag.close()


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
def test_cache_writes_land_on_the_same_rows(dtype):
    """ellm_kv_append, ellm_kv_append_norm_rope (shared and per-sequence positions) and the
    fused projection (chunk and single-token) write the same bits into both caches."""
    import torch

    import ellm_amd

    p = _Pair(dtype)
    b = len(CAPS)
    rope = to_dev(_rope_table(max(CAPS), dtype), dtype)
    layer = 1
    # plain append: 40 tokens from position 0 (fits the shortest sequence, 64)
    ks, vs = (to_dev(rand_storage((40, b, HKV, D), 5 + i, dtype), dtype) for i in range(2))
    for c in (p.uni, p.rag):
        c.append(layer, 0, ks, vs)
    # norm + rope append at a shared position, then at per-sequence positions
    ks2, vs2 = (to_dev(rand_storage((20, b, HKV, D), 7 + i, dtype, scale=2.0), dtype) for i in range(2))
    for c in (p.uni, p.rag):
        c.append_norm_rope(layer, 40, ks2, vs2, rope)
    starts = np.array([300, 60, 900, 100], dtype=np.int32)
    dstarts = torch.from_numpy(starts).cuda()
    ks3, vs3 = (to_dev(rand_storage((3, b, HKV, D), 9 + i, dtype), dtype) for i in range(2))
    for c in (p.uni, p.rag):
        c.append_norm_rope(layer, 0, ks3, vs3, rope, positions=dstarts, max_position=int(starts.max()))
    torch.cuda.synchronize()
    assert p.planes_equal(layer)

    # the fused projection: a chunk of 70 rows x 4 sequences is too long for sequence 1 ...
    w = [to_dev(rand_storage((h * D, HIDDEN), 20 + i, dtype, scale=HIDDEN ** -0.5), dtype)
         for i, h in enumerate((HQ, HKV, HKV))]
    hid = to_dev(rand_storage((50, b, HIDDEN), 30, dtype), dtype)
    outs = []
    for c, ragged in ((p.uni, False), (p.rag, True)):
        q = torch.zeros((50, b, HQ, D), dtype=p.td, device="cuda")
        if ragged:
            view = c.layer_ragged(0)
            kt, vt = c.layer_flat_tensors(0, p.td)
            op = ellm_amd.MatMul3(hid, w[0], q, w[1], kt, w[2], vt, rope, D, b, HQ, HKV, view.strides, 0,
                                  seq_table=view)
            with pytest.raises(ellm_amd.EllmError) as e:
                op.run(20, 50, b)            # positions 20..69 do not fit sequence 1 (64)
            assert e.value.status == 3 and "sequence 1" in e.value.message
        else:
            kt, vt = c.layer_tensors(0, p.td)
            _, _, strides = c.layer(0)
            op = ellm_amd.MatMul3(hid, w[0], q, w[1], kt, w[2], vt, rope, D, b, HQ, HKV, strides, max(CAPS))
        op.run(10, 50, b)                    # 200 rows: an MFMA tile kernel
        op.run_ragged(dstarts, int(starts.max()), b)   # 4 rows: the few-rows kernel
        torch.cuda.synchronize()
        outs.append(_bits(q))
        op.close()
    assert np.array_equal(outs[0], outs[1])
    assert p.planes_equal(0)
    p.close()


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
def test_attention_reads_the_same_rows(dtype):
    import torch

    import ellm_amd

    p = _Pair(dtype)
    p.fill_random(0, 3)
    b = len(CAPS)
    scale = 1.0 / np.sqrt(D)
    uk, uv = p.uni.layer_tensors(0, p.td)
    _, _, ustr = p.uni.layer(0)
    view = p.rag.layer_ragged(0)
    rk, rv = p.rag.layer_flat_tensors(0, p.td)

    def ops(q, out, lse, interval):
        return (ellm_amd.Attention(q, uk, uv, out[0], b, HQ, HKV, D, ustr, scale, lse=lse[0],
                                   sequence_capacity=max(CAPS), max_position_interval=interval),
                ellm_amd.Attention(q, rk, rv, out[1], b, HQ, HKV, D, view.strides, scale, lse=lse[1],
                                   max_position_interval=interval, seq_table=view))

    # single token, one position per sequence: the last row of every plane
    qh = rand_storage((1, b, HQ, D), 11, dtype)
    q = to_dev(qh, dtype)
    out = [torch.zeros_like(q) for _ in range(2)]
    lse = [torch.zeros((1, b, HQ), dtype=torch.float32, device="cuda") for _ in range(2)]
    pos = np.array([c - 1 for c in CAPS], dtype=np.int32)
    dpos = torch.from_numpy(pos).cuda()
    u, r = ops(q, out, lse, 1)
    u.run_ragged(dpos, int(pos.max()), b)
    r.run_ragged(dpos, int(pos.max()), b)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(out[0]), _bits(out[1]))
    assert np.array_equal(lse[0].cpu().numpy().view(np.uint32), lse[1].cpu().numpy().view(np.uint32))
    # ... and against the oracle on what the ragged cache holds
    kh = _bits(uk).view(np.float16 if dtype == orc.F16 else np.uint16)
    vh = _bits(uv).view(np.float16 if dtype == orc.F16 else np.uint16)
    want, want_lse = orc.attention(qh, kh, vh, scale, dtype, positions=pos.astype(np.uint32))
    res = compare(to_host(out[1], dtype), orc.from_storage(want, dtype), dtype)
    assert res["ok"], res
    assert np.abs(lse[1].cpu().numpy() - want_lse).max() <= 1e-4
    # a position beyond a sequence's own capacity is clamped to its last row on the device
    wild = torch.from_numpy(np.array([999, 999, 999, 999], dtype=np.int32)).cuda()
    out2 = torch.zeros_like(q)
    r2 = ellm_amd.Attention(q, rk, rv, out2, b, HQ, HKV, D, view.strides, scale, max_position_interval=1,
                            seq_table=view)
    r2.run_ragged(wild, 999, b)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(out2), _bits(out[1]))
    r2.close()
    # a shared position must fit every sequence of the call
    with pytest.raises(ellm_amd.EllmError) as e:
        r.run(64, 1, b)
    assert e.value.status == 3
    r.run(63, 1, b)
    u.run(63, 1, b)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(out[0]), _bits(out[1]))
    u.close()
    r.close()

    # a chunk of 50 tokens at positions 10..59 of all four sequences
    qh = rand_storage((50, b, HQ, D), 12, dtype)
    q = to_dev(qh, dtype)
    out = [torch.zeros_like(q) for _ in range(2)]
    lse = [torch.zeros((50, b, HQ), dtype=torch.float32, device="cuda") for _ in range(2)]
    u, r = ops(q, out, lse, 50)
    u.run(10, 50, b)
    r.run(10, 50, b)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(out[0]), _bits(out[1]))
    assert np.array_equal(lse[0].cpu().numpy().view(np.uint32), lse[1].cpu().numpy().view(np.uint32))
    u.close()
    r.close()

    # a view that starts at sequence 2: the operator's sequences 0, 1 are the cache's 2, 3
    view2 = p.rag.layer_ragged(0, first_sequence=2)
    assert view2.capacities == CAPS[2:]
    qh = rand_storage((1, 2, HQ, D), 13, dtype)
    q = to_dev(qh, dtype)
    outv = torch.zeros_like(q)
    rv2 = ellm_amd.Attention(q, rk, rv, outv, 2, HQ, HKV, D, view2.strides, scale, max_position_interval=1,
                             seq_table=view2)
    pos2 = np.array([CAPS[2] - 1, CAPS[3] - 1], dtype=np.int32)
    rv2.run_ragged(torch.from_numpy(pos2).cuda(), int(pos2.max()), 2)
    torch.cuda.synchronize()
    want, _ = orc.attention(qh, np.ascontiguousarray(kh[2:]), np.ascontiguousarray(vh[2:]), scale, dtype,
                            positions=pos2.astype(np.uint32))
    res = compare(to_host(outv, dtype), orc.from_storage(want, dtype), dtype)
    assert res["ok"], res
    rv2.close()
    p.close()


def test_ragged_cache_argument_checks():
    import ctypes

    import ellm_amd
    from ellm_amd import _lib

    lib = ellm_amd.load_library()
    c = ellm_amd.KVCache.ragged(1, [16, 48], 2, ellm_amd.DTYPE_F16)
    k, v = ctypes.c_void_p(), ctypes.c_void_p()
    strides = (ctypes.c_size_t * 4)()
    assert lib.ellm_kv_layer(c._handle, 0, ctypes.byref(k), ctypes.byref(v), ctypes.byref(strides)) == 1
    assert b"ellm_kv_layer_ragged" in lib.ellm_last_error_string()
    table = _lib.KvSeqTable()
    assert lib.ellm_kv_layer_ragged(c._handle, 0, 2, ctypes.byref(k), ctypes.byref(v), ctypes.byref(strides),
                                    ctypes.byref(table)) == 3
    assert lib.ellm_kv_layer_ragged(c._handle, 1, 0, ctypes.byref(k), ctypes.byref(v), ctypes.byref(strides),
                                    ctypes.byref(table)) == 3
    view = c.layer_ragged(0)
    assert view.capacities == [16, 48] and view.offsets == [0, 16 * 128]
    assert view.strides[1] == 64 * 128 and view.strides[2] == 128 and view.strides[3] == 1
    u = ellm_amd.KVCache(1, 2, 2, 16, ellm_amd.DTYPE_F16)
    assert lib.ellm_kv_layer_ragged(u._handle, 0, 0, ctypes.byref(k), ctypes.byref(v), ctypes.byref(strides),
                                    ctypes.byref(table)) == 1
    caps = (ctypes.c_size_t * 2)(16, 0)
    bad = _lib.KvRaggedDesc(1, 2, 2, 128, caps, 0)
    h = ctypes.c_void_p()
    assert lib.ellm_kv_create_ragged(ctypes.byref(bad), ctypes.byref(h)) == 1 and not h.value
    c.close()
    u.close()
