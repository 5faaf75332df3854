"""ellm_kv_append_attn_run / _run_ragged: the cache write of one new token per sequence (key RMS
norm + rotation) and the attention over the cache including it, as one launch.  Checked against
the two ordinary calls on the GPU (cache rows bit for bit: the same arithmetic, which
tests/test_gpu_kv_norm_rope.py checks against the oracle bit for bit) and against the oracle's
attention over the rows the cache then holds."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, LSE_TOL, compare, rand_storage, to_dev, torch_dtype

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


def _positions_dev(positions):
    import torch

    return torch.from_numpy(np.asarray(positions, dtype=np.uint32).view(np.int32).copy()).cuda()


def _bits(t):
    import torch

    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16).copy()


class _Step:
    """One layer of a cache (the second of two, so that layer offsets count), an attention operator over it
    and the new token's rows."""

    def __init__(self, dtype, bcap, hq, hkv, cap, seed, caps=None):
        import torch

        import ellm_amd

        self.dtype, self.bcap, self.hq, self.hkv = dtype, bcap, hq, hkv
        self.layer = 1
        tdt = torch_dtype(dtype)
        self.scale = 1.0 / np.sqrt(D)
        if caps is None:
            self.cache = ellm_amd.KVCache(2, bcap, hkv, cap, _code(dtype))
            self.kt, self.vt = self.cache.layer_tensors(self.layer, tdt)
            _, _, strides = self.cache.layer(self.layer)
            table = None
            self.caps = [cap] * bcap
        else:
            self.cache = ellm_amd.KVCache.ragged(2, caps, hkv, _code(dtype))
            self.kt, self.vt = self.cache.layer_flat_tensors(self.layer, tdt)
            table = self.cache.layer_ragged(self.layer)
            strides = table.strides
            self.caps = list(caps)
        self.k0 = to_dev(rand_storage(tuple(self.kt.shape), seed, dtype), dtype)
        self.v0 = to_dev(rand_storage(tuple(self.vt.shape), seed + 1, dtype), dtype)
        self.rope = to_dev(_rope_table(max(self.caps), dtype), dtype)
        self.q = to_dev(rand_storage((1, bcap, hq, D), seed + 2, dtype), dtype)
        self.k_new = to_dev(rand_storage((1, bcap, hkv, D), seed + 3, dtype, scale=1.7), dtype)
        self.v_new = to_dev(rand_storage((1, bcap, hkv, D), seed + 4, dtype), dtype)
        self.out = torch.zeros_like(self.q)
        self.lse = torch.zeros((1, bcap, hq), dtype=torch.float32, device="cuda")
        self.attn = ellm_amd.Attention(self.q, self.kt, self.vt, self.out, bcap, hq, hkv, D, strides, self.scale,
                                       lse=self.lse, sequence_capacity=None if table else cap,
                                       max_position_interval=1, seq_table=table)

    def reset(self):
        self.kt.copy_(self.k0)
        self.vt.copy_(self.v0)
        self.out.fill_(float("nan"))
        self.lse.fill_(float("nan"))

    def snapshot(self):
        import torch

        torch.cuda.synchronize()
        return [_bits(self.kt), _bits(self.vt), _bits(self.out), self.lse.cpu().numpy().copy()]

    def two_calls(self, positions, batch, shared=None, stream=None):
        if shared is not None:
            self.cache.append_norm_rope(self.layer, shared, self.k_new, self.v_new, self.rope, batch_size=batch, stream=stream)
            self.attn.run(shared, 1, batch, stream=stream)
        else:
            self.cache.append_norm_rope(self.layer, 0, self.k_new, self.v_new, self.rope, batch_size=batch,
                                        positions=positions, max_position=max(self.caps) - 1, stream=stream)
            self.attn.run_ragged(positions, max(self.caps) - 1, batch, stream=stream)

    def fused(self, positions, batch, shared=None, stream=None):
        if shared is not None:
            self.cache.append_norm_rope_with_attention(self.layer, self.attn, shared, self.k_new, self.v_new, self.rope,
                                                       batch_size=batch, stream=stream)
        else:
            self.cache.append_norm_rope_with_attention(self.layer, self.attn, 0, self.k_new, self.v_new, self.rope,
                                                       batch_size=batch, positions=positions,
                                                       max_position=max(self.caps) - 1, stream=stream)

    def close(self):
        self.attn.close()
        self.cache.close()


def _compare(step, plain, fused, batch):
    dtype = step.dtype
    assert np.array_equal(plain[0], fused[0]), "key cache"
    assert np.array_equal(plain[1], fused[1]), "value cache"
    f = lambda a: orc.from_storage(a, dtype)
    r = compare(f(fused[2])[:, :batch], f(plain[2])[:, :batch], dtype)
    assert r["ok"], r
    assert np.abs(fused[3][:, :batch] - plain[3][:, :batch]).max() <= LSE_TOL
    if batch < step.bcap:   # rows of sequences beyond the live batch are never written
        assert np.isnan(f(fused[2])[:, batch:]).all()


def _oracle_check(step, fused, positions, batch):
    """Attention of the oracle over the uniform cache the GPU now holds."""
    dtype = step.dtype
    pos = np.zeros(step.bcap, dtype=np.uint32)
    pos[:batch] = positions
    npdt = orc.storage_np_dtype(dtype)
    q = _bits(step.q).view(npdt)
    want, want_lse = orc.attention(q, fused[0].view(npdt), fused[1].view(npdt), step.scale, dtype, positions=pos, batch=batch)
    f = lambda a: orc.from_storage(a, dtype)
    r = compare(f(fused[2])[:, :batch], f(want)[:, :batch], dtype)
    assert r["ok"], r
    assert np.abs(fused[3][:, :batch] - want_lse[:, :batch]).max() <= LSE_TOL


# (name, dtype, batch capacity, batch, q heads, kv heads, capacity, per-sequence positions or one shared position)
CASES = [
    ("ragged_small_incl_first_token", orc.F16, 5, 5, 8, 2, 256, [17, 0, 200, 64, 99]),
    ("shared_position_on_chunk_edge", orc.F16, 4, 4, 8, 2, 1100, 1023),
    ("last_split_holds_only_the_new_key", orc.F16, 2, 2, 8, 2, 600, 512),
    ("first_token_of_every_sequence", orc.F16, 3, 3, 8, 2, 128, 0),
    ("batch_below_capacity_bf16", orc.BF16, 5, 3, 8, 2, 640, [600, 63, 301]),
    ("mha", orc.F16, 2, 2, 4, 4, 1024, [700, 15]),
    ("g32_two_head_groups_bf16", orc.BF16, 1, 1, 32, 1, 4096, 4000),
    ("qwen3_heads_b4_1k", orc.F16, 4, 4, 32, 4, 1100, [1023, 0, 511, 1099]),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_fused_cache_write_matches_the_two_calls_and_the_oracle(case):
    name, dtype, bcap, batch, hq, hkv, cap, positions = case
    print("case", name, flush=True)
    step = _Step(dtype, bcap, hq, hkv, cap, seed=11)
    try:
        shared = positions if np.isscalar(positions) else None
        plist = [positions] * batch if shared is not None else list(positions)
        dpos = None if shared is not None else _positions_dev(plist)
        step.reset()
        step.two_calls(dpos, batch, shared)
        plain = step.snapshot()
        step.reset()
        step.fused(dpos, batch, shared)
        fused = step.snapshot()
        _compare(step, plain, fused, batch)
        _oracle_check(step, fused, plist, batch)
        # the rows did change, and only they
        k0 = _bits(step.k0)
        mask = np.ones((bcap, hkv, cap), dtype=bool)
        for b in range(batch):
            mask[b, :, plist[b]] = False
        assert np.array_equal(fused[0][mask], k0[mask]) and not np.array_equal(fused[0][~mask], k0[~mask])
    finally:
        step.close()


def test_fused_cache_write_on_the_kernel_for_sequences_of_different_lengths():
    """Enough keys for the kernel that deals the planes' keys in equal shares (path 1 of
    ellm_attn_ragged_path)."""
    dtype = orc.F16
    bcap, hq, hkv, cap = 16, 32, 4, 4200
    positions = [4199, 0, 63, 64, 1000, 2047, 2048, 3000, 17, 4100, 128, 129, 500, 3999, 1, 2500]
    step = _Step(dtype, bcap, hq, hkv, cap, seed=40)
    try:
        assert step.attn.ragged_path(cap - 1, bcap) == 1
        dpos = _positions_dev(positions)
        step.reset()
        step.two_calls(dpos, bcap)
        plain = step.snapshot()
        step.reset()
        step.fused(dpos, bcap)
        fused = step.snapshot()
        _compare(step, plain, fused, bcap)
        _oracle_check(step, fused, positions, bcap)
    finally:
        step.close()


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16], ids=["f16", "bf16"])
def test_fused_cache_write_on_a_cache_with_per_sequence_capacities(dtype):
    caps = [320, 64, 1000, 129]
    step = _Step(dtype, len(caps), 8, 2, None, seed=60, caps=caps)
    try:
        for positions in ([319, 63, 999, 128], [0, 17, 512, 64]):
            dpos = _positions_dev(positions)
            step.reset()
            step.two_calls(dpos, len(caps))
            plain = step.snapshot()
            step.reset()
            step.fused(dpos, len(caps))
            fused = step.snapshot()
            _compare(step, plain, fused, len(caps))
    finally:
        step.close()


def test_fused_cache_write_recorded_into_a_graph_replays_like_eager():
    """The fused call + the advance of the positions recorded once and replayed while the positions
    move: equal to the eager calls bit for bit."""
    import torch

    import ellm_amd

    dtype = orc.F16
    bcap, hq, hkv, cap = 6, 16, 2, 700
    start = np.array([600, 3, 63, 255, 127, 400], dtype=np.uint32)
    steps = 4
    step = _Step(dtype, bcap, hq, hkv, cap, seed=70)
    stream = torch.cuda.Stream()

    def walk(use_graph):
        step.reset()
        pos = _positions_dev(start)
        snaps, graph = [], None
        with torch.cuda.stream(stream):
            def one():
                step.fused(pos, bcap, stream=stream)
                ellm_amd.positions_advance(pos, 1, stream=stream)

            for _ in range(steps):
                if not use_graph:
                    one()
                else:
                    if graph is None:
                        stream.synchronize()
                        with ellm_amd.StepGraph(stream) as graph:
                            one()
                    graph.launch()
                stream.synchronize()
                snaps.append(step.snapshot())
                _ = float(step.out.float().sum())     # eager work between replays
        if graph is not None:
            graph.close()
        return snaps, pos.cpu().numpy().view(np.uint32)

    try:
        eager, pos_e = walk(False)
        replay, pos_g = walk(True)
        assert np.array_equal(pos_e, start + steps) and np.array_equal(pos_g, pos_e)
        for n in range(steps):
            for a, b in zip(eager[n], replay[n]):
                assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), n
    finally:
        step.close()


def test_fused_cache_write_refuses_an_operator_over_other_memory():
    import torch

    import ellm_amd

    step = _Step(orc.F16, 2, 8, 2, 128, seed=80)
    other = _Step(orc.F16, 2, 8, 2, 128, seed=80)
    try:
        with pytest.raises(ellm_amd.EllmError) as e:   # other's operator reads other's cache
            step.cache.append_norm_rope_with_attention(step.layer, other.attn, 5, step.k_new, step.v_new, step.rope)
        assert e.value.status == 1 and "this layer of the cache" in e.value.message
        with pytest.raises(ellm_amd.EllmError) as e:   # the operator is over layer 1
            step.cache.append_norm_rope_with_attention(0, step.attn, 5, step.k_new, step.v_new, step.rope)
        assert e.value.status == 1
        with pytest.raises(ellm_amd.EllmError) as e:   # position beyond the capacity
            step.cache.append_norm_rope_with_attention(step.layer, step.attn, 128, step.k_new, step.v_new, step.rope)
        assert e.value.status == 3
        torch.cuda.synchronize()
    finally:
        step.close()
        other.close()


def test_random_shapes_against_the_two_calls_and_the_oracle():
    """Seeded sweep: group sizes 1..32, batches below capacity, capacities from a few rows to a few
    thousand, shared and per-sequence positions, both storage types."""
    rng = np.random.default_rng(77)
    for n in range(14):
        dtype = orc.F16 if n % 2 == 0 else orc.BF16
        hkv = int(rng.integers(1, 5))
        hq = hkv * int(rng.choice([1, 2, 3, 4, 8, 16, 32]))
        if hq > 64:
            hq = hkv * 8
        bcap = int(rng.integers(1, 7))
        batch = int(rng.integers(1, bcap + 1))
        cap = int(rng.choice([8, 65, 130, 700, 2100, 5000]))
        if n % 3 == 0:
            positions = int(rng.integers(0, cap))
        else:
            positions = [int(x) for x in rng.integers(0, cap, size=batch)]
        name = f"rand{n}_b{batch}of{bcap}_h{hq}kv{hkv}_cap{cap}_{positions}"
        print("case", name, flush=True)
        step = _Step(dtype, bcap, hq, hkv, cap, seed=200 + n)
        try:
            shared = positions if np.isscalar(positions) else None
            plist = [positions] * batch if shared is not None else list(positions)
            dpos = None if shared is not None else _positions_dev(plist)
            step.reset()
            step.two_calls(dpos, batch, shared)
            plain = step.snapshot()
            step.reset()
            step.fused(dpos, batch, shared)
            fused = step.snapshot()
            _compare(step, plain, fused, batch)
            _oracle_check(step, fused, plist, batch)
        finally:
            step.close()
