"""ellm_matmul3_attn_run / _run_ragged: the Q/K/V projection and the attention of a single-token
step as one call, in which the projection leaves raw sums and the attention launch finishes the
query rows and the new key / value row.  Checked against the oracle's MatMul3 followed by its
attention (the reference's two consecutive operators, src/qwen3_moe/attention.rs:126-174), and
against the two ordinary calls on the GPU."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, LSE_TOL, compare, compare_ulps, rand_storage, to_dev, to_host, torch_dtype

pytestmark = pytest.mark.gpu


def _rope_table(positions, dtype, theta=1.0e6):
    jj = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(positions, dtype=np.float64)[:, None] * theta ** (-2.0 * jj / D)[None, :]
    t = np.empty((positions, D), dtype=np.float32)
    t[:, 0::2], t[:, 1::2] = np.cos(ang), np.sin(ang)
    return orc.to_storage(t, dtype)


class _Layer:
    """Device buffers and the two operators of one layer's step."""

    def __init__(self, dtype, bcap, hq, hkv, cap, hidden, seed):
        import torch

        import ellm_amd

        self.dtype, self.bcap, self.hq, self.hkv, self.cap, self.hidden = dtype, bcap, hq, hkv, cap, hidden
        self.scale = 1.0 / np.sqrt(D)
        self.rope = _rope_table(cap, dtype)
        self.w = [rand_storage((h * D, hidden), seed + i, dtype, scale=hidden ** -0.5) for i, h in enumerate((hq, hkv, hkv))]
        self.k0 = rand_storage((bcap, hkv, cap, D), seed + 5, dtype)
        self.v0 = rand_storage((bcap, hkv, cap, D), seed + 6, dtype)
        self.x0 = rand_storage((1, bcap, hidden), seed + 7, dtype)
        tdt = torch_dtype(dtype)
        self.cache = ellm_amd.KVCache(1, bcap, hkv, cap, ellm_amd.DTYPE_F16 if dtype == orc.F16 else ellm_amd.DTYPE_BF16)
        self.kt, self.vt = self.cache.layer_tensors(0, tdt)
        _, _, self.strides = self.cache.layer(0)
        self.x = to_dev(self.x0, dtype)
        self.q = torch.zeros((1, bcap, hq, D), dtype=tdt, device="cuda")
        self.att = torch.zeros_like(self.q)
        self.lse = torch.zeros((1, bcap, hq), dtype=torch.float32, device="cuda")
        self.dev = [to_dev(a, dtype) for a in (*self.w, self.rope)]
        self.qkv = ellm_amd.MatMul3(self.x, self.dev[0], self.q, self.dev[1], self.kt, self.dev[2], self.vt, self.dev[3],
                                    D, bcap, hq, hkv, self.strides, cap)
        self.attn = ellm_amd.Attention(self.q, self.kt, self.vt, self.att, bcap, hq, hkv, D, self.strides, self.scale,
                                       lse=self.lse, sequence_capacity=cap, max_position_interval=1)

    def reset(self):
        self.kt.copy_(to_dev(self.k0, self.dtype))
        self.vt.copy_(to_dev(self.v0, self.dtype))
        self.q.fill_(float("nan"))
        self.att.fill_(float("nan"))
        self.lse.fill_(float("nan"))

    def snapshot(self):
        import torch

        torch.cuda.synchronize()
        bits = [t.view(torch.int16).cpu().numpy().view(np.uint16).copy() for t in (self.q, self.kt, self.vt, self.att)]
        return bits + [self.lse.cpu().numpy().copy()]

    def close(self):
        self.qkv.close()
        self.attn.close()
        self.cache.close()


def _positions_dev(positions):
    import torch

    return torch.from_numpy(np.asarray(positions, dtype=np.uint32).view(np.int32).copy()).cuda()


def _check_against_oracle(layer, got, positions, batch):
    """got: snapshot after the fused call.  Projection rows within one unit in the last place of the
    oracle's, untouched cache rows untouched, attention within the operator's tolerance of the oracle's
    attention over the rows the GPU produced."""
    dtype, hq, hkv, cap = layer.dtype, layer.hq, layer.hkv, layer.cap
    gq, gk, gv, gatt, glse = got
    oq = np.zeros((1, layer.bcap, hq, D), dtype=np.uint16)
    kc, vc = layer.k0.view(np.uint16).copy(), layer.v0.view(np.uint16).copy()
    pos = np.zeros(layer.bcap, dtype=np.uint32)
    pos[:batch] = positions
    assert orc.matmul3(layer.x0, *layer.w, oq, kc, vc, layer.rope, (hkv * cap * D, cap * D, D, 1), cap, 0, 1, dtype,
                       batch_size=batch, positions=pos) == 0
    f = lambda a: orc.from_storage(a, dtype)
    r = compare_ulps(f(gq)[:, :batch], f(oq)[:, :batch], dtype)
    assert r["ok"], ("q", r)
    r = compare_ulps(f(gk), f(kc), dtype)
    assert r["ok"], ("k", r)
    r = compare_ulps(f(gv), f(vc), dtype)
    assert r["ok"], ("v", r)
    # only the rows at the sequences' positions changed
    mask = np.ones((layer.bcap, hkv, cap), dtype=bool)
    for b in range(batch):
        mask[b, :, pos[b]] = False
    assert np.array_equal(gk[mask], layer.k0.view(np.uint16)[mask]) and np.array_equal(gv[mask], layer.v0.view(np.uint16)[mask])
    want, want_lse = orc.attention(gq.view(layer.k0.dtype), gk.view(layer.k0.dtype), gv.view(layer.k0.dtype), layer.scale,
                                   dtype, positions=pos, batch=batch)
    r = compare(f(gatt)[:, :batch], f(want)[:, :batch], dtype)
    assert r["ok"], ("attention", r)
    assert np.abs(glse[:, :batch] - want_lse[:, :batch]).max() <= LSE_TOL
    if batch < layer.bcap:   # rows of sequences beyond the live batch are never written
        assert np.isnan(f(gatt)[:, batch:]).all() and np.isnan(f(gq)[:, batch:]).all()


# (name, dtype, batch capacity, batch, q heads, kv heads, capacity, hidden, positions or one shared position)
CASES = [
    ("ragged_small_incl_first_token", orc.F16, 5, 5, 8, 2, 256, 1024, [17, 0, 200, 64, 99]),
    ("shared_position_on_chunk_edge", orc.F16, 4, 4, 8, 2, 1100, 1024, 1023),
    ("last_split_holds_only_the_new_key", orc.F16, 2, 2, 8, 2, 600, 1024, 512),
    ("first_token_of_every_sequence", orc.F16, 3, 3, 8, 2, 128, 1024, 0),
    ("batch_below_capacity_bf16", orc.BF16, 5, 3, 8, 2, 640, 1024, [600, 63, 301]),
    ("mha", orc.F16, 2, 2, 4, 4, 1024, 1024, [700, 15]),
    ("g16_bf16", orc.BF16, 2, 2, 16, 1, 2100, 1024, [2047, 1500]),
    ("g32_two_head_groups", orc.F16, 1, 1, 32, 1, 4096, 1024, 4000),
    ("qwen3_heads_b16_2048_wide", orc.F16, 16, 16, 32, 4, 1100, 2048,
     [1023, 0, 5, 64, 63, 1000, 512, 511, 256, 700, 1, 1099, 128, 333, 900, 65]),
    ("k4096_sixteen_waves", orc.F16, 3, 3, 8, 2, 300, 4096, [299, 7, 128]),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_fused_step_matches_the_oracle_and_the_two_ordinary_calls(case):
    import torch

    name, dtype, bcap, batch, hq, hkv, cap, hidden, positions = case
    print("case", name, flush=True)
    layer = _Layer(dtype, bcap, hq, hkv, cap, hidden, seed=10)
    try:
        assert layer.qkv.attention_path(layer.attn, batch) == 1
        ragged = not np.isscalar(positions)
        plist = list(positions) if ragged else [positions] * batch
        dpos = _positions_dev(plist) if ragged else None
        bound = int(max(plist))
        # the two ordinary calls
        layer.reset()
        if ragged:
            layer.qkv.run_ragged(dpos, bound, batch)
            layer.attn.run_ragged(dpos, bound, batch)
        else:
            layer.qkv.run(bound, 1, batch)
            layer.attn.run(bound, 1, batch)
        plain = layer.snapshot()
        # fused
        layer.reset()
        layer.qkv.run_with_attention(layer.attn, bound, batch, positions=dpos)
        fused = layer.snapshot()
        _check_against_oracle(layer, fused, plist, batch)
        # against the ordinary calls: the finishing arithmetic is the same, lane for lane, so the
        # projection's rows carry the same bits; attention takes the new key in a different chunk
        for what, a, b in zip(("q", "k", "v"), plain[:3], fused[:3]):
            live = (slice(None), slice(0, batch)) if what == "q" else slice(None)
            assert np.array_equal(a[live], b[live]), what
        f = lambda a: orc.from_storage(a, dtype)
        r = compare(f(fused[3])[:, :batch], f(plain[3])[:, :batch], dtype)
        assert r["ok"], r
        assert np.abs(fused[4][:, :batch] - plain[4][:, :batch]).max() <= LSE_TOL
        torch.cuda.synchronize()
    finally:
        layer.close()


def test_fused_step_takes_the_kernel_for_sequences_of_different_lengths():
    """Enough keys for the kernel that deals the planes' keys in equal shares (path 1 of
    ellm_attn_ragged_path): the piece that ends a plane finishes the new key there too."""
    dtype = orc.F16
    bcap, hq, hkv, cap, hidden = 16, 32, 4, 4200, 2048
    positions = [4199, 0, 63, 64, 1000, 2047, 2048, 3000, 17, 4100, 128, 129, 500, 3999, 1, 2500]
    layer = _Layer(dtype, bcap, hq, hkv, cap, hidden, seed=40)
    try:
        assert layer.attn.ragged_path(cap - 1, bcap) == 1
        assert layer.qkv.attention_path(layer.attn, bcap) == 1
        layer.reset()
        layer.qkv.run_with_attention(layer.attn, cap - 1, bcap, positions=_positions_dev(positions))
        _check_against_oracle(layer, layer.snapshot(), positions, bcap)
    finally:
        layer.close()


def test_fused_step_recorded_into_a_graph_replays_like_eager():
    """The fused call + the output projection + the advance of the positions recorded once and
    replayed while the positions move: equal to the eager calls bit for bit."""
    import torch

    import ellm_amd

    dtype = orc.F16
    bcap, hq, hkv, cap, hidden = 6, 16, 2, 700, 1024
    start = np.array([600, 3, 63, 255, 127, 400], dtype=np.uint32)
    steps = 4
    layer = _Layer(dtype, bcap, hq, hkv, cap, hidden, seed=70)
    wo = to_dev(rand_storage((hidden, hq * D), 99, dtype, scale=(hq * D) ** -0.5), dtype)
    out = torch.zeros((1, bcap, hidden), dtype=torch.float16, device="cuda")
    oproj = ellm_amd.MatMulAdd(layer.att.view(1, bcap, hq * D), wo, layer.x, out)
    stream = torch.cuda.Stream()

    def walk(use_graph):
        layer.reset()
        pos = _positions_dev(start)
        snaps, graph = [], None
        with torch.cuda.stream(stream):
            def step():
                layer.qkv.run_with_attention(layer.attn, cap - 1, bcap, positions=pos, stream=stream)
                oproj.run(0, 1, bcap, stream=stream)
                ellm_amd.positions_advance(pos, 1, stream=stream)

            for _ in range(steps):
                if not use_graph:
                    step()
                else:
                    if graph is None:
                        stream.synchronize()
                        with ellm_amd.StepGraph(stream) as graph:
                            step()
                    graph.launch()
                stream.synchronize()
                snaps.append(layer.snapshot() + [out.view(torch.int16).cpu().numpy().copy()])
                _ = float(out.float().sum())     # eager work between replays
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
        oproj.close()
        layer.close()


def test_fused_step_refuses_handles_of_different_steps():
    import torch

    import ellm_amd

    a = _Layer(orc.F16, 2, 8, 2, 128, 1024, seed=80)
    b = _Layer(orc.F16, 2, 8, 2, 128, 1024, seed=80)
    try:
        with pytest.raises(ellm_amd.EllmError) as e:
            a.qkv.run_with_attention(b.attn, 5, 2)      # b's attention reads b's q and caches
        assert e.value.status == 1 and "q_state" in e.value.message
        torch.cuda.synchronize()
    finally:
        a.close()
        b.close()


def _two_calls_and_fused(make_ops, reset, snapshot, positions, batch):
    """Runs the step as the two ordinary calls and as the fused call on freshly reset buffers;
    returns both snapshots."""
    import torch

    qkv, attn = make_ops()
    try:
        assert qkv.attention_path(attn, batch) == 1
        dpos = _positions_dev(positions)
        bound = int(max(positions))
        reset()
        qkv.run_ragged(dpos, bound, batch)
        attn.run_ragged(dpos, bound, batch)
        plain = snapshot()
        reset()
        qkv.run_with_attention(attn, bound, batch, positions=dpos)
        fused = snapshot()
        torch.cuda.synchronize()
    finally:
        qkv.close()
        attn.close()
    return plain, fused


def _assert_fused_equals_plain(plain, fused, dtype, batch):
    for what, a, b in zip(("q", "k", "v"), plain[:3], fused[:3]):
        live = (slice(None), slice(0, batch)) if what == "q" else slice(None)
        assert np.array_equal(a[live], b[live]), what
    f = lambda a: orc.from_storage(a, dtype)
    r = compare(f(fused[3])[:, :batch], f(plain[3])[:, :batch], dtype)
    assert r["ok"], r
    assert np.abs(fused[4][:, :batch] - plain[4][:, :batch]).max() <= LSE_TOL


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16], ids=["f16", "bf16"])
def test_fused_step_on_a_cache_with_per_sequence_capacities(dtype):
    """Both handles over one layer of an ellm_kv_create_ragged cache (the same sequence table):
    the new rows land where the two ordinary calls put them, bit for bit, the last row of the
    shortest plane included; the ordinary calls on this cache are checked against the uniform
    cache and the oracle in test_gpu_ragged_cache.py."""
    import torch

    import ellm_amd

    caps = [320, 64, 1000, 129]
    hq, hkv, hidden, b = 8, 2, 1024, 4
    tdt = torch_dtype(dtype)
    cache = ellm_amd.KVCache.ragged(1, caps, hkv, ellm_amd.DTYPE_F16 if dtype == orc.F16 else ellm_amd.DTYPE_BF16)
    view = cache.layer_ragged(0)
    kt, vt = cache.layer_flat_tensors(0, tdt)
    k0 = to_dev(rand_storage(tuple(kt.shape), 3, dtype), dtype)
    v0 = to_dev(rand_storage(tuple(vt.shape), 4, dtype), dtype)
    w = [to_dev(rand_storage((h * D, hidden), 20 + i, dtype, scale=hidden ** -0.5), dtype) for i, h in enumerate((hq, hkv, hkv))]
    rope = to_dev(_rope_table(max(caps), dtype), dtype)
    x = to_dev(rand_storage((1, b, hidden), 30, dtype), dtype)
    q = torch.zeros((1, b, hq, D), dtype=tdt, device="cuda")
    att = torch.zeros_like(q)
    lse = torch.zeros((1, b, hq), dtype=torch.float32, device="cuda")

    def make_ops():
        return (ellm_amd.MatMul3(x, w[0], q, w[1], kt, w[2], vt, rope, D, b, hq, hkv, view.strides, 0, seq_table=view),
                ellm_amd.Attention(q, kt, vt, att, b, hq, hkv, D, view.strides, 1.0 / np.sqrt(D), lse=lse,
                                   max_position_interval=1, seq_table=view))

    def reset():
        kt.copy_(k0.view(kt.shape))
        vt.copy_(v0.view(vt.shape))
        for t in (q, att, lse):
            t.fill_(float("nan"))

    def snapshot():
        torch.cuda.synchronize()
        return [t.view(torch.int16).cpu().numpy().view(np.uint16).copy() for t in (q, kt, vt, att)] + [lse.cpu().numpy().copy()]

    try:
        for positions in ([319, 63, 999, 128], [0, 17, 512, 64]):
            print("positions", positions, flush=True)
            plain, fused = _two_calls_and_fused(make_ops, reset, snapshot, positions, b)
            _assert_fused_equals_plain(plain, fused, dtype, b)
            assert not np.isnan(orc.from_storage(fused[3], dtype)).any()
    finally:
        cache.close()


def test_fused_step_on_the_reference_state_layout():
    """K/V as the reference's own [position][sequence][kv_head][128] state
    (src/qwen3_moe/attention.rs:149-166), kv_strides = [Hkv*D, D, B*Hkv*D, 1]: the fused call
    against the two ordinary calls, whose results on this layout test_gpu_parity.py and
    test_gpu_projection.py check against the oracle."""
    import torch

    import ellm_amd

    dtype = orc.F16
    b, hq, hkv, cap, hidden = 3, 8, 2, 600, 1024
    strides = [hkv * D, D, b * hkv * D, 1]
    k0 = to_dev(rand_storage((cap, b, hkv, D), 5, dtype), dtype)
    v0 = to_dev(rand_storage((cap, b, hkv, D), 6, dtype), dtype)
    kt, vt = torch.zeros_like(k0), torch.zeros_like(v0)
    w = [to_dev(rand_storage((h * D, hidden), 40 + i, dtype, scale=hidden ** -0.5), dtype) for i, h in enumerate((hq, hkv, hkv))]
    rope = to_dev(_rope_table(cap, dtype), dtype)
    x = to_dev(rand_storage((1, b, hidden), 50, dtype), dtype)
    q = torch.zeros((1, b, hq, D), dtype=torch.float16, device="cuda")
    att = torch.zeros_like(q)
    lse = torch.zeros((1, b, hq), dtype=torch.float32, device="cuda")

    def make_ops():
        return (ellm_amd.MatMul3(x, w[0], q, w[1], kt, w[2], vt, rope, D, b, hq, hkv, strides, cap),
                ellm_amd.Attention(q, kt, vt, att, b, hq, hkv, D, strides, 1.0 / np.sqrt(D), lse=lse,
                                   sequence_capacity=cap, max_position_interval=1))

    def reset():
        kt.copy_(k0)
        vt.copy_(v0)
        for t in (q, att, lse):
            t.fill_(float("nan"))

    def snapshot():
        torch.cuda.synchronize()
        return [t.view(torch.int16).cpu().numpy().view(np.uint16).copy() for t in (q, kt, vt, att)] + [lse.cpu().numpy().copy()]

    positions = [599, 0, 300]
    plain, fused = _two_calls_and_fused(make_ops, reset, snapshot, positions, b)
    _assert_fused_equals_plain(plain, fused, dtype, b)
    # only the rows at the sequences' positions changed, and they did change
    kb, k0b = fused[1], k0.view(torch.int16).cpu().numpy().view(np.uint16)
    mask = np.ones((cap, b, hkv), dtype=bool)
    for s, p in enumerate(positions):
        mask[p, s, :] = False
    assert np.array_equal(kb[mask], k0b[mask]) and not np.array_equal(kb[~mask], k0b[~mask])
