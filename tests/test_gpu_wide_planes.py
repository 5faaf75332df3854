"""K/V planes that span more than 2^31 elements: the reference's own physical state
[position][sequence][kv_head][128] (src/qwen3_moe/attention.rs:149-166, viewed [sequence][kv_head]
[position][128] through its four strides) at the scale of BASELINE configs[4], 33 sequences x 4 K/V
heads x 131072 positions: rows of a plane lie 33 x 4 x 128 elements apart and the last one starts
4.4e9 bytes behind the first.  Every kernel that walks a plane (tile kernel, its split form, the
streaming chunk kernel, both single-token kernels) and the projection that writes K/V rows there,
against the oracle on sampled rows."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, LSE_TOL, compare, compare_ulps, rand_storage, to_dev, to_host

pytestmark = pytest.mark.gpu

SEQS, HKV, HQ, POSITIONS = 33, 4, 32, 131072
G = HQ // HKV
STRIDES = [HKV * D, D, SEQS * HKV * D, 1]        # sequence, kv head, position, element


@pytest.fixture(scope="module")
def state():
    import torch

    free, _ = torch.cuda.mem_get_info()
    if free < 12 * 2 ** 30:
        pytest.skip("needs 12 GB of free device memory")
    g = torch.Generator(device="cuda")
    g.manual_seed(123)
    k = torch.empty((POSITIONS, SEQS, HKV, D), dtype=torch.float16, device="cuda")
    v = torch.empty_like(k)
    for t in (k, v):                 # in slabs: randn makes binary32 first
        for p0 in range(0, POSITIONS, 8192):
            t[p0:p0 + 8192] = torch.randn((8192, SEQS, HKV, D), generator=g, device="cuda", dtype=torch.float32).to(torch.float16)
    assert k.numel() > 2 ** 31
    yield k, v
    del k, v
    torch.cuda.empty_cache()


def _plane(t, seq, kvh):
    """The rows of one (sequence, kv head) plane as a compact [1, 1, positions, 128] storage array."""
    import torch

    return t[:, seq, kvh, :].contiguous().view(torch.int16).cpu().numpy().view(np.float16)[None, None]


def _oracle_rows(q_rows, kp, vp, positions, scale):
    """q_rows [n, 128] (one head each) at `positions` over the compact plane: float32 rows + lse."""
    n = len(positions)
    out = np.zeros((n, D), dtype=np.float32)
    lse = np.zeros(n, dtype=np.float32)
    for i in range(n):
        o, l = orc.flash_attention_row(q_rows[i], kp[0, 0], vp[0, 0], scale, int(positions[i]), orc.F16)
        out[i], lse[i] = orc.from_storage(o, orc.F16), l
    return out, lse


def _check_rows(got, got_lse, q, kp_vp, rows, p0, scale):
    """rows: (token, sequence, head) triples of the call; kp_vp[(seq, kvh)] = compact planes."""
    for tok, seq, head in rows:
        kp, vp = kp_vp[(seq, head // G)]
        want, want_lse = _oracle_rows(q[tok, seq, head][None], kp, vp, [p0 + tok], scale)
        r = compare(got[tok, seq, head][None], want, orc.F16)
        assert r["ok"], ((tok, seq, head), r)
        assert abs(got_lse[tok, seq, head] - want_lse[0]) <= LSE_TOL, (tok, seq, head)


@pytest.mark.parametrize("interval,p0", [(1, POSITIONS - 1), (8, POSITIONS - 8), (70, POSITIONS - 70), (600, 130000)],
                         ids=["single_token", "stream_chunk", "split_tiles", "tiles"])
def test_attention_over_planes_beyond_2_31_elements(state, interval, p0):
    import torch

    import ellm_amd

    k, v = state
    batch = SEQS if interval <= 70 else 2
    scale = 1.0 / np.sqrt(D)
    q = rand_storage((interval, SEQS, HQ, D), 7, orc.F16)
    dq = to_dev(q, orc.F16)
    dout = torch.full_like(dq, float("nan"))
    dlse = torch.full((interval, SEQS, HQ), float("nan"), dtype=torch.float32, device="cuda")
    op = ellm_amd.Attention(dq, k, v, dout, SEQS, HQ, HKV, D, STRIDES, scale, lse=dlse,
                            sequence_capacity=POSITIONS, max_position_interval=interval)
    try:
        op.run(p0, interval, batch)
        torch.cuda.synchronize()
        got, got_lse = to_host(dout, orc.F16), dlse.cpu().numpy()
        seqs = sorted({0, batch - 1})
        planes = {(s, h): (_plane(k, s, h), _plane(v, s, h)) for s in seqs for h in (0, HKV - 1)}
        toks = sorted({0, interval // 2, interval - 1})
        rows = [(t, s, h) for t in toks for s in seqs for h in (0, G - 1, HQ - 1)]
        _check_rows(got, got_lse, q, planes, rows, p0, scale)
        assert not np.isnan(got[:, :batch]).any()
        if interval == 1:      # the same through per-sequence positions (the kernel that deals the keys in equal shares)
            pos = np.full(SEQS, POSITIONS - 1, dtype=np.uint32)
            pos[1::2] = np.arange(SEQS // 2) * 3001 + 70000
            dpos = torch.from_numpy(pos.view(np.int32)).cuda()
            assert op.ragged_path(POSITIONS - 1, SEQS) == 1
            dout.fill_(float("nan"))
            op.run_ragged(dpos, POSITIONS - 1, SEQS)
            torch.cuda.synchronize()
            got, got_lse = to_host(dout, orc.F16), dlse.cpu().numpy()
            for seq in (0, 1, SEQS - 1):
                for head in (0, HQ - 1):
                    kp, vp = _plane(k, seq, head // G), _plane(v, seq, head // G)
                    want, want_lse = _oracle_rows(q[0, seq, head][None], kp, vp, [int(pos[seq])], scale)
                    assert compare(got[0, seq, head][None], want, orc.F16)["ok"], (seq, head)
                    assert abs(got_lse[0, seq, head] - want_lse[0]) <= LSE_TOL
    finally:
        op.close()


def test_projection_writes_rows_beyond_2_31_elements(state):
    """The fused Q/K/V projection writing its key / value rows to token coordinates of this state,
    at a position whose row starts more than 2^32 bytes into the plane (few-rows kernel and
    one-head tiles)."""
    import torch

    import ellm_amd

    k, v = state
    hidden = 1024
    w = [rand_storage((h * D, hidden), 20 + i, orc.F16, scale=hidden ** -0.5) for i, h in enumerate((HQ, HKV, HKV))]
    rope = np.zeros((8, D), dtype=np.float32)
    rope[:, 0::2] = 1.0                                   # (cos, sin) = (1, 0): rotation by nothing
    rope = orc.to_storage(rope, orc.F16)
    dev = [to_dev(a, orc.F16) for a in (*w, rope)]
    for interval, pos in ((1, POSITIONS - 3), (3, POSITIONS - 40)):
        x = rand_storage((interval, SEQS, hidden), 30 + interval, orc.F16)
        dx = to_dev(x, orc.F16)
        dq = torch.zeros((interval, SEQS, HQ, D), dtype=torch.float16, device="cuda")
        proj = ellm_amd.MatMul3(dx, dev[0], dq, dev[1], k, dev[2], v, dev[3], D, SEQS, HQ, HKV, STRIDES, POSITIONS,
                                rope_position_stride=0, rope_head_stride=0)
        try:
            proj.run(pos, interval, SEQS)
            torch.cuda.synchronize()
            # oracle on compact states of two sequences
            for seq in (0, SEQS - 1):
                xs = np.ascontiguousarray(x[:, seq:seq + 1])
                oq = np.zeros((interval, 1, HQ, D), dtype=np.uint16)
                kc = np.zeros((1, HKV, interval, D), dtype=np.uint16)
                vc = np.zeros_like(kc)
                assert orc.matmul3(xs, *w, oq, kc, vc, rope, (HKV * interval * D, interval * D, D, 1), interval, 0,
                                   interval, orc.F16, rope_position_stride=0) == 0
                gk = k[pos:pos + interval, seq].permute(1, 0, 2).contiguous()
                gv = v[pos:pos + interval, seq].permute(1, 0, 2).contiguous()
                f = lambda a: orc.from_storage(a, orc.F16)
                assert compare_ulps(to_host(gk, orc.F16), f(kc)[0], orc.F16)["ok"], (interval, seq)
                assert compare_ulps(to_host(gv, orc.F16), f(vc)[0], orc.F16)["ok"], (interval, seq)
                assert compare_ulps(to_host(dq[:, seq], orc.F16), f(oq)[:, 0], orc.F16)["ok"], (interval, seq)
        finally:
            proj.close()
