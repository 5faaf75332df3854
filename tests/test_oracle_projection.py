"""Pins for the oracle's projections (MatMul3, MatMulAdd): the input formulas of the
reference's own tests against an independent float64 product, and what the mathematics
fixes (identity weights, linearity, the finalize built from the separately pinned
rms_norm and complex_mul, placement through the strides)."""
import numpy as np
import pytest

import oracle_lib as orc

D = 128


def _f64(a, dtype):
    return orc.from_storage(a, dtype).astype(np.float64)


def _reference_test_inputs(batch, hidden, q_dim, kv_dim):
    """Input and weight formulas of test_matmul3_f16, src/ptensor/tensor.rs:1132-1163."""
    x = np.array([[((i * 7 + k * 3) % 19) * 0.01 for k in range(hidden)] for i in range(batch)], dtype=np.float32)
    wq = np.array([[((k * 5 + n * 11) % 23) * 0.01 for k in range(hidden)] for n in range(q_dim)], dtype=np.float32)
    wk = np.array([[((k * 3 + n * 7) % 29) * 0.01 for k in range(hidden)] for n in range(kv_dim)], dtype=np.float32)
    wv = np.array([[((k * 9 + n * 4) % 31) * 0.01 for k in range(hidden)] for n in range(kv_dim)], dtype=np.float32)
    return x, wq, wk, wv


def test_product_on_the_reference_test_inputs_equals_float64():
    # tensor.rs:1089-1094: batch 3, hidden 64, q_dim = kv_dim = 96; its check is |out - f32 sum| < 0.5
    x, wq, wk, wv = _reference_test_inputs(3, 64, 96, 96)
    for dtype in (orc.F16, orc.F32):
        xs = orc.to_storage(x, dtype)
        for w in (wq, wk, wv):
            ws = orc.to_storage(w, dtype)
            got = orc.matmul_nt(xs, ws, dtype)
            want = _f64(xs, dtype) @ _f64(ws, dtype).T
            assert np.abs(got - want).max() <= 4e-6 * np.abs(want).max()
            assert np.abs(got - want).max() < 0.5                      # the reference's own bound


def test_matmul3_f32_72_rows_inputs():
    # src/compiler/mul/matmul3.rs:620-700: m 72, k 256, 32 + 4 + 4 heads, rope all ones
    m, k, hq, hkv = 72, 256, 4, 2        # fewer heads than the reference's 32 / 4: same formulas, CPU seconds
    a = (np.arange(m * k) % 100).astype(np.float32).reshape(m, k) * 0.01

    def w_nt(n):
        jj, kk = np.meshgrid(np.arange(n), np.arange(k), indexing="ij")
        return (((kk * n + jj + 1) % 7) * 0.01).astype(np.float32)

    wq, wk, wv = w_nt(hq * D), w_nt(hkv * D), w_nt(hkv * D)
    rope = np.ones(max(hq, hkv) * D, dtype=np.float32)
    q = np.zeros((1, m, hq, D), dtype=np.float32)
    kst = np.zeros((1, m, hkv, D), dtype=np.float32)
    vst = np.zeros_like(kst)
    strides = (hkv * D, D, m * hkv * D, 1)       # the reference's [position][sequence][head][128] state
    # the reference indexes the table by output column: position stride 0, head stride 128
    assert orc.matmul3(a[None], wq, wk, wv, q, kst, vst, rope, strides, 1, 0, 1, orc.F32,
                       rope_position_stride=0, rope_head_stride=D) == 0

    def post(c, heads):                           # ref_post_process_f32, matmul3.rs:533-546, in float64
        c = c.reshape(m, heads, D)
        y = c / (np.sqrt((c * c).mean(-1, keepdims=True)) + 1e-6)
        out = np.empty_like(y)
        out[..., 0::2] = y[..., 0::2] - y[..., 1::2]       # (a + ib)(1 + i)
        out[..., 1::2] = y[..., 0::2] + y[..., 1::2]
        return out

    a64 = a.astype(np.float64)
    assert np.abs(q[0] - post(a64 @ wq.astype(np.float64).T, hq)).max() < 2e-5      # reference: 1e-3
    assert np.abs(kst[0] - post(a64 @ wk.astype(np.float64).T, hkv)).max() < 2e-5
    assert np.abs(vst[0].reshape(m, -1) - a64 @ wv.astype(np.float64).T).max() < 2e-4


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16, orc.F32])
def test_identity_weights_return_the_finalized_input(dtype):
    rng = np.random.default_rng(3)
    interval, pitch, hq, hkv, cap, p0 = 3, 2, 1, 1, 16, 5
    k = D
    hidden = orc.to_storage(rng.standard_normal((interval, pitch, k), dtype=np.float32), dtype)
    eye = orc.to_storage(np.eye(D, dtype=np.float32), dtype)
    ang = rng.uniform(0, 6.28, size=(cap, D // 2))
    table = np.empty((cap, D), dtype=np.float32)
    table[:, 0::2], table[:, 1::2] = np.cos(ang), np.sin(ang)
    rope = orc.to_storage(table, dtype)
    q = np.zeros((interval, pitch, hq, D), dtype=hidden.dtype)
    kc = np.zeros((pitch, hkv, cap, D), dtype=hidden.dtype)
    vc = np.zeros_like(kc)
    assert orc.matmul3(hidden, eye, eye, eye, q, kc, vc, rope, (hkv * cap * D, cap * D, D, 1), cap,
                       p0, interval, dtype) == 0
    for t in range(interval):
        for b in range(pitch):
            want = orc.norm_rope_row(hidden[t, b], rope[p0 + t], 1e-6, dtype)   # pinned separately
            assert np.array_equal(q[t, b, 0], want)
            assert np.array_equal(kc[b, 0, p0 + t], want)
            assert np.array_equal(vc[b, 0, p0 + t], hidden[t, b])
    # nothing else was written
    mask = np.ones(kc.shape[:3], dtype=bool)
    mask[:, :, p0:p0 + interval] = False
    assert not kc[mask].any() and not vc[mask].any()


def test_linearity_and_value_heads_are_plain_products():
    rng = np.random.default_rng(4)
    k, hq, hkv, cap = 64, 1, 2, 8
    x1 = rng.standard_normal((1, 3, k), dtype=np.float32)
    x2 = rng.standard_normal((1, 3, k), dtype=np.float32)
    w = [rng.standard_normal((h * D, k), dtype=np.float32) for h in (hq, hkv, hkv)]
    rope = np.zeros((cap, D), dtype=np.float32)
    rope[:, 0::2] = 1.0
    outs = []
    for x in (x1, x2, x1 + 2 * x2):
        q = np.zeros((1, 3, hq, D), dtype=np.float32)
        kc = np.zeros((3, hkv, cap, D), dtype=np.float32)
        vc = np.zeros_like(kc)
        assert orc.matmul3(x, *w, q, kc, vc, rope, (hkv * cap * D, cap * D, D, 1), cap, 2, 1, orc.F32) == 0
        outs.append((q, kc, vc))
    v1, v2, v3 = (o[2][:, :, 2] for o in outs)
    assert np.allclose(v3, v1 + 2 * v2, rtol=0, atol=1e-4)
    assert np.allclose(v1.reshape(3, -1), x1[0].astype(np.float64) @ w[2].astype(np.float64).T, atol=1e-4)
    # normalised heads are scale invariant, not linear: q(3 x) == q(x)
    q3 = np.zeros((1, 3, hq, D), dtype=np.float32)
    kc = np.zeros((3, hkv, cap, D), dtype=np.float32)
    assert orc.matmul3(3 * x1, *w, q3, kc, np.zeros_like(kc), rope, (hkv * cap * D, cap * D, D, 1), cap, 2, 1,
                       orc.F32) == 0
    assert np.allclose(q3, outs[0][0], atol=2e-6)
    assert np.allclose((outs[0][0] ** 2).mean(-1), 1.0, atol=1e-4)       # unit RMS after the norm


def test_ragged_positions_strides_and_bounds():
    rng = np.random.default_rng(5)
    k, hq, hkv, cap, pitch = 64, 2, 1, 12, 4
    hidden = orc.to_storage(rng.standard_normal((1, pitch, k), dtype=np.float32), orc.F16)
    w = [orc.to_storage(rng.standard_normal((h * D, k), dtype=np.float32) / 8, orc.F16) for h in (hq, hkv, hkv)]
    rope = orc.to_storage(rng.standard_normal((cap, D), dtype=np.float32), orc.F16)
    pos = np.array([3, 0, 11, 7], dtype=np.uint32)
    strides = (hkv * cap * D, cap * D, D, 1)

    def run(positions, batch):
        q = np.zeros((1, pitch, hq, D), dtype=np.uint16)
        kc = np.zeros((pitch, hkv, cap, D), dtype=np.uint16)
        vc = np.zeros_like(kc)
        rc = orc.matmul3(hidden, *w, q, kc, vc, rope, strides, cap, 0, 1, orc.F16, batch_size=batch,
                         positions=positions)
        return rc, q, kc, vc

    rc, q, kc, vc = run(pos, 3)
    assert rc == 0
    for b in range(3):
        one = np.zeros((1, pitch, hq, D), dtype=np.uint16)
        k1 = np.zeros_like(kc)
        assert orc.matmul3(hidden, *w, one, k1, np.zeros_like(k1), rope, strides, cap, int(pos[b]), 1, orc.F16) == 0
        assert np.array_equal(q[0, b], one[0, b]) and np.array_equal(kc[b, 0, pos[b]], k1[b, 0, pos[b]])
    assert not q[0, 3].any() and not kc[3].any()                            # sequence 3 is not live
    assert run(np.array([3, 0, 12, 7], dtype=np.uint32), 3)[0] == 1          # position 12 of 12


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16, orc.F32])
def test_matmul_add_is_residual_plus_product(dtype):
    rng = np.random.default_rng(6)
    interval, pitch, k, n = 2, 3, 96, 256
    a = orc.to_storage(rng.standard_normal((interval, pitch, k), dtype=np.float32), dtype)
    w = orc.to_storage(rng.standard_normal((n, k), dtype=np.float32) / 8, dtype)
    r = orc.to_storage(rng.standard_normal((interval, pitch, n), dtype=np.float32), dtype)
    out = orc.matmul_add(a, w, r, dtype, batch_size=2)
    want = _f64(r, dtype) + _f64(a, dtype) @ _f64(w, dtype).T
    got = _f64(out, dtype)
    tol = {orc.F16: 2e-3, orc.BF16: 1.6e-2, orc.F32: 1e-5}[dtype] * max(1.0, np.abs(want).max())
    assert np.abs(got[:, :2] - want[:, :2]).max() <= tol
    assert not out[:, 2].any()                                               # beyond batch_size: untouched
    zero = orc.to_storage(np.zeros((n, k), dtype=np.float32), dtype)
    assert np.array_equal(orc.matmul_add(a, zero, r, dtype), r)               # zero weights: the residual
