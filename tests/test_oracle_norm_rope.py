"""Pins for the oracle's key-row path (RMS norm, rotary rotation, cache write): the
reference's own known answers first, then what the mathematics fixes."""
import numpy as np
import pytest

import oracle_lib as orc

D = 128

# src/kernel/generic/rms_norm.rs:54-86: rms_norm([1..18], eps = 1e-6), checked there to 4 ulps
RMS_NORM_1_TO_18 = [
    0.09238425642251968, 0.18476851284503937, 0.27715277671813965, 0.36953702569007874,
    0.4619212746620178, 0.5543055534362793, 0.646689772605896, 0.7390740513801575,
    0.831458330154419, 0.9238425493240356, 1.0162267684936523, 1.1086111068725586,
    1.2009953260421753, 1.293379545211792, 1.3857638835906982, 1.478148102760315,
    1.5705323219299316, 1.662916660308838,
]
# src/kernel/generic/complex_mul.rs:33-49: (1+2i)^2, (3+4i)^2, ... as interleaved pairs
COMPLEX_SQUARES = [-3.0, 4.0, -7.0, 24.0, -11.0, 60.0, -15.0, 112.0, -19.0, 180.0, -23.0, 264.0,
                   -27.0, 364.0, -31.0, 480.0, -35.0, 612.0, -39.0, 760.0, -43.0, 924.0, -47.0,
                   1104.0, -51.0, 1300.0, -55.0, 1512.0, -59.0, 1740.0, -63.0, 1984.0, -67.0, 2244.0]


def _ulps(a, b):
    a = np.asarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    b = np.asarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    return np.abs(a - b).max()


def test_rms_norm_reference_literal():
    got = orc.rms_norm(np.arange(1, 19, dtype=np.float32), 1e-6)
    assert _ulps(got, np.array(RMS_NORM_1_TO_18, dtype=np.float32)) <= 4


def test_add_rms_norm_reference_literal():
    # src/kernel/generic/rms_norm.rs:88-125: ([0..17] + 1) normalised gives the same vector
    got = orc.rms_norm(np.arange(0, 18, dtype=np.float32) + np.ones(18, dtype=np.float32), 1e-6)
    assert _ulps(got, np.array(RMS_NORM_1_TO_18, dtype=np.float32)) <= 4


def test_complex_mul_reference_literal():
    x = np.arange(1, 35, dtype=np.float32)
    assert np.array_equal(orc.complex_mul(x, x), np.array(COMPLEX_SQUARES, dtype=np.float32))


def test_eps_is_added_to_the_rms_not_under_the_root():
    # rms_norm.rs:19: 1 / (sqrt(mean) + eps).  With a large eps the two readings differ widely.
    x = np.full(16, 3.0, dtype=np.float32)
    got = orc.rms_norm(x, 1.0)
    assert np.allclose(got, 3.0 / (3.0 + 1.0), rtol=1e-6)            # outside the root
    assert not np.allclose(got, 3.0 / np.sqrt(9.0 + 1.0), rtol=1e-3)  # what inside would give


def test_zero_row_stays_zero():
    assert np.array_equal(orc.rms_norm(np.zeros(D, dtype=np.float32), 1e-6), np.zeros(D, np.float32))


def test_unit_output_rms_and_scale_invariance():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(D).astype(np.float32)
    y = orc.rms_norm(x, 0.0)
    assert abs(np.sqrt(np.mean(y.astype(np.float64) ** 2)) - 1.0) < 1e-6
    assert np.allclose(orc.rms_norm(7.5 * x, 0.0), y, rtol=1e-6, atol=1e-7)


def test_rotation_keeps_pair_norms_and_composes():
    rng = np.random.default_rng(1)
    x = rng.standard_normal(D).astype(np.float32)
    th1, th2 = rng.uniform(0, 6.28, D // 2), rng.uniform(0, 6.28, D // 2)

    def table(th):
        r = np.empty(D, dtype=np.float32)
        r[0::2], r[1::2] = np.cos(th), np.sin(th)
        return r

    y = orc.complex_mul(x, table(th1))
    assert np.allclose(y[0::2] ** 2 + y[1::2] ** 2, x[0::2] ** 2 + x[1::2] ** 2, rtol=1e-5)
    both = orc.complex_mul(y, table(th2))
    assert np.allclose(both, orc.complex_mul(x, table(th1 + th2)), atol=1e-5)
    # the identity rotation (cos 1, sin 0) changes nothing, a quarter turn maps (a, b) to (-b, a)
    assert np.array_equal(orc.complex_mul(x, table(np.zeros(D // 2))), x)
    quarter = np.empty(D, dtype=np.float32)
    quarter[0::2], quarter[1::2] = 0.0, 1.0
    q = orc.complex_mul(x, quarter)
    assert np.array_equal(q[0::2], -x[1::2]) and np.array_equal(q[1::2], x[0::2])


def _reference_fixture_rows():
    """Inputs of src/kernel/x86_64/f16_512/matmul_rms_complex.rs:215-262."""
    c = np.array([[0.01 * r + 0.001 * col for col in range(D)] for r in range(3)], dtype=np.float32)
    rope = np.empty(D, dtype=np.float32)
    th = 0.01 * np.arange(D // 2, dtype=np.float32)
    rope[0::2], rope[1::2] = np.cos(th), np.sin(th)
    return c, rope


@pytest.mark.parametrize("dtype", [orc.F32, orc.F16, orc.BF16])
def test_fused_row_equals_the_two_calls(dtype):
    """matmul_rms_complex.rs:264-322 checks the fused finalize against rms_norm followed by
    complex_mul on the same rows; here the same fixture, in binary32 with one final rounding."""
    c, rope = _reference_fixture_rows()
    eps = 1e-5
    rope_s = orc.to_storage(rope, dtype)
    rope32 = orc.from_storage(rope_s, dtype)
    for r in range(3):
        row_s = orc.to_storage(c[r], dtype)
        fused = orc.norm_rope_row(row_s, rope_s, eps, dtype)
        two = orc.to_storage(orc.complex_mul(orc.rms_norm(orc.from_storage(row_s, dtype), eps), rope32), dtype)
        assert np.array_equal(np.asarray(fused).view(np.uint8), np.asarray(two).view(np.uint8))


def test_fused_row_against_float64():
    rng = np.random.default_rng(2)
    for trial in range(20):
        x = (rng.standard_normal(D) * rng.uniform(0.1, 30)).astype(np.float32)
        th = rng.uniform(0, 6.28, D // 2)
        rope = np.empty(D, dtype=np.float32)
        rope[0::2], rope[1::2] = np.cos(th), np.sin(th)
        eps = 1e-6
        got = orc.norm_rope_row(x, rope, eps, orc.F32)
        x64, r64 = x.astype(np.float64), rope.astype(np.float64)
        y = x64 / (np.sqrt(np.mean(x64 ** 2)) + eps)
        want = np.empty(D)
        want[0::2] = y[0::2] * r64[0::2] - y[1::2] * r64[1::2]
        want[1::2] = y[0::2] * r64[1::2] + y[1::2] * r64[0::2]
        assert np.allclose(got, want, rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
def test_kv_append_places_rows_at_token_coordinates(dtype):
    rng = np.random.default_rng(3)
    seqs, hkv, cap, pitch, n_tok, p0 = 3, 2, 40, 4, 5, 7
    k_cache = orc.to_storage(rng.standard_normal((seqs, hkv, cap, D)), dtype)
    v_cache = orc.to_storage(rng.standard_normal((seqs, hkv, cap, D)), dtype)
    k0, v0 = k_cache.copy(), v_cache.copy()
    k_src = orc.to_storage(rng.standard_normal((n_tok, pitch, hkv, D)), dtype)
    v_src = orc.to_storage(rng.standard_normal((n_tok, pitch, hkv, D)), dtype)
    th = rng.uniform(0, 6.28, (cap, D // 2))
    rope32 = np.empty((cap, D), dtype=np.float32)
    rope32[:, 0::2], rope32[:, 1::2] = np.cos(th), np.sin(th)
    rope = orc.to_storage(rope32, dtype)
    assert orc.kv_append_norm_rope(k_cache, v_cache, p0, k_src, v_src, rope, 1e-6, dtype,
                                   batch_size=seqs) == 0
    for b in range(seqs):
        for h in range(hkv):
            for t in range(n_tok):
                want = orc.norm_rope_row(k_src[t, b, h], rope[p0 + t], 1e-6, dtype)
                assert np.array_equal(k_cache[b, h, p0 + t], want)
                assert np.array_equal(v_cache[b, h, p0 + t], v_src[t, b, h])
    # nothing else moved, and the unused source column (pitch > batch) was never read into the cache
    mask = np.ones((seqs, hkv, cap), dtype=bool)
    mask[:, :, p0:p0 + n_tok] = False
    assert np.array_equal(k_cache[mask], k0[mask]) and np.array_equal(v_cache[mask], v0[mask])


def test_kv_append_per_sequence_positions_and_bounds():
    dtype = orc.F16
    rng = np.random.default_rng(4)
    seqs, hkv, cap = 3, 1, 16
    k_cache = np.zeros((seqs, hkv, cap, D), dtype=np.float16)
    v_cache = np.zeros_like(k_cache)
    k_src = orc.to_storage(rng.standard_normal((1, seqs, hkv, D)), dtype)
    v_src = orc.to_storage(rng.standard_normal((1, seqs, hkv, D)), dtype)
    rope32 = np.zeros((cap, D), dtype=np.float32)
    rope32[:, 0::2] = 1.0                      # identity rotation
    rope = orc.to_storage(rope32, dtype)
    positions = [0, 9, 15]
    assert orc.kv_append_norm_rope(k_cache, v_cache, 99, k_src, v_src, rope, 1e-6, dtype,
                                   positions=positions) == 0
    for b, p in enumerate(positions):
        assert np.array_equal(v_cache[b, 0, p], v_src[0, b, 0])
        assert np.array_equal(k_cache[b, 0, p], orc.norm_rope_row(k_src[0, b, 0], rope[p], 1e-6, dtype))
        assert np.count_nonzero(v_cache[b]) == np.count_nonzero(v_src[0, b, 0])
    # one position past the end: refused, nothing written
    before = k_cache.copy()
    assert orc.kv_append_norm_rope(k_cache, v_cache, 0, k_src, v_src, rope, 1e-6, dtype,
                                   positions=[0, 9, 16]) == 1
    assert np.array_equal(k_cache, before)
