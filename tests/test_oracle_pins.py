"""Pins for the CPU oracle (oracle/ellm_oracle.cpp).

The reference cannot be compiled here (nightly Rust), so the oracle is pinned by
(1) every known answer the reference's own tests hold for this path, (2) closed
forms and invariants of causal soft-max attention, (3) a float64 brute force and
torch's scaled_dot_product_attention, neither of which shares code with it.
"""
import os

import numpy as np
import pytest

import oracle_lib as orc

D = 128


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# ---- known answers held by the reference's tests --------------------------------

def test_dot_product_literals():
    lib = orc.load()
    # src/kernel/generic/flash_attention.rs:95-101 -> 32
    a, b = _f32([1, 2, 3]), _f32([4, 5, 6])
    assert lib.ellm_oracle_dot_product_f32(a.ctypes.data, b.ctypes.data, 3) == 32.0
    # src/kernel/x86_64/f16_512/dot_product.rs:49-57 -> 128
    a = b = _f32(np.ones(128))
    assert lib.ellm_oracle_dot_product_f32(a.ctypes.data, b.ctypes.data, 128) == 128.0
    # src/kernel/generic/dot_product.rs:22-29 -> 38
    a, b = _f32(np.ones(19)), _f32(np.full(19, 2.0))
    assert lib.ellm_oracle_dot_product_f32(a.ctypes.data, b.ctypes.data, 19) == 38.0


def test_scalar_vector_mul_and_acc_literal():
    # src/kernel/generic/flash_attention.rs:103-116: 1*1 + 2*2 = 5, 128 wide
    lib = orc.load()
    o, v = _f32(np.ones(128)), _f32(np.full(128, 2.0))
    lib.ellm_oracle_scalar_vector_mul_and_acc_f32(1.0, o.ctypes.data, 2.0, v.ctypes.data, 128)
    assert np.all(o == 5.0)


@pytest.mark.parametrize("dtype,prefill", [(orc.F32, 1.0), (orc.F16, 0.0), (orc.BF16, 3.0)])
def test_all_ones_known_answer(dtype, prefill):
    # src/kernel/generic/flash_attention.rs:119-147 (o pre-filled with 1) and
    # src/kernel/x86_64/f16_512/flash_attention.rs:135-157 (o pre-filled with 0):
    # q = K = V = 1, 8 rows, scale 1, position 7 -> o == 1 to 1e-6
    q = orc.to_storage(np.ones(D), dtype)
    K = orc.to_storage(np.ones((8, D)), dtype)
    V = orc.to_storage(np.ones((8, D)), dtype)
    o_init = orc.to_storage(np.full(D, prefill), dtype)
    o, lse = orc.flash_attention_row(q, K, V, 1.0, 7, dtype, o_init=o_init)
    assert np.abs(orc.from_storage(o, dtype) - 1.0).max() < 1e-6
    assert abs(lse - (128.0 + np.log(8.0))) < 1e-4


def test_scale_softmax_literal():
    # src/kernel/test.rs:605-629: softmax(0.65 * [1..18]), 4 ulps
    want = np.array([
        7.5933926382276695e-06, 1.4545462363457773e-05, 2.7862415663548745e-05,
        5.337157563189976e-05, 0.00010223548451904207, 0.00019583618268370628,
        0.0003751322510652244, 0.0007185811409726739, 0.0013764717150479555,
        0.0026366880629211664, 0.005050681531429291, 0.009674787521362305,
        0.01853245310485363, 0.035499654710292816, 0.06800107657909393,
        0.13025879859924316, 0.24951595067977905, 0.4779582619667053], dtype=np.float32)
    x = _f32(np.arange(1, 19))
    out = np.zeros(18, dtype=np.float32)
    orc.load().ellm_oracle_scale_softmax_f32(x.ctypes.data, out.ctypes.data, 18, 0.65)
    ulps = np.abs(out.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
    assert ulps.max() <= 4
    # the attention row with these scores gives the same weights: V = identity rows
    q = np.zeros(D, dtype=np.float32)
    q[0] = 1.0
    K = np.zeros((18, D), dtype=np.float32)
    K[:, 0] = np.arange(1, 19)
    V = np.zeros((18, D), dtype=np.float32)
    V[np.arange(18), np.arange(18)] = 1.0
    o, _ = orc.flash_attention_row(q, K, V, 0.65, 17, orc.F32)
    assert np.allclose(o[:18], want, rtol=2e-6, atol=1e-9)
    # this is what separates "softmax(scale*x)" from the generic kernel's defect
    # (unscaled score in one exponent, src/kernel/generic/flash_attention.rs:76)
    wrong = np.exp(x - 0.65 * x.max())
    assert not np.allclose(o[:18], wrong / wrong.sum(), rtol=1e-3)


def test_assign_literals():
    # src/compiler/assign.rs:141-190
    assert orc.assign(5, 8, 5) is None
    assert orc.assign(5, 8, 4) == (4, 5)
    assert [orc.assign(10, 3, i) for i in range(3)] == [(0, 4), (4, 7), (7, 10)]
    assert [orc.assign(11, 3, i) for i in range(3)] == [(0, 4), (4, 8), (8, 11)]
    assert [orc.assign(12, 3, i) for i in range(3)] == [(0, 4), (4, 8), (8, 12)]


@pytest.mark.parametrize("length,num", [(1, 1), (7, 3), (100, 8), (3, 8), (513, 16)])
def test_assign_is_a_partition(length, num):
    parts = [orc.assign(length, num, i) for i in range(num)]
    covered = []
    for p in parts:
        if p is not None:
            covered.extend(range(*p))
    assert covered == list(range(length))
    sizes = [p[1] - p[0] for p in parts if p is not None]
    assert max(sizes) - min(sizes) <= 1


def test_barrier():
    # src/runtime/barrier.rs:57-83 in spirit: phases never mix
    assert orc.load().ellm_oracle_barrier_selftest(4, 200) == 0


# ---- storage conversions ------------------------------------------------------------

def test_f16_conversions_match_numpy():
    lib = orc.load()
    bits = np.arange(0, 65536, dtype=np.uint32)
    ours = np.array([lib.ellm_oracle_f16_to_f32(int(b)) for b in bits[::7]], dtype=np.float32)
    ref = bits[::7].astype(np.uint16).view(np.float16).astype(np.float32)
    assert np.array_equal(np.isnan(ours), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(ours[ok], ref[ok])
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(3000) * 10.0 ** rng.integers(-9, 6, 3000),
                        [0.0, -0.0, 65504.0, 65520.0, 65519.9, 6e-8, 2.98e-8, 2.9802322e-8, 1e-10,
                         np.inf, -np.inf, 0.00006103515625, 6.1e-5]]).astype(np.float32)
    for v in x:
        got = lib.ellm_oracle_f32_to_f16(float(v))
        with np.errstate(over="ignore"):
            want = int(np.float32(v).astype(np.float16).view(np.uint16))
        assert got == want, (v, hex(got), hex(want))


def test_bf16_conversions():
    lib = orc.load()
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(2000) * 10.0 ** rng.integers(-20, 20, 2000)).astype(np.float32)
    want = orc.to_storage(x, orc.BF16)
    for v, w in zip(x, want):
        assert lib.ellm_oracle_f32_to_bf16(float(v)) == int(w)
        assert lib.ellm_oracle_bf16_to_f32(int(w)) == orc.from_storage(np.array([w], np.uint16), orc.BF16)[0]


# ---- closed forms ------------------------------------------------------------------

def _rand(shape, seed, dtype=orc.F32):
    return orc.to_storage(np.random.default_rng(seed).standard_normal(shape), dtype)


def test_position_zero_returns_first_value_row():
    q, K, V = _rand(D, 1), _rand((4, D), 2), _rand((4, D), 3)
    o, lse = orc.flash_attention_row(q, K, V, 0.3, 0, orc.F32)
    assert np.array_equal(o, V[0])
    assert abs(lse - 0.3 * float(q @ K[0])) < 1e-5


def test_equal_scores_give_the_mean():
    K, V = _rand((9, D), 4), _rand((9, D), 5)
    q = np.zeros(D, dtype=np.float32)
    for p in (0, 3, 8):
        o, lse = orc.flash_attention_row(q, K, V, 1.0, p, orc.F32)
        assert np.allclose(o, V[:p + 1].mean(0), atol=1e-6)
        assert abs(lse - np.log(p + 1.0)) < 1e-6


def test_constant_values_pass_through():
    q, K = _rand(D, 6), _rand((20, D), 7)
    V = np.full((20, D), 0.375, dtype=np.float32)
    o, _ = orc.flash_attention_row(q, K, V, 0.2, 19, orc.F32)
    assert np.allclose(o, 0.375, atol=1e-6)


def test_dominant_key_selects_its_value():
    q = np.zeros(D, dtype=np.float32)
    q[3] = 1.0
    K, V = _rand((12, D), 8) * 0.1, _rand((12, D), 9)
    K[7, 3] = 40.0
    o, _ = orc.flash_attention_row(q, _f32(K), V, 1.0, 11, orc.F32)
    assert np.allclose(o, V[7], atol=1e-5)


def test_shift_invariance():
    q, K, V = _rand(D, 10), _rand((15, D), 11), _rand((15, D), 12)
    scale, c = 0.25, 3.0
    o1, lse1 = orc.flash_attention_row(q, K, V, scale, 14, orc.F32)
    shift = (c / float(q @ q)) * q          # q.(K + shift) = q.K + c for every key
    o2, lse2 = orc.flash_attention_row(q, _f32(K + shift), V, scale, 14, orc.F32)
    assert np.allclose(o1, o2, atol=2e-5)
    assert abs((lse2 - lse1) - scale * c) < 2e-5


def test_future_rows_and_old_output_do_not_leak():
    q, K, V = _rand(D, 13), _rand((10, D), 14), _rand((10, D), 15)
    base, lse0 = orc.flash_attention_row(q, K, V, 0.2, 5, orc.F32)
    K2, V2 = K.copy(), V.copy()
    K2[6:], V2[6:] = np.nan, np.inf
    o, lse = orc.flash_attention_row(q, K2, V2, 0.2, 5, orc.F32,
                                     o_init=np.full(D, np.nan, dtype=np.float32))
    assert np.array_equal(o, base) and lse == lse0


# ---- the operator: index arithmetic, GQA, chunks, threads ------------------------------

def _brute(q, k, v, scale, p0, positions=None):
    """float64 two-pass soft-max; q [S,B,Hq,D], k/v [B,Hkv,cap,D] as binary32."""
    S, B, Hq, _ = q.shape
    G = Hq // k.shape[1]
    out = np.zeros(q.shape)
    lse = np.zeros((S, B, Hq))
    for t in range(S):
        for b in range(B):
            n = (int(positions[b]) if positions is not None else p0 + t) + 1
            for h in range(Hq):
                s = (k[b, h // G, :n].astype(np.float64) @ q[t, b, h].astype(np.float64)) * scale
                e = np.exp(s - s.max())
                out[t, b, h] = (e / e.sum()) @ v[b, h // G, :n].astype(np.float64)
                lse[t, b, h] = s.max() + np.log(e.sum())
    return out, lse


@pytest.mark.parametrize("hq,hkv", [(1, 1), (4, 4), (4, 2), (8, 2), (6, 1), (6, 3)])
@pytest.mark.parametrize("dtype", [orc.F32, orc.F16, orc.BF16])
def test_operator_matches_float64_brute_force(hq, hkv, dtype):
    S, B, cap, p0 = 6, 2, 20, 5
    q = _rand((S, B, hq, D), 20 + hq, dtype)
    k = _rand((B, hkv, cap, D), 21 + hkv, dtype)
    v = _rand((B, hkv, cap, D), 22, dtype)
    scale = 1.0 / np.sqrt(D)
    out, lse = orc.attention(q, k, v, scale, dtype, position_index=p0, n_threads=3)
    want, want_lse = _brute(orc.from_storage(q, dtype), orc.from_storage(k, dtype),
                            orc.from_storage(v, dtype), scale, p0)
    tol = {orc.F32: 2e-6, orc.F16: 1e-3, orc.BF16: 8e-3}[dtype]
    assert np.abs(orc.from_storage(out, dtype) - want).max() <= tol
    assert np.abs(lse - want_lse).max() <= 2e-5


def test_gqa_heads_with_identical_queries_agree():
    S, B, hq, hkv, cap = 3, 1, 8, 2, 12
    q = _rand((S, B, hq, D), 30)
    q[:, :, 1:4] = q[:, :, 0:1]     # heads 0..3 share kv head 0
    k, v = _rand((B, hkv, cap, D), 31), _rand((B, hkv, cap, D), 32)
    out, _ = orc.attention(q, k, v, 0.1, orc.F32, position_index=2)
    for h in range(1, 4):
        assert np.array_equal(out[:, :, h], out[:, :, 0])
    q2 = q.copy()
    q2[:, :, 4] = q[:, :, 0]        # head 4 reads kv head 1: must differ
    out2, _ = orc.attention(q2, k, v, 0.1, orc.F32, position_index=2)
    assert not np.allclose(out2[:, :, 4], out2[:, :, 0])


def test_batch_capacity_pitch_and_reference_kv_strides():
    """Q/O rows are pitched by the capacity, not the live batch
    (src/compiler/mul/attention.rs:86, 118-119); K/V may be the reference's
    permuted view of [position][sequence][kv_head][D] (src/qwen3_moe/attention.rs:149-166)."""
    S, bcap, B, hq, hkv, cap, p0 = 4, 3, 2, 4, 2, 10, 3
    q = _rand((S, bcap, hq, D), 40)
    kphys = _rand((cap, bcap, hkv, D), 41)          # [position][sequence][kv_head][D]
    vphys = _rand((cap, bcap, hkv, D), 42)
    out = np.full_like(q, 123.0)
    lse = np.zeros((S, bcap, hq), dtype=np.float32)
    strides = [hkv * D, D, bcap * hkv * D, 1]      # sequence, kv head, position, 1
    op = orc.Operator(q, kphys, vphys, out, lse, bcap, hq, hkv, D, strides, 0.2, orc.F32)
    op.run(p0, S, B)
    k = np.ascontiguousarray(kphys.transpose(1, 2, 0, 3))
    v = np.ascontiguousarray(vphys.transpose(1, 2, 0, 3))
    want, _ = _brute(q, k, v, 0.2, p0)
    assert np.abs(out[:, :B] - want[:, :B]).max() < 2e-6
    assert np.all(out[:, B:] == 123.0)              # rows beyond the live batch untouched


def test_thread_partition_is_exact():
    """Calling run for thread ids 0..n-1 one after the other (the way the reference tests
    multi-threading, e.g. src/compiler/operator.rs:290-298) equals one thread, bit for bit."""
    S, B, hq, hkv, cap = 5, 2, 4, 2, 9
    q, k, v = _rand((S, B, hq, D), 50), _rand((B, hkv, cap, D), 51), _rand((B, hkv, cap, D), 52)
    strides = [hkv * cap * D, cap * D, D, 1]
    one = np.zeros_like(q)
    orc.Operator(q, k, v, one, None, B, hq, hkv, D, strides, 0.3, orc.F32).run(4, S, B)
    for n in (2, 3, 7, 64):
        many = np.zeros_like(q)
        op = orc.Operator(q, k, v, many, None, B, hq, hkv, D, strides, 0.3, orc.F32)
        for tid in range(n):
            op.run(4, S, B, cpu_num=n, thread_id=tid)
        assert np.array_equal(one, many)
    threaded = np.zeros_like(q)
    orc.Operator(q, k, v, threaded, None, B, hq, hkv, D, strides, 0.3, orc.F32).run_threads(
        4, S, B, 4)
    assert np.array_equal(one, threaded)


def test_chunk_invariance():
    """One pass, chunks (src/serving/'start copy.rs':86-98) and token-by-token steps give
    the same rows, bit for bit (each row only depends on its own position)."""
    S, B, hq, hkv, cap = 12, 2, 4, 2, 16
    q, k, v = _rand((S, B, hq, D), 60), _rand((B, hkv, cap, D), 61), _rand((B, hkv, cap, D), 62)
    strides = [hkv * cap * D, cap * D, D, 1]
    whole, _ = orc.attention(q, k, v, 0.2, orc.F32, position_index=3)
    for chunk in (1, 5, 12):
        got = np.zeros_like(q)
        for t0 in range(0, S, chunk):
            n = min(chunk, S - t0)
            qs, os_ = q[t0:t0 + n], got[t0:t0 + n]      # contiguous views
            orc.Operator(qs, k, v, os_, None, B, hq, hkv, D, strides, 0.2, orc.F32).run(
                3 + t0, n, B)
        assert np.array_equal(got, whole)


def test_ragged_positions():
    B, hq, hkv, cap = 3, 4, 2, 30
    q, k, v = _rand((1, B, hq, D), 70), _rand((B, hkv, cap, D), 71), _rand((B, hkv, cap, D), 72)
    pos = np.array([0, 29, 11], dtype=np.uint32)
    out, lse = orc.attention(q, k, v, 0.15, orc.F32, positions=pos)
    want, want_lse = _brute(q, k, v, 0.15, 0, positions=pos)
    assert np.abs(out - want).max() < 2e-6 and np.abs(lse - want_lse).max() < 1e-5


def test_selected_rows_equal_the_full_run():
    S, B, hq, hkv, cap = 6, 2, 4, 2, 12
    q, k, v = _rand((S, B, hq, D), 80), _rand((B, hkv, cap, D), 81), _rand((B, hkv, cap, D), 82)
    whole, lse = orc.attention(q, k, v, 0.2, orc.F32, position_index=5)
    op = orc.Operator(q, k, v, np.zeros_like(q), None, B, hq, hkv, D,
                      [hkv * cap * D, cap * D, D, 1], 0.2, orc.F32)
    rows = np.array([[0, 0, 0], [5, 1, 3], [2, 0, 2], [3, 1, 1]], dtype=np.uint32)
    got, got_lse, _ = op.run_rows(5, rows, 2)
    for i, (t, b, h) in enumerate(rows):
        assert np.array_equal(got[i], whole[t, b, h]) and got_lse[i] == lse[t, b, h]


def test_selected_rows_with_per_sequence_positions_and_pinned_threads_equal_the_full_run():
    B, hq, hkv, cap = 3, 4, 2, 20
    q, k, v = _rand((1, B, hq, D), 83), _rand((B, hkv, cap, D), 84), _rand((B, hkv, cap, D), 85)
    pos = np.array([3, 19, 11], dtype=np.uint32)
    whole, lse = orc.attention(q, k, v, 0.2, orc.F32, positions=pos)
    op = orc.Operator(q, k, v, np.zeros_like(q), None, B, hq, hkv, D,
                      [hkv * cap * D, cap * D, D, 1], 0.2, orc.F32)
    rows = np.array([[0, b, h] for b in range(B) for h in (0, 3)], dtype=np.uint32)
    got, got_lse, _ = op.run_rows(0, rows, 3, positions=pos, pin=True)
    for i, (t, b, h) in enumerate(rows):
        assert np.array_equal(got[i], whole[t, b, h]) and got_lse[i] == lse[t, b, h]


# ---- independent library and committed vectors -------------------------------------------

def test_matches_torch_sdpa():
    torch = pytest.importorskip("torch")
    S, B, hq, hkv, cap, p0 = 8, 2, 8, 2, 24, 16
    q, k, v = _rand((S, B, hq, D), 90), _rand((B, hkv, cap, D), 91), _rand((B, hkv, cap, D), 92)
    out, _ = orc.attention(q, k, v, 0.11, orc.F32, position_index=p0)
    tq = torch.from_numpy(q).permute(1, 2, 0, 3)                    # [B, Hq, S, D]
    tk, tv = torch.from_numpy(k)[:, :, :p0 + S], torch.from_numpy(v)[:, :, :p0 + S]
    mask = torch.arange(p0 + S)[None, :] <= (p0 + torch.arange(S))[:, None]
    ref = torch.nn.functional.scaled_dot_product_attention(
        tq, tk, tv, attn_mask=mask, scale=0.11, enable_gqa=True)
    assert np.abs(out - ref.permute(2, 0, 1, 3).numpy()).max() < 5e-6


@pytest.mark.parametrize("name", ["mha", "gqa", "mqa_decode"])
@pytest.mark.parametrize("dtype", [orc.F16, orc.F32])
def test_golden_vectors(name, dtype):
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_small.npz")
    z = np.load(path)
    q, k, v = z[name + "_q"], z[name + "_k"], z[name + "_v"]
    if dtype == orc.F32:
        q, k, v = (a.astype(np.float32) for a in (q, k, v))
    out, lse = orc.attention(q, k, v, 1.0 / np.sqrt(D), dtype, position_index=int(z[name + "_p0"]))
    tol = 1e-3 if dtype == orc.F16 else 3e-6
    assert np.abs(orc.from_storage(out, dtype) - z[name + "_out"]).max() <= tol
    assert np.abs(lse - z[name + "_lse"]).max() <= 2e-5
