"""Seeded sweep of chunk attention shapes against the CPU oracle through the C ABI: head layouts,
batch below capacity, chunk lengths either side of the kernels' row limits (128 / 256 / 384 query
rows per K/V plane), cached lengths on and off tile edges.  The shapes are drawn so that the
planner splits the key range evenly, unevenly and not at all.  Below them: single-token steps over
sequences of different lengths, and uniform single-token steps over the split plans (one or two
workgroups per compute unit, one to hundreds of splits per plane, one and two fold levels)."""
import numpy as np
import pytest

import oracle_lib as orc
from gpu_util import D, LSE_TOL, compare, gpu_attention, rand_storage

pytestmark = pytest.mark.gpu

INTERVALS = [2, 3, 7, 15, 16, 17, 24, 31, 32, 33, 40, 47, 48, 49, 64, 100]
CACHED = [0, 5, 63, 64, 500, 1000, 1023, 1024, 2047, 3000, 5000]


def _draw(rng):
    hkv = int(rng.choice([1, 2, 4]))
    g = int(rng.choice([1, 2, 3, 4, 8, 16]))
    bcap = int(rng.choice([1, 2, 3, 6, 12, 24]))
    b = int(rng.integers(max(1, bcap - 2), bcap + 1))
    s = int(rng.choice(INTERVALS))
    p0 = int(rng.choice(CACHED))
    # keep the oracle's work (rows x keys) and the cache size small
    while b * hkv * g * s * (p0 + s) > 6e7 or bcap * hkv * (p0 + s) * D > 3e7:
        if p0 > 1000:
            p0 = 1000
        elif bcap > 2:
            bcap = b = 2
        else:
            s = 16
    cap = p0 + s + int(rng.integers(0, 5))
    return dict(hq=hkv * g, hkv=hkv, bcap=bcap, b=b, s=s, p0=p0, cap=cap)


@pytest.mark.parametrize("block", range(6))
def test_random_chunk_shapes_match_oracle(block):
    rng = np.random.default_rng(1000 + block)
    for n in range(8):
        c = _draw(rng)
        dtype = orc.F16 if (n + block) % 2 else orc.BF16
        print("case", block, n, c, "f16" if dtype == orc.F16 else "bf16", flush=True)
        q = rand_storage((c["s"], c["bcap"], c["hq"], D), 7000 + 10 * block + n, dtype)
        k = rand_storage((c["bcap"], c["hkv"], c["cap"], D), 8000 + 10 * block + n, dtype)
        v = rand_storage((c["bcap"], c["hkv"], c["cap"], D), 9000 + 10 * block + n, dtype)
        scale = 1.0 / np.sqrt(D)
        want, want_lse = orc.attention(q, k, v, scale, dtype, position_index=c["p0"], batch=c["b"])
        got, got_lse = gpu_attention(q, k, v, scale, dtype, position_index=c["p0"], batch=c["b"])
        res = compare(got[:, :c["b"]], orc.from_storage(want, dtype)[:, :c["b"]], dtype)
        lse_err = float(np.abs(got_lse[:, :c["b"]] - want_lse[:, :c["b"]]).max())
        assert res["ok"], (c, res)
        assert lse_err <= LSE_TOL, (c, lse_err)


def _draw_ragged(rng):
    hkv = int(rng.choice([1, 2, 4, 8]))
    g = int(rng.choice([1, 2, 3, 4, 8, 16, 32]))
    b = int(rng.choice([1, 5, 16, 33, 64, 65, 130, 300]))
    cap = int(rng.choice([300, 2500, 8192, 20000, 50000]))
    # cache size and the oracle's work bounded
    while b * hkv * cap * D * 2 > 2.5e8 or b * hkv * g * cap > 5e7:
        if b > 16:
            b //= 2
        elif cap > 1024:
            cap //= 2
        else:
            g = max(1, g // 2)
    kind = int(rng.integers(0, 4))
    if kind == 0:
        pos = rng.integers(0, cap, size=b)
    elif kind == 1:                                  # one long, the rest short
        pos = rng.integers(0, min(cap, 200), size=b)
        pos[int(rng.integers(0, b))] = cap - 1
    elif kind == 2:                                  # all equal
        pos = np.full(b, int(rng.integers(0, cap)))
    else:                                            # around the 64-key unit
        pos = rng.choice([0, 62, 63, 64, 65, 127, 128, cap - 1, cap - 2], size=b)
    return dict(hq=hkv * g, hkv=hkv, b=b, cap=cap, pos=np.minimum(pos, cap - 1).astype(np.uint32))


@pytest.mark.parametrize("block", range(3))
def test_random_ragged_single_token_steps_match_oracle(block):
    """Per-sequence positions: small calls keep the kernel that splits every plane alike, large ones
    take the kernel that deals the keys evenly; both paths are drawn."""
    import torch

    import ellm_amd

    rng = np.random.default_rng(2000 + block)
    paths = set()
    for n in range(6):
        c = _draw_ragged(rng)
        dtype = orc.F16 if (n + block) % 2 else orc.BF16
        print("case", block, n, {k: v for k, v in c.items() if k != "pos"}, c["pos"][:8], flush=True)
        b, hq, hkv, cap = c["b"], c["hq"], c["hkv"], c["cap"]
        q = rand_storage((1, b, hq, D), 7500 + 10 * block + n, dtype)
        k = rand_storage((b, hkv, cap, D), 8500 + 10 * block + n, dtype)
        v = rand_storage((b, hkv, cap, D), 9500 + 10 * block + n, dtype)
        scale = 1.0 / np.sqrt(D)
        want, want_lse = orc.attention(q, k, v, scale, dtype, positions=c["pos"], batch=b)
        got, got_lse = gpu_attention(q, k, v, scale, dtype, positions=c["pos"], batch=b)
        res = compare(got, orc.from_storage(want, dtype), dtype)
        assert res["ok"], (c, res)
        assert float(np.abs(got_lse - want_lse).max()) <= LSE_TOL, c


# (sequences, kv heads, group, cached positions): shapes whose planes divide the compute units
# and shapes that do not, one to hundreds of splits per plane, one and two fold levels
UNIFORM_STEPS = [
    (20, 4, 2, 8192),    # 80 planes: 3 splits, one workgroup per unit
    (24, 4, 2, 4096),    # 96 planes: 5 splits, two per unit
    (3, 1, 8, 40000),    # 3 planes: 79 splits, five clusters to fold
    (7, 2, 4, 5000),     # 14 planes: a full cluster of 16 splits
    (1, 2, 4, 70000),    # 2 planes: 122 splits
    (33, 4, 2, 3000),    # 132 planes: 3 splits, two per unit
    (100, 4, 1, 1024),   # more planes than units: no split
    (64, 1, 16, 2048),   # 64 planes x 4, sixteen heads a group
]


@pytest.mark.parametrize("case", UNIFORM_STEPS, ids=["%dx%dx%d_%d" % c for c in UNIFORM_STEPS])
def test_uniform_single_token_steps_over_split_plans(case):
    b, hkv, g, cached = case
    dtype = orc.F16 if (b + cached) % 2 == 0 else orc.BF16
    hq = hkv * g
    print("case", case, "f16" if dtype == orc.F16 else "bf16", flush=True)
    q = rand_storage((1, b, hq, D), 31, dtype)
    k = rand_storage((b, hkv, cached, D), 32, dtype)
    v = rand_storage((b, hkv, cached, D), 33, dtype)
    scale = 1.0 / np.sqrt(D)
    want, want_lse = orc.attention(q, k, v, scale, dtype, position_index=cached - 1)
    got, got_lse = gpu_attention(q, k, v, scale, dtype, position_index=cached - 1)
    res = compare(got, orc.from_storage(want, dtype), dtype)
    assert res["ok"], (case, res)
    assert float(np.abs(got_lse - want_lse).max()) <= LSE_TOL, case
