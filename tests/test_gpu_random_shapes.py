"""Seeded sweep of chunk attention shapes against the CPU oracle through the C ABI: head layouts,
batch below capacity, chunk lengths either side of the kernels' row limits (128 / 256 / 384 query
rows per K/V plane), cached lengths on and off tile edges.  The shapes are drawn so that the
planner splits the key range evenly, unevenly and not at all."""
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
