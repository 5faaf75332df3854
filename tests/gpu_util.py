"""Helpers for the GPU parity tests: run the HIP path through the C ABI on numpy
storage arrays and compare with the CPU oracle under the stated tolerance."""
import numpy as np

import oracle_lib as orc

D = 128

# Tolerance of the operator's numerical contract (binary32 accumulation on both
# sides), stated for binary16 storage: output max-abs <= 2e-3 and max-rel <= 1e-2,
# log-sum-exp within 1e-4.  bfloat16 keeps 3 fewer significand bits, in the output
# and in the probabilities fed to the second MFMA, so its output bounds are 8x wider.
ATOL = {orc.F16: 2e-3, orc.BF16: 1.6e-2}
RTOL = {orc.F16: 1e-2, orc.BF16: 8e-2}
LSE_TOL = 1e-4
# Relative error is taken over elements with |reference| >= REL_FLOOR.  The second
# matrix product runs on 16-bit MFMA inputs, so every probability carries a relative
# rounding error of up to 2^-11 (2^-8 for bfloat16) and the output an absolute
# perturbation of that size times the values it averages; no implementation of this
# design can bound the error relative to outputs far smaller than those values
# (cancellation), which is what the absolute bound is for.  Measured on MI355X: max-rel
# 3.7e-3 over |ref| >= 2^-4 and 1.5e-2 over |ref| >= 2^-6 (binary16, rows with few keys).
REL_FLOOR = 2.0 ** -4
# A second, wider bound two octaves further down, so that a regression among the small outputs
# fails a test instead of only showing in a printed figure: 2x RTOL over |ref| >= 2^-6
# (measured worst case 1.8e-2, the 32768-token prefill of BASELINE configs[2]).
REL_FLOOR_LOW = 2.0 ** -6
RTOL_LOW = {orc.F16: 2e-2, orc.BF16: 1.6e-1}


def storage_ulp(ref, dtype):
    """Spacing of the storage type at |ref| (binary16: 11-bit, bfloat16: 8-bit significand)."""
    bits = 10 if dtype == orc.F16 else 7
    a = np.maximum(np.abs(ref), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - bits)


def compare(got, want, dtype):
    """got/want: binary32 arrays decoded from storage.  Returns error figures and `ok`.

    The absolute bound is ATOL, strictly, wherever one unit in the last place of the storage
    type at the reference value is below ATOL (binary16: |ref| < 4).  Above that both sides
    round binary32 results to storage values that are further apart than ATOL, so results
    that differ by 1e-6 before rounding can land on adjacent values: there, and only there,
    the bound is one unit in the last place (`n_beyond_atol_within_1ulp` counts the elements
    that needed it).  The relative bound RTOL is taken over |ref| >= REL_FLOOR, and RTOL_LOW
    (twice as wide) over |ref| >= REL_FLOOR_LOW = 2^-6."""
    err = np.abs(got - want)
    ulp = storage_ulp(want, dtype)
    coarse = ulp > ATOL[dtype]                  # storage spacing wider than the absolute bound
    fine_err = err[~coarse]
    max_abs_fine = float(fine_err.max()) if fine_err.size else 0.0
    ok_abs = max_abs_fine <= ATOL[dtype] and bool((err[coarse] <= ulp[coarse]).all())

    def rel_at(floor):
        sel = np.abs(want) >= floor
        return float((err[sel] / np.abs(want[sel])).max()) if sel.any() else 0.0

    rel = rel_at(REL_FLOOR)
    rel_low = rel_at(REL_FLOOR_LOW)
    return {
        "max_abs": float(err.max()),
        "max_abs_where_1ulp_below_atol": max_abs_fine,
        "n_beyond_atol_within_1ulp": int((err[coarse] > ATOL[dtype]).sum()),
        "max_rel": rel,
        "max_rel_floor_2^-6": rel_low,
        "ok": ok_abs and rel <= RTOL[dtype] and rel_low <= RTOL_LOW[dtype] and not np.isnan(got).any(),
    }


def torch_dtype(dtype):
    import torch

    return torch.float16 if dtype == orc.F16 else torch.bfloat16


def to_dev(a, dtype):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(torch_dtype(dtype))


def to_host(t, dtype):
    import torch

    return orc.from_storage(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16), dtype)


def gpu_attention(q, k, v, scale, dtype, position_index=0, batch=None, positions=None,
                  kv_strides=None, cap=None, out_fill=None, kv_heads=None):
    """q [S,Bcap,Hq,D]; k, v [B,Hkv,cap,D] storage arrays (or any layout with kv_strides).
    Returns (out binary32 [S,Bcap,Hq,D], lse [S,Bcap,Hq])."""
    import torch

    import ellm_amd

    S, bcap, hq, _ = q.shape
    if kv_strides is None:
        hkv, cap = k.shape[1], k.shape[2]
        kv_strides = [hkv * cap * D, cap * D, D, 1]
    else:
        hkv = kv_heads
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    dout = torch.full_like(dq, float("nan") if out_fill is None else out_fill)
    dlse = torch.full((S, bcap, hq), float("nan"), dtype=torch.float32, device="cuda")
    op = ellm_amd.Attention(dq, dk, dv, dout, bcap, hq, hkv, D, kv_strides, scale, lse=dlse,
                            sequence_capacity=cap, max_position_interval=S)
    b = bcap if batch is None else batch
    if positions is None:
        op.run(position_index, S, b)
    else:
        dpos = torch.from_numpy(np.asarray(positions, dtype=np.uint32).view(np.int32)).cuda()
        op.run_ragged(dpos, int(np.max(positions)), b)
    torch.cuda.synchronize()
    out = to_host(dout, dtype)
    lse = dlse.cpu().numpy()
    op.close()
    return out, lse


def rand_storage(shape, seed, dtype, scale=1.0):
    rng = np.random.default_rng(seed)
    return orc.to_storage(rng.standard_normal(shape, dtype=np.float32) * np.float32(scale), dtype)


def compare_ulps(got, want, dtype, ulps=1.0, floor=2.0 ** -3):
    """Projection outputs: both sides accumulate in binary32 (in different orders) and round
    once, so they may land on adjacent storage values: |got - want| <= `ulps` units in the
    last place of the storage type at max(|want|, floor)."""
    err = np.abs(got - want)
    bound = ulps * storage_ulp(np.maximum(np.abs(want), floor), dtype)
    return {"max_abs": float(err.max()), "worst_ulps": float((err / bound * ulps).max()),
            "ok": bool((err <= bound).all()) and not np.isnan(got).any()}
