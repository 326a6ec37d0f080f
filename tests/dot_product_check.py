"""The TOSA DOT_PRODUCT compliance check for floating-point CONV2D / MATMUL results, restated from
reference_model/src/verify/verify_dot_product.cpp:30-139 (constants: verify_utils.h:178-200; ksb, abs_bound and
var_bound: verif/generator/tosa_test_gen.py:275-297).  Test infrastructure only.

ref  = the operator evaluated in fp64 on the same operands,
bnd  = the same with |operands| (and |bias|),
imp  = the implementation's result.
"""
from __future__ import annotations

import math

import numpy as np

NORMAL_FRAC = {"fp16": 10, "bf16": 7, "fp32": 23}
NORMAL_MIN = {"fp16": 2.0 ** -14, "bf16": 2.0 ** -126, "fp32": 2.0 ** -126}
ACC_FRAC = {"fp32": 23, "fp16": 10}


def kernel_size_bound(ks: int, out_type: str, acc_type: str = "fp32", has_bias: bool = True) -> int:
    """ksb = ceil(KS / 2^((frac(acc) - frac(out)) / 2)) + (1 if bias)"""
    scale = 2.0 ** ((ACC_FRAC[acc_type] - NORMAL_FRAC[out_type]) / 2.0) if ACC_FRAC[acc_type] > NORMAL_FRAC[out_type] else 1.0
    return int(math.ceil(ks / scale)) + (1 if has_bias else 0)


def _overflows(x: np.ndarray, out_type: str) -> np.ndarray:
    """isinf(cast<OutType>(x)) for non-negative fp64 x, the cast rounding to nearest even"""
    with np.errstate(over="ignore"):
        if out_type == "fp16":
            return np.isinf(x.astype(np.float16))
        f32 = x.astype(np.float32)
        if out_type == "fp32":
            return np.isinf(f32)
        # bf16: the float32 value rounds up to infinity from 0x7f7f8000 on
        bits = f32.view(np.uint32).astype(np.uint64)
        rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
        return (rounded & 0x7FFF) >= 0x7F80


def check(imp: np.ndarray, ref: np.ndarray, bnd: np.ndarray, out_type: str, ksb: int, set_number: int = -1):
    """validateDataDP (verify_dot_product.cpp:89-139) over validateElement (:30-87): a NaN reference must be matched
    by a NaN; a NaN bound, or a bound at which the dot product may overflow the output type, asks for nothing; a zero
    bound asks for exact zeros; otherwise the error in units of max(bnd * 2^-(1+frac), normal_min) must stay within
    abs_bound = 2 ksb.  Over the tensor: the sum of squared errors within 1.6 ksb T, and for the data sets 3..5 the
    error sum within sqrt(10 * 1.6 ksb * T).  Returns a dict with pass/fail and the statistics; raises nothing."""
    imp = np.asarray(imp, np.float64).ravel()
    ref = np.asarray(ref, np.float64).ravel()
    bnd = np.asarray(bnd, np.float64).ravel()
    abs_bound = 2 * ksb
    var_bound = 4.0 * 0.4 * ksb
    frac = NORMAL_FRAC[out_type]
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        nan_ref = np.isnan(ref)
        nan_bnd = ~nan_ref & np.isnan(bnd)
        overflow = ~nan_ref & ~nan_bnd & _overflows(np.nan_to_num(bnd * (1 + abs_bound * 2.0 ** (-1 - frac)), nan=0.0),
                                                    out_type)
        zero_bnd = ~nan_ref & ~nan_bnd & ~overflow & (bnd == 0.0)
        ranged = ~(nan_ref | nan_bnd | overflow | zero_bnd)
        unit = np.maximum(bnd * 2.0 ** (-1 - frac), NORMAL_MIN[out_type])
        err = np.where(ranged, (imp - ref) / unit, 0.0)
        failed = (nan_ref & ~np.isnan(imp)) | (zero_bnd & ~((ref == 0.0) & (imp == 0.0))) | \
                 (ranged & ~(np.abs(err) <= abs_bound))
    max_err = float(np.max(np.abs(err))) if err.size else 0.0
    err_sum = float(np.sum(err))
    sumsq = float(np.sum(err * err))
    T = imp.size
    ok = not bool(failed.any()) and sumsq <= var_bound * T
    if 3 <= set_number <= 5:
        ok = ok and abs(err_sum) <= math.sqrt(10 * var_bound * T)
    # ULP as the reference's ULP verifier defines it (verify_ulp.cpp:27-47: the unit is the last bit at the power of
    # two of |ref|, not below normal_min; a zero reference has no ULP), the relative error, and the error relative
    # to the bound tensor (the sum of the absolute products, the scale the DOT_PRODUCT check itself uses)
    fin = np.isfinite(ref) & np.isfinite(imp) & (ref != 0.0)
    with np.errstate(invalid="ignore", divide="ignore"):
        mag = np.maximum(2.0 ** np.floor(np.log2(np.maximum(np.abs(ref[fin]), 1e-300))), NORMAL_MIN[out_type])
        ulp = np.abs(imp[fin] - ref[fin]) / (mag * 2.0 ** (-frac))
        nz = np.abs(ref[fin]) > 0
        rel = np.abs(imp[fin] - ref[fin])[nz] / np.abs(ref[fin])[nz]
        # elements without cancellation worth speaking of: |ref| at least an eighth of the sum of absolute products
        cond = np.abs(ref[fin]) >= bnd[fin] / 8
        pos = fin & (bnd > 0)
        to_bound = np.abs(imp[pos] - ref[pos]) / bnd[pos]
    return dict(ok=bool(ok), max_rel_to_bound=float(to_bound.max()) if to_bound.size else 0.0, max_err=max_err, abs_bound=abs_bound, err_sum=err_sum, err_sumsq=sumsq,
                var_limit=var_bound * T, failed_elements=int(failed.sum()),
                max_ulp=float(ulp.max()) if ulp.size else 0.0,
                max_ulp_conditioned=float(ulp[cond].max()) if cond.any() else 0.0, max_rel=float(rel.max()) if rel.size else 0.0)
