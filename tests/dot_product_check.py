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


def check(imp: np.ndarray, ref: np.ndarray, bnd: np.ndarray, out_type: str, ksb: int):
    """Returns a dict with pass/fail and the statistics the reference reports; raises nothing."""
    imp = np.asarray(imp, np.float64).ravel()
    ref = np.asarray(ref, np.float64).ravel()
    bnd = np.asarray(bnd, np.float64).ravel()
    abs_bound = 2 * ksb
    var_bound = 4.0 * 0.4 * ksb
    unit = np.maximum(bnd * 2.0 ** (-1 - NORMAL_FRAC[out_type]), NORMAL_MIN[out_type])
    zero_bnd = bnd == 0.0
    err = np.where(zero_bnd, 0.0, (imp - ref) / unit)
    ok_zero = np.all((ref[zero_bnd] == 0.0) & (imp[zero_bnd] == 0.0))
    ok_nan = not np.any(np.isnan(imp) & ~np.isnan(ref))
    max_err = float(np.max(np.abs(err))) if err.size else 0.0
    sumsq = float(np.sum(err * err))
    T = imp.size
    # ULP and relative error as the reference's ULP verifier defines them (verify_ulp.cpp:27-47)
    mag = np.maximum(2.0 ** np.floor(np.log2(np.maximum(np.abs(ref), 1e-300))), NORMAL_MIN[out_type])
    ulp = np.abs(imp - ref) / (mag * 2.0 ** (-NORMAL_FRAC[out_type]))
    nz = np.abs(ref) > 0
    rel = np.abs(imp - ref)[nz] / np.abs(ref)[nz]
    return dict(ok=bool(ok_zero and ok_nan and max_err <= abs_bound and sumsq <= var_bound * T),
                max_err=max_err, abs_bound=abs_bound, err_sumsq=sumsq, var_limit=var_bound * T,
                max_ulp=float(ulp.max()) if ulp.size else 0.0, max_rel=float(rel.max()) if rel.size else 0.0)
