"""ORACLE — TEST INFRASTRUCTURE ONLY.  ctypes loaders for

  libtde_oracle.so      oracle/tde_oracle.c, the scalar C restatement (built by `make -C oracle`)
  _ref/libunit_ref.so   the reference's own CPU check test::allreduce_rmsnorm_ref
                        (test/unit_test.cpp:175-217), compiled from the reference's file; present
                        only where the reference tree was available at build time.

numpy in, numpy out; bf16/fp16 arrays travel as uint16 bit patterns."""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libtde_oracle.so")
REF_LIB = os.path.join(HERE, "_ref", "libunit_ref.so")

BF16, F16, F32 = 0, 1, 2
QUANT = {"none": 0, "fp8_token": 1, "fp8_group": 2, "int8_token": 3}
SUMSQ_F32_SEQ, SUMSQ_F64, SUMSQ_F32_PAIRWISE, SUMSQ_TORCH = 0, 1, 2, 3

_lib = None
_ref = None


def build():
    import subprocess
    subprocess.run(["make", "-C", HERE], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        L = ctypes.CDLL(LIB)
        L.tdo_bf16_to_f32.restype = ctypes.c_float
        L.tdo_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.tdo_f32_to_bf16.restype = ctypes.c_uint16
        L.tdo_f32_to_bf16.argtypes = [ctypes.c_float]
        L.tdo_f16_to_f32.restype = ctypes.c_float
        L.tdo_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.tdo_f32_to_f16.restype = ctypes.c_uint16
        L.tdo_f32_to_f16.argtypes = [ctypes.c_float]
        L.tdo_e4m3_to_f32.restype = ctypes.c_float
        L.tdo_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.tdo_f32_to_e4m3.restype = ctypes.c_uint8
        L.tdo_f32_to_e4m3.argtypes = [ctypes.c_float]
        L.tdo_reduce_rms.restype = ctypes.c_int
        L.tdo_reduce_rms.argtypes = [
            ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_void_p),
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        L.tdo_torch_row_sum.restype = ctypes.c_float
        L.tdo_torch_row_sum.argtypes = [ctypes.c_void_p, ctypes.c_int64]
        L.tdo_unit_test_ref.restype = ctypes.c_int
        L.tdo_unit_test_ref.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int64, ctypes.c_int64, ctypes.c_int] + \
            [ctypes.c_void_p] * 2 + [ctypes.c_float]
        _lib = L
    return _lib


def have_ref():
    return os.path.exists(REF_LIB)


def ref():
    global _ref
    if _ref is None:
        R = ctypes.CDLL(REF_LIB)
        R.ref_allreduce_rmsnorm.restype = ctypes.c_int
        R.ref_allreduce_rmsnorm.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_void_p] * 2 + \
            [ctypes.c_float]
        _ref = R
    return _ref


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def reduce_rms(dtype, parts, residual, gamma, eps, quant="none", sumsq_mode=SUMSQ_F64, want_norm=True):
    """parts: list of N C-contiguous [T,H] arrays (uint16 bit patterns for bf16/f16, float32 for f32).
    Returns dict(residual_out, norm_out[, q (uint8), scale (float32)])."""
    T, H = residual.shape
    n = len(parts)
    parts = [np.ascontiguousarray(p) for p in parts]
    residual = np.ascontiguousarray(residual)
    gamma = np.ascontiguousarray(gamma)
    arr = (ctypes.c_void_p * n)(*[p.ctypes.data for p in parts])
    res_out = np.empty_like(residual)
    norm_out = np.empty_like(residual) if want_norm else None
    q = scale = None
    qm = QUANT[quant]
    if qm:
        q = np.empty((T, H), dtype=np.uint8)
        scale = np.empty((T, H // 128) if quant == "fp8_group" else (T,), dtype=np.float32)
    rc = lib().tdo_reduce_rms(dtype, n, T, H, arr, _ptr(residual), _ptr(gamma), eps, qm, sumsq_mode, _ptr(res_out),
                              _ptr(norm_out) if want_norm else None, _ptr(q) if qm else None,
                              _ptr(scale) if qm else None)
    if rc != 0:
        raise ValueError("tdo_reduce_rms rejected its arguments")
    out = {"residual_out": res_out}
    if want_norm:
        out["norm_out"] = norm_out
    if qm:
        out["q"], out["scale"] = q, scale
    return out


def torch_row_sums(a):
    """Row sums of a C-contiguous float32 [T, n] array in the order of torch's CPU reduction (tdo_torch_row_sum)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    L = lib()
    return np.array([L.tdo_torch_row_sum(a[i].ctypes.data, a.shape[1]) for i in range(a.shape[0])], dtype=np.float32)


def _unit(fn, parts, residual, gamma, eps, int64_sizes):
    n, T, H = parts.shape
    parts = np.ascontiguousarray(parts, dtype=np.float32)
    residual = np.ascontiguousarray(residual, dtype=np.float32)
    gamma = np.ascontiguousarray(gamma, dtype=np.float32)
    res_out = np.empty((T, H), dtype=np.float32)
    norm_out = np.empty((T, H), dtype=np.float32)
    rc = fn(_ptr(parts), _ptr(residual), _ptr(gamma), T * H, H, n, _ptr(res_out), _ptr(norm_out), eps)
    assert rc == 0
    return res_out, norm_out


def unit_test_ref(parts, residual, gamma, eps):
    """This build's restatement of test/unit_test.cpp:175-217 (fp32 only). parts [N,T,H] float32."""
    return _unit(lib().tdo_unit_test_ref, parts, residual, gamma, eps, True)


def reference_unit_test_ref(parts, residual, gamma, eps):
    """The reference's own function (oracle/_ref).  Only where have_ref()."""
    return _unit(ref().ref_allreduce_rmsnorm, parts, residual, gamma, eps, False)
