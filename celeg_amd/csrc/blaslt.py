"""bfloat16 matrix products of many rows through hipBLASLt, called directly.

The products of a prompt's rows are the library's, as in the reference (cuBLASLt there:
src/backend/cuda/model/prefill_batched/non_attention.cpp:175-201).  torch's own call of the
same library costs the host 17 us a product on this machine, which at 65 products a step
makes an unrecorded step of a small model wait for the host; here a product is one call of
``hipblasLtMatmul`` with descriptors and an algorithm that are looked up by the sizes and
made once (3 us).  The library is the copy that torch has loaded, so both paths run the
same kernels.

out[M, N] = x[M, K] w[N, K]^T, all row-major.  In the library's column-major terms that is
D (N x M, ld ldo) = A^T B with A = w (K x N, ld K) and B = x (K x M, ld ldx).
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Optional, Tuple

import torch

HIPBLAS_OP_N, HIPBLAS_OP_T = 111, 112
HIPBLAS_COMPUTE_32F = 2
HIP_R_32F, HIP_R_16BF = 0, 14
DESC_TRANSA, DESC_TRANSB = 0, 1
PREF_MAX_WORKSPACE_BYTES = 1
WORKSPACE_BYTES = 32 << 20


class _Algo(ctypes.Structure):
    _fields_ = [("data", ctypes.c_uint8 * 16), ("max_workspace_bytes", ctypes.c_size_t)]


class _Heuristic(ctypes.Structure):
    _fields_ = [("algo", _Algo), ("workspace_size", ctypes.c_size_t), ("state", ctypes.c_int),
                ("waves_count", ctypes.c_float), ("reserved", ctypes.c_int * 4)]


class BlasLtError(RuntimeError):
    pass


def _library() -> ctypes.CDLL:
    bundled = os.path.join(os.path.dirname(torch.__file__), "lib", "libhipblaslt.so")
    for name in (bundled, "libhipblaslt.so.1", "libhipblaslt.so"):
        try:
            return ctypes.CDLL(name)
        except OSError:
            continue
    raise BlasLtError("libhipblaslt.so was not found (looked beside torch and on the loader's path)")


class BlasLt:
    """One handle, one workspace and the plans (layouts and algorithm) by sizes, per device."""

    def __init__(self, device):
        self.device = torch.device(device)
        self.lib = _library()
        for name in ("hipblasLtCreate", "hipblasLtMatmulDescCreate", "hipblasLtMatmulDescSetAttribute",
                     "hipblasLtMatrixLayoutCreate", "hipblasLtMatmulPreferenceCreate",
                     "hipblasLtMatmulPreferenceSetAttribute", "hipblasLtMatmulAlgoGetHeuristic",
                     "hipblasLtMatmul"):
            getattr(self.lib, name).restype = ctypes.c_int
        self.lib.hipblasLtMatmul.argtypes = [
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
            ctypes.c_void_p]
        self.handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            self._ok(self.lib.hipblasLtCreate(ctypes.byref(self.handle)), "hipblasLtCreate")
        self.desc = ctypes.c_void_p()
        self._ok(self.lib.hipblasLtMatmulDescCreate(ctypes.byref(self.desc), ctypes.c_int(HIPBLAS_COMPUTE_32F),
                                                    ctypes.c_int(HIP_R_32F)), "hipblasLtMatmulDescCreate")
        for attr, op in ((DESC_TRANSA, HIPBLAS_OP_T), (DESC_TRANSB, HIPBLAS_OP_N)):
            value = ctypes.c_int32(op)
            self._ok(self.lib.hipblasLtMatmulDescSetAttribute(self.desc, ctypes.c_int(attr), ctypes.byref(value),
                                                              ctypes.c_size_t(4)), "hipblasLtMatmulDescSetAttribute")
        self.pref = ctypes.c_void_p()
        self._ok(self.lib.hipblasLtMatmulPreferenceCreate(ctypes.byref(self.pref)), "hipblasLtMatmulPreferenceCreate")
        size = ctypes.c_uint64(WORKSPACE_BYTES)
        self._ok(self.lib.hipblasLtMatmulPreferenceSetAttribute(
            self.pref, ctypes.c_int(PREF_MAX_WORKSPACE_BYTES), ctypes.byref(size), ctypes.c_size_t(8)),
            "hipblasLtMatmulPreferenceSetAttribute")
        self.workspace = torch.empty(WORKSPACE_BYTES, dtype=torch.uint8, device=self.device)
        self._workspace_ptr = self.workspace.data_ptr()
        self._one, self._zero = ctypes.c_float(1.0), ctypes.c_float(0.0)
        self._alpha, self._beta = ctypes.addressof(self._one), ctypes.addressof(self._zero)
        self._plans: Dict[Tuple[int, int, int, int, int], Optional[tuple]] = {}

    @staticmethod
    def _ok(status: int, what: str) -> None:
        if status != 0:
            raise BlasLtError(f"{what} failed with hipblasStatus {status}")

    def _layout(self, rows: int, cols: int, ld: int) -> ctypes.c_void_p:
        layout = ctypes.c_void_p()
        self._ok(self.lib.hipblasLtMatrixLayoutCreate(ctypes.byref(layout), ctypes.c_int(HIP_R_16BF),
                                                      ctypes.c_uint64(rows), ctypes.c_uint64(cols),
                                                      ctypes.c_int64(ld)), "hipblasLtMatrixLayoutCreate")
        return layout

    def _plan(self, key):
        M, N, K, ldx, ldo = key
        a, b, d = self._layout(K, N, K), self._layout(K, M, ldx), self._layout(N, M, ldo)
        result, found = _Heuristic(), ctypes.c_int(0)
        status = self.lib.hipblasLtMatmulAlgoGetHeuristic(self.handle, self.desc, a, b, d, d, self.pref,
                                                          ctypes.c_int(1), ctypes.byref(result), ctypes.byref(found))
        if status != 0 or found.value < 1 or result.state != 0 or result.workspace_size > WORKSPACE_BYTES:
            return None          # the library has no kernel for these sizes: the caller takes another way
        return (a, b, d, result.algo, ctypes.addressof(result.algo))

    def matmul(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, stream: int) -> bool:
        """out = x w^T for bfloat16 x [M, K] (rows ldx apart), w [N, K] (dense) and out [M, N]
        (rows ldo apart), on ``stream`` (a raw handle).  False if the library has no kernel
        for these sizes (nothing was launched)."""
        M, K = x.shape
        N = w.shape[0]
        key = (M, N, K, x.stride(0), out.stride(0))
        plan = self._plans.get(key, False)
        if plan is False:
            plan = self._plans[key] = self._plan(key)
        if plan is None:
            return False
        a, b, d, _algo, algo_ptr = plan
        status = self.lib.hipblasLtMatmul(self.handle, self.desc, self._alpha, w.data_ptr(), a, x.data_ptr(), b,
                                          self._beta, out.data_ptr(), d, out.data_ptr(), d, algo_ptr,
                                          self._workspace_ptr, WORKSPACE_BYTES, stream)
        if status != 0:
            raise BlasLtError(f"hipblasLtMatmul failed with hipblasStatus {status} for M, N, K = {M}, {N}, {K}")
        return True
