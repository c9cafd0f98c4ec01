"""TEST INFRASTRUCTURE ONLY -- ctypes front end of the C oracle (ss2d_oracle.c).

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this module; the shipped package never does.  Tensors are torch CPU tensors
(torch is used as a typed buffer here, nothing more); bf16/f16 inputs of the
selective scan are widened to fp32 exactly before they reach C, which is what
the reference does with ``.float()`` (kernels/selective_scan/test_selective_scan.py:184-200).
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libss2d_oracle.so")
_lib = None

CHUNK = 2048  # kernels/selective_scan/csrc/selective_scan/cusoflex/selective_scan_oflex.cpp:206


def build(force=False):
    """Compile ss2d_oracle.c with the Makefile beside it."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.ss2d_oracle_num_threads.restype = ctypes.c_int
        for name in ("ss2d_oracle_cross_scan", "ss2d_oracle_cross_merge_f32",
                     "ss2d_oracle_cross_merge_bf16", "ss2d_oracle_selective_scan"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def num_threads():
    return int(lib().ss2d_oracle_num_threads())


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _cpu(t):
    assert t.device.type == "cpu", "the oracle works on CPU tensors"
    return t.contiguous()


def cross_scan(x):
    """x (B,C,H,W) any dtype -> (B,4,C,H*W); csm_triton.py:22-29."""
    x = _cpu(x)
    B, C, H, W = x.shape
    y = torch.empty((B, 4, C, H * W), dtype=x.dtype)
    rc = lib().ss2d_oracle_cross_scan(_p(x), _p(y), B, C, H, W, x.element_size())
    assert rc == 0, rc
    return y


def cross_merge(ys, order=0):
    """ys (B,4,C,H,W) f32|bf16 -> (B,C,H*W); csm_triton.py:56-62 (order 0) or :362-370 (order 1)."""
    ys = _cpu(ys)
    B, K, C, H, W = ys.shape
    assert K == 4
    out = torch.empty((B, C, H * W), dtype=ys.dtype)
    if ys.dtype == torch.float32:
        rc = lib().ss2d_oracle_cross_merge_f32(_p(ys), _p(out), B, C, H, W, order)
    elif ys.dtype == torch.bfloat16:
        rc = lib().ss2d_oracle_cross_merge_bf16(_p(ys), _p(out), B, C, H, W, order)
    else:
        raise TypeError(f"oracle cross_merge: unsupported dtype {ys.dtype}")
    assert rc == 0, rc
    return out


def selective_scan(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False,
                   out_float=True, wide=False, return_x=False):
    """selective_scan_ref (test_selective_scan.py:168-234) with 4-D B/C.

    Returns out (batch, dim, L): fp32 when ``out_float`` (csms6s.py:68, oflex) else
    rounded to u.dtype (test_selective_scan.py:233); float64 when ``wide``.
    With ``return_x`` also the chunk-end states (batch, dim, ceil(L/2048), 2N).
    """
    dtype_in = u.dtype
    u, delta, B, C = (_cpu(t).float() for t in (u, delta, B, C))
    A = _cpu(A).float()
    D = _cpu(D).float() if D is not None else None
    delta_bias = _cpu(delta_bias).float() if delta_bias is not None else None
    batch, dim, L = u.shape
    delta_dim = delta.shape[1]
    _, G, N, _ = B.shape
    assert A.shape == (dim, N) and C.shape == B.shape and delta.shape == (batch, delta_dim, L)
    n_chunks = (L + CHUNK - 1) // CHUNK
    out = torch.empty((batch, dim, L), dtype=torch.float32) if not wide else None
    out64 = torch.empty((batch, dim, L), dtype=torch.float64) if wide else None
    xst = torch.zeros((batch, dim, n_chunks, 2 * N), dtype=torch.float32) if (return_x and not wide) else None
    rc = lib().ss2d_oracle_selective_scan(
        _p(u), _p(delta), _p(A), _p(B), _p(C), _p(D), _p(delta_bias), int(bool(delta_softplus)),
        batch, dim, L, N, G, delta_dim, _p(out), _p(xst), _p(out64), int(bool(wide)))
    assert rc == 0, rc
    if wide:
        return out64
    res = out if out_float else out.to(dtype_in)
    return (res, xst) if return_x else res
