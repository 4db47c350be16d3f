"""CPU oracle for the BGEMM / BWTA hot path -- TEST INFRASTRUCTURE ONLY.

Nothing under the product package may import this module.  It is used by the
tests, by the smoke check and by the CPU-baseline leg of the benchmark, always as
the checker and never as the thing shipped or measured as the product.

Three layers live here:

* ``lib()`` and the ``c_*`` wrappers: the plain-C restatement of the reference
  arithmetic in ``bgemm_oracle.c`` (pack rule, the three INSTR modes, ternary
  BWTA, the split-K partition and the fp16 rounding of the reference launcher).
* ``dense_*``: the same quantities written as dense integer matmuls on
  de-binarised operands.  They are the closed forms that pin the C code (and the
  HIP kernels) independently of any bit trick, and are what the reference's own
  drivers compare against (lowbit_kernel/csrc/benchmark.cu:146-159,
  tests/python/test_kernel.py:48-63).
* ``cpu_path_*``: the reference CPU path, "torch matmul on +-1/0 tensors"
  (tests/python/bgemm_linear.py:222-275 and :599-645), used as the CPU baseline.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libbgemm_oracle.so")
_lib = None

AND_POP, XOR_POP, ATTN_MM = 0, 1, 2  # lowbit_kernel/csrc/include/configs.h:70-72


def build(force=False):
    """Compile bgemm_oracle.c with gcc into oracle/libbgemm_oracle.so."""
    src = os.path.join(_HERE, "bgemm_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["gcc", "-O2", "-Wall", "-Wextra", "-fPIC", "-shared", "-o", _SO, src])
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        i64, p = ctypes.c_int64, ctypes.c_void_p
        L.oracle_pack_sign_f16.argtypes = [p, i64, i64, i64, p]
        L.oracle_pack_sign_f16.restype = None
        L.oracle_pack_ternary_f16.argtypes = [p, i64, i64, i64, p, p]
        L.oracle_pack_ternary_f16.restype = None
        L.oracle_bgemm_packed.argtypes = [ctypes.c_int, p, p, p, i64, i64, i64]
        L.oracle_bgemm_packed.restype = ctypes.c_int
        L.oracle_bwta_packed.argtypes = [p, p, p, p, i64, i64, i64]
        L.oracle_bwta_packed.restype = None
        L.oracle_int_to_f16.argtypes = [ctypes.c_int32]
        L.oracle_int_to_f16.restype = ctypes.c_uint16
        L.oracle_bgemm_f16.argtypes = [p, p, p, p, i64, i64, i64, ctypes.c_int, ctypes.c_int]
        L.oracle_bgemm_f16.restype = ctypes.c_int
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _as_u16(x):
    """fp16 ndarray (or uint16 bit patterns) -> contiguous uint16 view, 2-D."""
    x = np.ascontiguousarray(x)
    if x.dtype == np.float16:
        x = x.view(np.uint16)
    assert x.dtype == np.uint16 and x.ndim == 2
    return x


def words_for(K):
    return (K + 31) // 32


# ---------------------------------------------------------------- C oracle wrappers
def c_pack_sign(x_f16):
    x = _as_u16(x_f16)
    R, K = x.shape
    out = np.zeros((R, words_for(K)), dtype=np.uint32)
    lib().oracle_pack_sign_f16(_ptr(x), R, K, K, _ptr(out))
    return out


def c_pack_ternary(x_f16):
    x = _as_u16(x_f16)
    R, K = x.shape
    nz = np.zeros((R, words_for(K)), dtype=np.uint32)
    sg = np.zeros_like(nz)
    lib().oracle_pack_ternary_f16(_ptr(x), R, K, K, _ptr(nz), _ptr(sg))
    return nz, sg


def c_bgemm_packed(mode, Wp, Xp, K):
    Wp = np.ascontiguousarray(Wp, dtype=np.uint32)
    Xp = np.ascontiguousarray(Xp, dtype=np.uint32)
    M, N = Wp.shape[0], Xp.shape[0]
    assert Wp.shape[1] == Xp.shape[1] == words_for(K)
    C = np.zeros((N, M), dtype=np.int32)
    rc = lib().oracle_bgemm_packed(mode, _ptr(Wp), _ptr(Xp), _ptr(C), M, N, K)
    if rc:
        raise ValueError("oracle_bgemm_packed: bad mode %r" % (mode,))
    return C


def c_bwta_packed(Wp, Xnz, Xsg, K):
    Wp = np.ascontiguousarray(Wp, dtype=np.uint32)
    Xnz = np.ascontiguousarray(Xnz, dtype=np.uint32)
    Xsg = np.ascontiguousarray(Xsg, dtype=np.uint32)
    M, N = Wp.shape[0], Xnz.shape[0]
    C = np.zeros((N, M), dtype=np.int32)
    lib().oracle_bwta_packed(_ptr(Wp), _ptr(Xnz), _ptr(Xsg), _ptr(C), M, N, K)
    return C


def c_int_to_f16(v):
    v = np.asarray(v, dtype=np.int32)
    f = lib().oracle_int_to_f16
    out = np.array([f(int(t)) for t in v.ravel()], dtype=np.uint16)
    return out.reshape(v.shape).view(np.float16)


def c_bgemm_f16(x_f16, w_f16, splitK=1, mode=XOR_POP):
    """The whole reference call: half[N,K], half[M,K] -> (half[N,M], int32[N,M])."""
    X, W = _as_u16(x_f16), _as_u16(w_f16)
    N, K = X.shape
    M = W.shape[0]
    assert W.shape[1] == K
    o16 = np.zeros((N, M), dtype=np.uint16)
    o32 = np.zeros((N, M), dtype=np.int32)
    rc = lib().oracle_bgemm_f16(_ptr(W), _ptr(X), _ptr(o16), _ptr(o32), M, N, K, splitK, mode)
    if rc:
        raise ValueError("oracle_bgemm_f16 failed with %d" % rc)
    return o16.view(np.float16), o32


# ---------------------------------------------------------------- dense closed forms
def signbit(x_f16):
    """1 where the IEEE sign bit is set (so -0.0 -> 1), as the kernel binarises."""
    return (_as_u16(x_f16) >> 15).astype(np.int64)


def dense_bgemm(mode, w_f16, x_f16):
    """C[n,m] by integer matmul on de-binarised operands.

    XOR : sum_k s(W)s(X),  s = -1 where sign bit set, else +1
    AND : #{k : W<0 and X<0}   (both sign bits set)
    ATTN: sum_k [sign bit of W clear] * s(X)      (benchmark.cu:146-159)
    """
    a, b = signbit(w_f16), signbit(x_f16)
    if mode == XOR_POP:
        return ((1 - 2 * b) @ (1 - 2 * a).T).astype(np.int32)
    if mode == AND_POP:
        return (b @ a.T).astype(np.int32)
    if mode == ATTN_MM:
        return ((1 - 2 * b) @ (1 - a).T).astype(np.int32)
    raise ValueError(mode)


def dense_bwta(w_f16, x_f16):
    """Binary weight x ternary activation: sign(X) @ s(W).T with torch.sign's 0."""
    xs = _as_u16(x_f16)
    t = np.where((xs & 0x7FFF) == 0, 0, np.where(xs >> 15, -1, 1)).astype(np.int64)
    return (t @ (1 - 2 * signbit(w_f16)).T).astype(np.int32)


def bits_to_f16(bits, zero_mask=None):
    """{0,1} bit array -> fp16 +-1.0 (bit 1 -> -1.0); zero_mask -> +0.0."""
    v = np.where(np.asarray(bits) != 0, np.float16(-1.0), np.float16(1.0)).astype(np.float16)
    if zero_mask is not None:
        v = np.where(zero_mask, np.float16(0.0), v).astype(np.float16)
    return v


# ---------------------------------------------------------------- layer prologue / epilogue
def np_center_to_f16(x, zero_point):
    """What the binary Linear layers hand to the kernel (bgemm_linear.py:479-482, :140-141):
    ``(x - zp)`` in the tensor's own type (fp32, or fp16 evaluated through fp32 and rounded),
    then ``.to(torch.half)``.  Returns the fp16 array whose sign bits get packed."""
    x = np.asarray(x)
    if x.dtype == np.float32:
        return (x - np.float32(zero_point)).astype(np.float16)
    assert x.dtype == np.float16
    return (x.astype(np.float32) - np.float32(np.float16(zero_point))).astype(np.float16)


def np_scale_epilogue(acc_i32, sw, sa, bias=None):
    """``half(acc) * sw * sa (+ bias)`` (bgemm_linear.py:482-484) with torch's type promotion:
    fp32 parameters -> every step is an fp32 operation and the result is fp32; fp16 parameters ->
    every step is evaluated in fp32 and rounded to fp16.  acc: int32 [N,M]; sw: [M]; sa: scalar."""
    with np.errstate(over="ignore"):
        h = np.asarray(acc_i32).astype(np.float32).astype(np.float16)
    sw = np.asarray(sw)
    if sw.dtype == np.float32:
        r = h.astype(np.float32) * sw[None, :]
        r = r * np.float32(sa)
        return r + np.asarray(bias, dtype=np.float32)[None, :] if bias is not None else r
    assert sw.dtype == np.float16
    with np.errstate(over="ignore", invalid="ignore"):
        r = (h.astype(np.float32) * sw.astype(np.float32)[None, :]).astype(np.float16)
        r = (r.astype(np.float32) * np.float32(np.float16(sa))).astype(np.float16)
        if bias is not None:
            r = (r.astype(np.float32) + np.asarray(bias, dtype=np.float16).astype(np.float32)[None, :]).astype(np.float16)
    return r


# ---------------------------------------------------------------- reference CPU path
def cpu_path_linear(x_vals, w_vals):
    """torch matmul on +-1/0 tensors: out = x @ w.T  (bgemm_linear.py:270-272)."""
    import torch
    return torch.matmul(x_vals, w_vals.transpose(-1, -2))


def cpu_path_bin_active(x):
    """BinActive.forward (bgemm_linear.py:603-608): sign with 0 -> +1."""
    import torch
    s = x.sign()
    return torch.where(s == 0, torch.ones_like(s), s)


def cpu_path_bnn_linear(x, weight, bias, sw, sa, zpw, zpa):
    """BNNLinear.forward (bgemm_linear.py:633-645)."""
    import torch
    bw = cpu_path_bin_active(weight - zpw)
    bx = cpu_path_bin_active(x - zpa)
    return torch.nn.functional.linear(bx, bw, bias) * sw * sa


def cpu_path_layer_scales(x, w):
    """_initialize of the reference layers (bgemm_linear.py:466-472)."""
    import torch
    sw = w.norm(1, 1).div(w.nelement())
    sa = 2 * x.abs().mean()
    return sw, sa, torch.mean(w), torch.mean(x)
