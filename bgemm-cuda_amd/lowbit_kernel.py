"""Drop-in for the reference's ``lowbit_kernel`` extension module (BGEMM part).

``bgemm_linear_forward_cuda(in_feats, weights, splitK=1, INSTR=1)`` has the reference's
name, argument order, defaults and return value (lowbit_kernel/csrc/pybind.cpp:12,
fp6_linear.cu:561-616): fp16 ``[N,K]`` x fp16 ``[M,K]`` -> fp16 ``[N,M]``.  Everything
else here is the packed-operand surface the reference only stubbed
(binary_weight_prepacking_cuda, fp6_linear.cu:519-542).

All work is enqueued on the current torch stream through the C ABI in
include/bgemm_mi355x.h; torch supplies device memory and streams only.
"""
import contextlib
import collections
import struct
import weakref

import torch

import _lib as _b
from _lib import (MODE_AND, MODE_XOR, MODE_ATTN, MODE_BWTA, MODE_ATTN_X, OUT_I32, OUT_F16, OUT_F32_SCALED,
                  OUT_F16_SCALED, OUT_BITS_F32, OUT_BITS_F16, SRC_F16, SRC_F32, VARIANT_AUTO, VARIANT_VALU, VARIANT_MFMA, VARIANT_MFMA_F4)

AND_POP, XOR_POP, ATTN_MM = 0, 1, 2   # lowbit_kernel/csrc/include/configs.h:70-72

__all__ = ["bgemm_linear_forward_cuda", "binary_weight_prepacking", "pack_sign", "pack_ternary",
           "pack_sign_transposed", "bgemm_packed_forward", "bgemm_packed_weight_forward", "PackedBits", "zeros_packed", "save_packed", "load_packed",
           "set_weight_cache", "packed_kernel_id", "DecodeChain", "AND_POP", "XOR_POP", "ATTN_MM"]


_NULL_CTX = contextlib.nullcontext()


# torch.cuda.current_stream() builds a Stream object (2.7 us a call, a quarter of a decode-size launch from
# Python); the raw handle of the current device's current stream is all the C ABI wants.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _on(device):
    """Context that makes `device` current; free when it already is (the usual case)."""
    if device.index is None or device.index == (_raw_device() if _raw_device is not None else torch.cuda.current_device()):
        return _NULL_CTX
    return torch.cuda.device(device)


# workspace needs per (mode, batch, M, N, K, splitK, variant): two C calls saved per launch
_ws_needs = {}


def _split_k_needs(L, key):
    need = _ws_needs.get(key)
    if need is None:
        need = (L.bgemm_packed_workspace_bytes(*key), L.bgemm_packed_counter_bytes(*key))
        _ws_needs[key] = need
    return need


def _need_cuda(t, name):
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor" % name)
    if not t.is_cuda:
        raise ValueError("%s must live on the GPU" % name)


# Split-K arrival counters must be zero before first use and every call leaves them zero, so
# one zero-filled buffer per (device, stream) is grown on demand and reused; partial tiles
# are plain scratch.
_counters = {}
_scratch = {}


def _split_k_buffers(part_bytes, counter_bytes, device):
    key = (device.index, _stream())
    cnt = _counters.get(key)
    if cnt is None or cnt.numel() < counter_bytes:
        cnt = torch.zeros(max(counter_bytes, 1 << 16), dtype=torch.uint8, device=device)
        _counters[key] = cnt
    ws = _scratch.get(key)
    if ws is None or ws.numel() < part_bytes:
        ws = torch.empty(max(part_bytes, 1 << 20), dtype=torch.uint8, device=device)
        _scratch[key] = ws
    return ws, cnt


class PackedBits:
    """A bit-packed operand in the tiled layout (32 rows x 256 K-bits per 1 KiB tile).

    ``data`` is an int32 tensor ``[batch, words]``; ``data2`` is the second plane of a ternary
    operand (sign & nonzero) or None.
    """

    def __init__(self, data, data2, batch, rows, K):
        self.data, self.data2, self.batch, self.rows, self.K = data, data2, batch, rows, K
        self.counts = None        # int32 [batch, rows] row popcounts once row_popcounts() has been called

    @property
    def ternary(self):
        return self.data2 is not None

    @property
    def words(self):
        return self.data.shape[1]

    def nbytes(self):
        return self.data.numel() * 4 * (2 if self.ternary else 1)


def _check_packed(p, name):
    """A PackedBits is a public constructor: its buffers must be what the kernels will index."""
    words = _b.lib().bgemm_tiled_words(p.rows, p.K)
    for plane in ((p.data, p.data2) if p.ternary else (p.data,)):
        _need_cuda(plane, name)
        if plane.dtype != torch.int32 or tuple(plane.shape) != (p.batch, words) or not plane.is_contiguous():
            raise ValueError("%s: every plane must be a contiguous int32 tensor of shape (%d, %d) for %d rows x %d bits, "
                             "got %s %s" % (name, p.batch, words, p.rows, p.K, plane.dtype, tuple(plane.shape)))
        if plane.device != p.data.device:
            raise ValueError("%s: both planes must live on one device" % name)


def row_popcounts(p):
    """Computes (once) and attaches the row popcounts of a binary packed operand, ``p.counts`` int32
    ``[batch, rows]``, and returns ``p``.  ``bgemm_packed_forward`` hands them to the library when both operands
    carry them: they are part of a prepacked operand, and the large tiles then leave the counting out of their
    main loop.  Call it again after writing new bits into ``p.data`` (it recomputes when ``p.counts`` is None)."""
    if p.ternary:
        raise ValueError("row popcounts are kept for binary operands")
    if p.counts is None:
        _check_packed(p, "p")
        counts = torch.empty((p.batch, p.rows), dtype=torch.int32, device=p.data.device)
        with _on(p.data.device):
            _b.check(_b.lib().bgemm_row_popcounts(p.data.data_ptr(), p.batch, p.rows, p.K, p.words if p.batch > 1 else 0,
                                                  counts.data_ptr(), _stream()))
        p.counts = counts
    return p


def packed_kernel_id(w, x, mode=MODE_XOR, splitK=1, variant=VARIANT_AUTO, out_dtype=torch.int32):
    """The kernel (``_lib.KERNEL_*``) that ``bgemm_packed_forward(w, x, mode, out_dtype, splitK, variant)`` runs
    (2-byte and 4-byte outputs can take different tiles)."""
    kind = OUT_F16 if out_dtype == torch.half else OUT_I32
    rc = _b.lib().bgemm_packed_kernel_id(mode, kind, max(w.batch, x.batch), w.rows, x.rows, w.K, splitK, variant)
    if rc < 0:
        _b.check(rc)
    return rc


def zeros_packed(rows, K, batch=1, device="cuda"):
    """An all-zero binary operand of `rows` x `K` bits: the buffer a GEMM with ``bits_out=`` writes the next
    layer's operand into (its padding must be zero, which later calls of the same shape preserve)."""
    words = _b.lib().bgemm_tiled_words(rows, K)
    return PackedBits(torch.zeros((batch, words), dtype=torch.int32, device=device), None, batch, rows, K)


def _batch_layout(x):
    """(outer, inner, stride_outer, stride_inner) of the leading dimensions of a 2-D to 4-D tensor."""
    if x.dim() == 2:
        return 1, 1, 0, 0
    if x.dim() == 3:
        return 1, x.shape[0], 0, x.stride(0)
    return x.shape[0], x.shape[1], x.stride(0), x.stride(1)


def _pack_source(x, what):
    """fp16 and fp32 tensors are read where they lie if their last dimension is dense and rows do not overlap;
    anything else is brought to contiguous fp16 first."""
    _need_cuda(x, what)
    if x.dim() not in (2, 3, 4):
        raise ValueError("expected a 2-D, 3-D or 4-D tensor, got %d-D" % x.dim())
    if x.dtype not in (torch.half, torch.float32):
        x = x.to(torch.half)
    if x.numel() and (x.stride(-1) != 1 or x.stride(-2) < x.shape[-1]):
        x = x.contiguous()
    return x


def _pack(x, ternary, zero_point=None):
    if zero_point is not None and isinstance(x, torch.Tensor) and x.dtype not in (torch.half, torch.float32):
        raise TypeError("centred packing reads fp16 or fp32 sources, got %s" % x.dtype)
    x = _pack_source(x, "input")
    if zero_point is not None:
        if ternary:
            raise ValueError("a zero point is only taken by the sign pack")
        if not isinstance(zero_point, torch.Tensor) or zero_point.numel() != 1:
            raise TypeError("zero_point must be a one-element tensor")
        _need_cuda(zero_point, "zero_point")
        zero_point = zero_point.detach().to(x.dtype)
    outer, inner, so, si = _batch_layout(x)
    batch = outer * inner
    rows, K = x.shape[-2], x.shape[-1]
    L = _b.lib()
    d0 = torch.empty((batch, L.bgemm_tiled_words(rows, K)), dtype=torch.int32, device=x.device)
    d1 = torch.empty_like(d0) if ternary else None
    with _on(x.device):
        _b.check(L.bgemm_pack_batched(x.data_ptr(), SRC_F32 if x.dtype == torch.float32 else SRC_F16, int(ternary),
                                      None if zero_point is None else zero_point.data_ptr(), outer, inner, rows, K,
                                      x.stride(-2), so, si, d0.data_ptr(), d1.data_ptr() if ternary else None, _stream()))
    return PackedBits(d0, d1, batch, rows, K)


def pack_sign(x, zero_point=None):
    """fp16 or fp32 (or castable) ``[R,K]`` / ``[B,R,K]`` / ``[B,H,R,K]`` -> tiled sign bits (bit = 1 for negative,
    -0.0 included), one launch for the whole batch.  Strided views whose last dimension is dense are read
    where they lie (``permute(0, 2, 1, 3)`` of a ``[B, S, H*d]`` projection, a slice of rows or columns).

    With ``zero_point`` (a one-element device tensor) the bits are those of
    ``(x - zero_point).to(torch.half)``, computed in the same pass: the operand the binary Linear layers
    feed the kernel (bgemm_linear.py:479-482)."""
    return _pack(x, False, zero_point)


def pack_sign_transposed(x):
    """``[K,R]`` / ``[B,K,R]`` / ``[B,H,K,R]`` -> tiled sign bits of the transposes (``R`` rows of ``K`` bits each),
    read as they lie: what ``pack_sign(x.transpose(-1, -2).contiguous())`` gives, without the copy.  The right-hand
    operand of a matmul ``a @ b`` (``b`` is ``[K, M]``) and the value operand of attention are of this kind."""
    x = _pack_source(x, "input")
    outer, inner, so, si = _batch_layout(x)
    K, rows = x.shape[-2], x.shape[-1]
    L = _b.lib()
    d0 = torch.empty((outer * inner, L.bgemm_tiled_words(rows, K)), dtype=torch.int32, device=x.device)
    with _on(x.device):
        _b.check(L.bgemm_pack_transposed_batched(x.data_ptr(), SRC_F32 if x.dtype == torch.float32 else SRC_F16,
                                                 outer, inner, rows, K, x.stride(-2), so, si, d0.data_ptr(), _stream()))
    return PackedBits(d0, None, outer * inner, rows, K)


def pack_ternary(x):
    """``[R,K]`` / ``[B,R,K]`` -> tiled (nonzero, sign&nonzero) planes of sign(x) in {-1,0,+1}."""
    return _pack(x, True)


def binary_weight_prepacking(weights):
    """half ``[OC,IC]`` -> int32 ``[OC, ceil(IC/32)]`` in the reference's logical format
    (bit 31-i of word j = sign bit of element 32j+i; weight_prepacking.h:181-230).  This is what
    binary_weight_prepacking_cuda (fp6_linear.cu:519-542) declares but leaves uninitialised."""
    _need_cuda(weights, "weights")
    if weights.dim() != 2:
        raise ValueError("weights must be 2-D")
    w = weights.to(torch.half).contiguous()
    OC, IC = w.shape
    out = torch.empty((OC, (IC + 31) // 32), dtype=torch.int32, device=w.device)
    with _on(w.device):
        _b.check(_b.lib().bgemm_pack_sign_f16_logical(w.data_ptr(), OC, IC, IC, out.data_ptr(), _stream()))
    return out


def tile_from_logical(logical, K):
    """int32 ``[R, ceil(K/32)]`` logical words -> PackedBits in the tiled layout."""
    _need_cuda(logical, "logical")
    logical = logical.contiguous()
    R = logical.shape[0]
    L = _b.lib()
    d0 = torch.empty((1, L.bgemm_tiled_words(R, K)), dtype=torch.int32, device=logical.device)
    with _on(logical.device):
        _b.check(L.bgemm_tile_from_logical(logical.data_ptr(), R, K, d0.data_ptr(), _stream()))
    return PackedBits(d0, None, 1, R, K)


def logical_from_tiled(packed, plane=0):
    """PackedBits (batch 1) -> int32 ``[R, ceil(K/32)]`` in the logical format."""
    src = packed.data if plane == 0 else packed.data2
    out = torch.empty((packed.rows, (packed.K + 31) // 32), dtype=torch.int32, device=src.device)
    with _on(src.device):
        _b.check(_b.lib().bgemm_logical_from_tiled(src.data_ptr(), packed.rows, packed.K, out.data_ptr(), _stream()))
    return out


def bgemm_packed_forward(w, x, mode=MODE_XOR, out_dtype=torch.int32, splitK=1, variant=VARIANT_AUTO, out=None,
                         scale=None, bits_out=None, next_zero_point=None):
    """GEMM on packed operands: ``out[b,n,m]`` for weight-side ``w`` (M rows) and activation-side
    ``x`` (N rows).  A batch of 1 on either side is shared across the other side's batch.

    ``scale=(sw, sa, bias)`` fuses the binary Linear's ``half(acc) * sw * sa (+ bias)``
    (bgemm_linear.py:482-484) into the store: ``sw`` [M], ``sa`` one element, ``bias`` [M] or None,
    all fp32 (fp32 output) or all fp16 (fp16 output), rounded step by step as torch does.

    ``bits_out=`` (a PackedBits of N rows x M bits from ``zeros_packed``, with ``scale``) stores no
    activations at all: the scaled output is centred by ``next_zero_point`` (a one-element tensor of the
    parameters' type, or None for 0), cast to fp16 and sign-packed as the next binary layer would do it, and
    those bits are written into ``bits_out``, which is returned."""
    if w.K != x.K:
        raise ValueError("K mismatch: %d vs %d" % (w.K, x.K))
    if (mode == MODE_BWTA) != x.ternary:
        raise ValueError("MODE_BWTA needs a ternary activation operand, the other modes a binary one")
    if w.ternary:
        raise ValueError("the weight side is binary")
    batch = max(w.batch, x.batch)
    if w.batch not in (1, batch) or x.batch not in (1, batch):
        raise ValueError("batch mismatch: %d vs %d" % (w.batch, x.batch))
    M, N, K = w.rows, x.rows, w.K
    dev = w.data.device
    _check_packed(w, "w")
    _check_packed(x, "x")
    if scale is not None:
        sw, sa, bias = scale
        out_dtype = sw.dtype
        if out_dtype not in (torch.float32, torch.half):
            raise TypeError("scales must be fp32 or fp16")
        for name, t, n in (("sw", sw, M), ("sa", sa, 1), ("bias", bias, M)):
            if t is None and name == "bias":
                continue
            _need_cuda(t, name)
            if t.dtype != out_dtype or t.numel() != n or not t.is_contiguous():
                raise ValueError("%s must be a contiguous %s tensor of %d elements" % (name, out_dtype, n))
        kind = OUT_F32_SCALED if out_dtype == torch.float32 else OUT_F16_SCALED
        if bits_out is not None:
            if bits_out.ternary or bits_out.rows != N or bits_out.K != M or bits_out.batch != batch:
                raise ValueError("bits_out must be a binary PackedBits of %d x %d rows x bits, batch %d" % (N, M, batch))
            _check_packed(bits_out, "bits_out")
            if next_zero_point is not None:
                _need_cuda(next_zero_point, "next_zero_point")
                if next_zero_point.dtype != out_dtype or next_zero_point.numel() != 1:
                    raise ValueError("next_zero_point must be a one-element %s tensor" % out_dtype)
            kind = OUT_BITS_F32 if out_dtype == torch.float32 else OUT_BITS_F16
    elif bits_out is not None:
        raise ValueError("bits_out needs scale=(sw, sa, bias)")
    elif out_dtype not in (torch.int32, torch.half):
        raise ValueError("out_dtype must be torch.int32 or torch.half")
    else:
        kind = OUT_F16 if out_dtype == torch.half else OUT_I32
    if out is None and bits_out is None:
        out = torch.empty((batch, N, M), dtype=out_dtype, device=dev)
    elif bits_out is None:
        # the kernel writes batch * N * M elements from out's first byte on
        _need_cuda(out, "out")
        if out.device != dev or out.dtype != out_dtype or not out.is_contiguous() or out.numel() != batch * N * M:
            raise ValueError("out must be a contiguous %s tensor of %d x %d x %d elements on %s"
                             % (out_dtype, batch, N, M, dev))
    L = _b.lib()
    with _on(dev):
        ws = cnt = None
        if splitK > 1:
            part_bytes, counter_bytes = _split_k_needs(L, (mode, batch, M, N, K, splitK, variant))
            if part_bytes:
                ws, cnt = _split_k_buffers(part_bytes, counter_bytes, dev)
        args = (mode, w.data.data_ptr(), x.data.data_ptr(), x.data2.data_ptr() if x.ternary else None,
                out.data_ptr() if bits_out is None else bits_out.data.data_ptr(), kind, batch, M, N, K,
                w.words if w.batch > 1 else 0, x.words if x.batch > 1 else 0,
                N * M if bits_out is None else bits_out.words, splitK, variant,
                ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
                cnt.data_ptr() if cnt is not None else None, cnt.numel() if cnt is not None else 0)
        counted = (scale is None and w.counts is not None and x.counts is not None and ws is None
                   and (variant & 0xff) != VARIANT_VALU)
        if counted:
            for name, p in (("w", w), ("x", x)):
                c = p.counts
                if (c.dtype != torch.int32 or tuple(c.shape) != (p.batch, p.rows) or not c.is_contiguous()
                        or c.device != dev):
                    raise ValueError("%s.counts must be a contiguous int32 tensor of shape (%d, %d) on %s"
                                     % (name, p.batch, p.rows, dev))
            _b.check(L.bgemm_packed_forward_counted(mode, args[1], args[2], w.counts.data_ptr(), x.counts.data_ptr(),
                                                    args[4], kind, batch, M, N, K, args[10], args[11], args[12],
                                                    variant, _stream()))
        elif scale is None:
            _b.check(L.bgemm_packed_forward(*args, _stream()))
        elif bits_out is not None:
            _b.check(L.bgemm_packed_forward_bits(*args, sw.data_ptr(), sa.data_ptr(),
                                                 bias.data_ptr() if bias is not None else None,
                                                 next_zero_point.data_ptr() if next_zero_point is not None else None,
                                                 _stream()))
            bits_out.counts = None       # row popcounts taken of the old contents no longer describe it
            return bits_out
        else:
            _b.check(L.bgemm_packed_forward_scaled(*args, sw.data_ptr(), sa.data_ptr(),
                                                   bias.data_ptr() if bias is not None else None, _stream()))
    return out


class DecodeChain:
    """A stack of dependent decode-shaped binary layers run as ONE launch (``bgemm_chain_forward``).

    ``layers`` is a list of ``(w, sw, sa, bias, next_zero_point)``: ``w`` a binary PackedBits of M x K bits (batch 1),
    ``sw`` [M], ``sa`` one element, ``bias`` [M] or None, ``next_zero_point`` one element or None, all of one dtype
    (fp16 or fp32).  Layer l + 1 reads the bits of ``half(y_l - next_zero_point_l)``, ``y_l = half(acc_l) * sw * sa (+ bias)``
    (tests/python/bgemm_linear.py:479-484): sign bits, or with ``mode=MODE_BWTA`` the ternary planes of its sign
    (:222-241).  ``__call__(x)`` takes the first layer's packed operand (up to 32 rows, 16 with BWTA) and returns the
    last layer's output: ``out_dtype`` torch.int32, torch.half (the rounded integer) or None for the scaled value
    of the parameters' type.  Calls on one GPU must not overlap in time (each holds every compute unit)."""

    def __init__(self, layers, mode=MODE_XOR, out_dtype=None, flags=0):
        if not layers:
            raise ValueError("a chain has at least one layer")
        self.mode, self.flags, self.layers = mode, flags, list(layers)
        w0, sw0 = layers[0][0], layers[0][1]
        self.device, self.pdtype = w0.data.device, sw0.dtype
        if self.pdtype not in (torch.float32, torch.half):
            raise TypeError("scales must be fp32 or fp16")
        self.out_dtype = self.pdtype if out_dtype is None else out_dtype
        if self.out_dtype not in (torch.int32, torch.half, torch.float32):
            raise ValueError("out_dtype must be torch.int32, torch.half or None (the parameters' type)")
        if out_dtype is None:
            self.kind = OUT_F32_SCALED if self.pdtype == torch.float32 else OUT_F16_SCALED
        elif out_dtype == torch.int32:
            self.kind = OUT_I32
        elif out_dtype == torch.half:
            self.kind = OUT_F16
        else:
            raise ValueError("a plain output is torch.int32 or torch.half")
        arr = (_b.ChainLayer * len(layers))()
        self._keep = []
        for l, (w, sw, sa, bias, zp) in enumerate(layers):
            if w.ternary or w.batch != 1:
                raise ValueError("layer %d: the weight side is one binary matrix" % l)
            _check_packed(w, "layer %d weights" % l)
            for name, t, n in (("sw", sw, w.rows), ("sa", sa, 1), ("bias", bias, w.rows), ("next_zero_point", zp, 1)):
                if t is None and name in ("bias", "next_zero_point"):
                    continue
                _need_cuda(t, name)
                if t.dtype != self.pdtype or t.numel() != n or not t.is_contiguous() or t.device != self.device:
                    raise ValueError("layer %d: %s must be a contiguous %s tensor of %d elements on %s" % (l, name, self.pdtype, n, self.device))
            arr[l].W_tiled, arr[l].sw, arr[l].sa = w.data.data_ptr(), sw.data_ptr(), sa.data_ptr()
            arr[l].bias = bias.data_ptr() if bias is not None else None
            arr[l].next_zero_point = zp.data_ptr() if zp is not None else None
            arr[l].M, arr[l].K = w.rows, w.K
            self._keep.append((w, sw, sa, bias, zp))
        self._host = arr
        raw = torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8)
        self._dev = raw.to(self.device)
        self._ws = {}

    def workspace(self, N):
        """The chain's workspace for N activation rows: zero-filled once, then left to the library."""
        ws = self._ws.get(N)
        if ws is None:
            need = _b.lib().bgemm_chain_workspace_bytes(self.mode, self._host, len(self.layers), N)
            if need == 0:
                _b.check(_b.EINVAL)          # the library has recorded why the chain cannot run
            ws = torch.zeros(need, dtype=torch.uint8, device=self.device)
            self._ws[N] = ws
        return ws

    def __call__(self, x, out=None):
        if (self.mode == MODE_BWTA) != x.ternary:
            raise ValueError("MODE_BWTA needs a ternary activation operand, the other modes a binary one")
        if x.batch != 1 or x.K != self.layers[0][0].K:
            raise ValueError("the operand must be one matrix of K = %d bits a row" % self.layers[0][0].K)
        _check_packed(x, "x")
        N, M = x.rows, self.layers[-1][0].rows
        ws = self.workspace(N)
        if out is None:
            out = torch.empty((N, M), dtype=self.out_dtype, device=self.device)
        elif out.dtype != self.out_dtype or out.numel() != N * M or not out.is_contiguous() or out.device != self.device:
            raise ValueError("out must be a contiguous %s tensor of %d x %d elements" % (self.out_dtype, N, M))
        with _on(self.device):
            _b.check(_b.lib().bgemm_chain_forward(self.mode, self._host, self._dev.data_ptr(), len(self.layers), x.data.data_ptr(),
                                                  x.data2.data_ptr() if x.ternary else None, N, out.data_ptr(), self.kind,
                                                  SRC_F32 if self.pdtype == torch.float32 else SRC_F16, ws.data_ptr(), ws.numel(),
                                                  self.flags, _stream()))
        return out

    def trace(self, N):
        """With flags & 4: microseconds since the launch's start at which block 0 (its first thread) had each layer's
        operand in LDS, the next layer's weights requested, its own K-tiles multiplied, the block's partial sums met and
        its outputs published, as an [n_layers, 5] tensor (of the last call with N rows)."""
        ws = self.workspace(N)
        t = ws[ws.numel() - (1 + 5 * 128) * 8:].view(torch.int64).cpu()
        return (t[1:1 + 5 * len(self.layers)] - t[0]).reshape(-1, 5).double() / 100.0

    def check(self, N):
        """Waits for the stream and raises if a launch of this chain gave up waiting (BGEMM_ETIMEOUT)."""
        with _on(self.device):
            _b.check(_b.lib().bgemm_chain_status(self.workspace(N).data_ptr(), _stream()))


# Opt-in cache of packed weights for the drop-in call.  The reference's interface takes fp16 weights
# on every call, so every call packs them again: at decode shapes that is most of the time (reading
# 90 MB of fp16 to produce 5.6 MB of bits).  With the cache on, a weight tensor that is the same object,
# at the same version counter, as on an earlier call is not packed again.  Off by default because the
# version counter only sees writes made through torch: memory changed behind torch's back (another
# library writing through the raw pointer) would go unnoticed.
_weight_cache = collections.OrderedDict()
_weight_cache_entries = 0


def set_weight_cache(entries):
    """Keep the packed form of up to `entries` weight tensors seen by bgemm_linear_forward_cuda (0 = off, the
    default).  An entry is used again only for the very same tensor object with an unchanged version counter."""
    global _weight_cache_entries
    _weight_cache_entries = max(0, int(entries))
    while len(_weight_cache) > _weight_cache_entries:
        _weight_cache.popitem(last=False)


def _cached_packed_weight(w):
    key = id(w)
    hit = _weight_cache.get(key)
    if hit is not None and hit[0]() is w and hit[1] == w._version and hit[2] == w.data_ptr():
        _weight_cache.move_to_end(key)
        return hit[3]
    packed = pack_sign(w)
    _weight_cache[key] = (weakref.ref(w), w._version, w.data_ptr(), packed)
    _weight_cache.move_to_end(key)
    while len(_weight_cache) > _weight_cache_entries:
        _weight_cache.popitem(last=False)
    return packed


_decode_shapes = {}       # (mode, M, N, K) -> does the decode kernel take unpacked activations of this shape


def decode_linear_launch(w, x, sw, sa, bias, zero_point):
    """The one-launch binary Linear of a decode step with every check left to the caller (the layers validate
    their parameters once, not on every token): ``x`` is a contiguous [N<=4, K] CUDA tensor of the parameters'
    dtype (fp16 or fp32), ``sw``/``sa``/``bias``/``zero_point`` contiguous tensors of that dtype (bias may be
    None), the shape one that ``bgemm_packed_weight_forward_supported`` accepts.  Returns [N, M]."""
    dt = x.dtype
    f32 = dt == torch.float32
    out = torch.empty((x.shape[0], w.rows), dtype=dt, device=x.device)
    with _on(x.device):
        _b.check(_b.lib().bgemm_packed_weight_forward(
            MODE_XOR, w.data.data_ptr(), x.data_ptr(), SRC_F32 if f32 else SRC_F16, x.shape[1], zero_point.data_ptr(),
            out.data_ptr(), OUT_F32_SCALED if f32 else OUT_F16_SCALED, w.rows, x.shape[0], w.K, VARIANT_AUTO,
            sw.data_ptr(), sa.data_ptr(), bias.data_ptr() if bias is not None else None, None, _stream()))
    return out


def decode_shape_supported(mode, M, N, K):
    one_launch = _decode_shapes.get((mode, M, N, K))
    if one_launch is None:
        one_launch = _decode_shapes[(mode, M, N, K)] = bool(N and M and K and _b.lib().bgemm_packed_weight_forward_supported(mode, M, N, K))
    return one_launch


def bgemm_packed_weight_forward(w, x, mode=MODE_XOR, out_dtype=torch.int32, scale=None, x_zero_point=None,
                                variant=VARIANT_AUTO):
    """Prepacked weights ``w`` (M rows) x activations ``x`` as they are, fp16 or fp32 ``[N,K]`` -> ``[N,M]``.

    For the few rows of a decode step (N <= 4) this is ONE launch: the kernel forms the
    activation bits itself (``MODE_BWTA``: the ternary planes of sign(x); the other modes: sign bits of ``x``
    or, with ``x_zero_point``, of ``(x - x_zero_point).to(torch.half)``).  Larger batches go through the pack
    kernel and the packed entry point: same results either way.  ``scale`` as in bgemm_packed_forward."""
    _need_cuda(x, "x")
    if x.dim() != 2 or x.shape[1] != w.K:
        raise ValueError("x must be [N, %d], got %s" % (w.K, tuple(x.shape)))
    if w.ternary or w.batch != 1:
        raise ValueError("the weight side is one binary matrix")
    if x.dtype not in (torch.half, torch.float32):
        raise TypeError("activations must be fp16 or fp32, got %s" % x.dtype)
    ternary = mode == MODE_BWTA
    if ternary and x_zero_point is not None:
        raise ValueError("a zero point is only taken by the sign modes")
    if x_zero_point is not None:
        _need_cuda(x_zero_point, "x_zero_point")
        if x_zero_point.numel() != 1:
            raise TypeError("x_zero_point must be a one-element tensor")
        x_zero_point = x_zero_point.detach().to(x.dtype)
    N, K, M = x.shape[0], w.K, w.rows
    L = _b.lib()
    if not decode_shape_supported(mode, M, N, K) or variant == VARIANT_VALU:
        xp = pack_ternary(x) if ternary else pack_sign(x, zero_point=x_zero_point)
        return bgemm_packed_forward(w, xp, mode, out_dtype, 8, variant, scale=scale)[0]
    if x.stride(1) != 1 or x.stride(0) < K:
        x = x.contiguous()
    sw = sa = bias = None
    if scale is not None:
        sw, sa, bias = scale
        out_dtype = sw.dtype
        if out_dtype not in (torch.float32, torch.half):
            raise TypeError("scales must be fp32 or fp16")
        for name, t, n in (("sw", sw, M), ("sa", sa, 1), ("bias", bias, M)):
            if t is None and name == "bias":
                continue
            _need_cuda(t, name)
            if t.dtype != out_dtype or t.numel() != n or not t.is_contiguous():
                raise ValueError("%s must be a contiguous %s tensor of %d elements" % (name, out_dtype, n))
        kind = OUT_F32_SCALED if out_dtype == torch.float32 else OUT_F16_SCALED
    elif out_dtype not in (torch.int32, torch.half):
        raise ValueError("out_dtype must be torch.int32 or torch.half")
    else:
        kind = OUT_F16 if out_dtype == torch.half else OUT_I32
    out = torch.empty((N, M), dtype=out_dtype, device=x.device)
    with _on(x.device):
        _b.check(L.bgemm_packed_weight_forward(
            mode, w.data.data_ptr(), x.data_ptr(), SRC_F32 if x.dtype == torch.float32 else SRC_F16, x.stride(0),
            x_zero_point.data_ptr() if x_zero_point is not None else None, out.data_ptr(), kind, M, N, K, variant,
            sw.data_ptr() if sw is not None else None, sa.data_ptr() if sa is not None else None,
            bias.data_ptr() if bias is not None else None, None, _stream()))
    return out


def bgemm_linear_forward_cuda(in_feats, weights, splitK=1, INSTR=1):
    """Computes BGEMM: half ``in_feats [N,K]``, half ``weights [M,K]`` -> half ``[N,M]``.

    INSTR 0 = and.popc, 1 = K - 2*xor.popc, 2 = attention ({0,1} weights side by sign bit clear).
    Unlike the reference (fp6_linear.cu:288-290, 568-576) any N, M, K >= 1 is accepted, inputs need
    not be contiguous, and the launch goes to the current stream."""
    _need_cuda(in_feats, "in_feats")
    _need_cuda(weights, "weights")
    if in_feats.dim() != 2 or weights.dim() != 2:
        raise ValueError("in_feats and weights must be 2-D")
    if in_feats.dtype != torch.half or weights.dtype != torch.half:
        raise TypeError("in_feats and weights must be torch.half")   # data_ptr<at::Half> in the reference
    if in_feats.shape[1] != weights.shape[1]:
        raise ValueError("K mismatch: in_feats %s vs weights %s" % (tuple(in_feats.shape), tuple(weights.shape)))
    if INSTR not in (AND_POP, XOR_POP, ATTN_MM):
        raise ValueError("INSTR must be 0 (and), 1 (xor) or 2 (attn), got %r" % (INSTR,))
    if int(splitK) < 1:
        raise ValueError("splitK must be at least 1, got %r" % (splitK,))
    if _weight_cache_entries and weights.is_contiguous() and weights.numel() and in_feats.numel():
        # the same arithmetic on packed operands: the weights' bits come from the cache
        out = bgemm_packed_forward(_cached_packed_weight(weights), pack_sign(in_feats), int(INSTR), torch.half,
                                   int(splitK))
        return out[0]
    x, w = in_feats.contiguous(), weights.contiguous()
    N, K = x.shape
    M = w.shape[0]
    out = torch.empty((N, M), dtype=torch.half, device=x.device)
    L = _b.lib()
    with _on(x.device):
        ws = torch.empty(max(L.bgemm_f16_workspace_bytes(M, N, K, splitK), 1), dtype=torch.uint8, device=x.device)
        _b.check(L.bgemm_f16_forward(w.data_ptr(), x.data_ptr(), out.data_ptr(), M, N, K,
                                     ws.data_ptr(), ws.numel(), int(splitK), int(INSTR), _stream()))
    return out


# ---- prepacked operands on disk -----------------------------------------------------------------
# The reference has no binary prepack format (its TODO list asks for one, README.md:25-33).  A file is
# a 64-byte little-endian header followed by the tiled words of plane 0 and, for ternary operands,
# plane 1: magic "BGEMMPK1", version of the tiled layout (_lib.LAYOUT_VERSION, which changes only when the
# layout does, not with the C ABI), planes, batch, rows, K, words per matrix.
_PK_MAGIC = b"BGEMMPK1"
_PK_HEADER = struct.Struct("<8sIIqqqq16x")


def save_packed(path, packed):
    """Writes a PackedBits (e.g. prepacked weights) to `path`."""
    head = _PK_HEADER.pack(_PK_MAGIC, _b.LAYOUT_VERSION, 2 if packed.ternary else 1, packed.batch, packed.rows,
                           packed.K, packed.words)
    with open(path, "wb") as f:
        f.write(head)
        f.write(packed.data.contiguous().cpu().numpy().tobytes())
        if packed.ternary:
            f.write(packed.data2.contiguous().cpu().numpy().tobytes())


def read_packed_header(path):
    """(planes, batch, rows, K, words) of a file written by save_packed; raises ValueError on anything else."""
    with open(path, "rb") as f:
        raw = f.read(_PK_HEADER.size)
    if len(raw) != _PK_HEADER.size:
        raise ValueError("%s: too short for a packed-operand header" % path)
    magic, version, planes, batch, rows, K, words = _PK_HEADER.unpack(raw)
    if magic != _PK_MAGIC:
        raise ValueError("%s: not a packed-operand file" % path)
    if version != _b.LAYOUT_VERSION:
        raise ValueError("%s: tiled layout version %d, this library reads %d: pack the weights again" %
                         (path, version, _b.LAYOUT_VERSION))
    if planes not in (1, 2) or batch < 1 or rows < 1 or K < 1 or words != ((rows + 31) // 32) * ((K + 255) // 256) * 256:
        raise ValueError("%s: inconsistent header" % path)
    return planes, batch, rows, K, words


def load_packed(path, device="cuda"):
    """Reads a file written by save_packed back into a PackedBits on `device`."""
    import numpy as np
    planes, batch, rows, K, words = read_packed_header(path)
    n = batch * words
    arr = np.fromfile(path, dtype=np.int32, offset=_PK_HEADER.size)
    if arr.size != planes * n:
        raise ValueError("%s: %d words of payload, header says %d" % (path, arr.size, planes * n))
    d0 = torch.from_numpy(arr[:n].reshape(batch, words).copy()).to(device)
    d1 = torch.from_numpy(arr[n:].reshape(batch, words).copy()).to(device) if planes == 2 else None
    return PackedBits(d0, d1, batch, rows, K)


def _fp6_only(*_a, **_k):
    raise NotImplementedError("FP6 entry points of the reference extension are outside this library")


linear_forward_cuda = weight_prepacking_cpu = weight_dequant_cpu = _fp6_only
