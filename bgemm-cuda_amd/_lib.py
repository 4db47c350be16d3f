"""ctypes binding of libbgemm_mi355x.so (the C ABI declared in include/bgemm_mi355x.h).

The library must have been built (``python _build.py`` or ``__graft_entry__.build()``);
there is no CPU fallback: a missing library raises ImportError.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "libbgemm_mi355x.so")

OK, EINVAL, ENULL, EWORKSPACE, ELAUNCH, EALIGN, ETIMEOUT = 0, -1, -2, -3, -4, -5, -6
MODE_AND, MODE_XOR, MODE_ATTN, MODE_BWTA, MODE_ATTN_X = 0, 1, 2, 3, 4
OUT_I32, OUT_F16, OUT_F32_SCALED, OUT_F16_SCALED, OUT_BITS_F32, OUT_BITS_F16 = 0, 1, 2, 3, 4, 5
SRC_F16, SRC_F32 = 0, 1
ABI_VERSION = 10
LAYOUT_VERSION = 6     # of the tiled operand layout, written into packed files; changes only when the layout does
STATIC_SCRATCH_BYTES = 32 << 20      # BGEMM_STATIC_SCRATCH_BYTES
VARIANT_AUTO, VARIANT_VALU, VARIANT_MFMA, VARIANT_MFMA_F4 = 0, 1, 2, 3
# BGEMM_KERNEL_*: what bgemm_packed_kernel_id() returns and force_kernel() takes
KERNEL_MFMA_256x256, KERNEL_MFMA_128x128, KERNEL_MFMA_64x128, KERNEL_MFMA_32x128, KERNEL_MFMA_256x128 = 0, 1, 2, 3, 4
KERNEL_MFMA_32x256, KERNEL_MFMA_64x64, KERNEL_MFMA_128x64, KERNEL_MFMA_128x256T = 5, 6, 7, 8
KERNEL_SKINNY_STREAM, KERNEL_SKINNY_SPLITK, KERNEL_SKINNY_QUAD, KERNEL_SKINNY_POPC, KERNEL_VALU = 16, 17, 18, 19, 32


def force_kernel(kernel_id, family=VARIANT_AUTO):
    """BGEMM_FORCE_KERNEL(id) | family: a `variant` that runs the named kernel whatever the shape (tests, benchmarks)."""
    return ((kernel_id + 1) << 8) | family


_i64, _p, _int, _sz = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t

# symbol -> (restype, argtypes); mirrors include/bgemm_mi355x.h one to one
SIGNATURES = {
    "bgemm_last_error": (ctypes.c_char_p, []),
    "bgemm_abi_version": (_int, []),
    "bgemm_tiled_words": (_i64, [_i64, _i64]),
    "bgemm_pack_sign_f16": (_int, [_p, _i64, _i64, _i64, _p, _p]),
    "bgemm_pack_sign_f16_logical": (_int, [_p, _i64, _i64, _i64, _p, _p]),
    "bgemm_pack_sign_centered": (_int, [_p, _int, _i64, _i64, _i64, _p, _p, _p]),
    "bgemm_pack_ternary_f16": (_int, [_p, _i64, _i64, _i64, _p, _p, _p]),
    "bgemm_tile_from_logical": (_int, [_p, _i64, _i64, _p, _p]),
    "bgemm_logical_from_tiled": (_int, [_p, _i64, _i64, _p, _p]),
    "bgemm_packed_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64, _int, _int]),
    "bgemm_packed_counter_bytes": (_sz, [_int, _i64, _i64, _i64, _i64, _int, _int]),
    "bgemm_packed_forward": (_int, [_int, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                    _int, _int, _p, _sz, _p, _sz, _p]),
    "bgemm_packed_kernel_id": (_int, [_int, _int, _i64, _i64, _i64, _i64, _int, _int]),
    "bgemm_row_popcounts": (_int, [_p, _i64, _i64, _i64, _i64, _p, _p]),
    "bgemm_packed_forward_counted": (_int, [_int, _p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                            _int, _p]),
    "bgemm_packed_forward_scaled": (_int, [_int, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                           _int, _int, _p, _sz, _p, _sz, _p, _p, _p, _p]),
    "bgemm_packed_forward_bits": (_int, [_int, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                         _int, _int, _p, _sz, _p, _sz, _p, _p, _p, _p, _p]),
    "bgemm_pack_sign_f16_transposed": (_int, [_p, _i64, _i64, _i64, _i64, _i64, _p, _p]),
    "bgemm_pack_batched": (_int, [_p, _int, _int, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _p, _p, _p]),
    "bgemm_pack_transposed_batched": (_int, [_p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _p, _p]),
    "bgemm_packed_weight_forward_supported": (_int, [_int, _i64, _i64, _i64]),
    "bgemm_packed_weight_forward": (_int, [_int, _p, _p, _int, _i64, _p, _p, _int, _i64, _i64, _i64, _int, _p, _p, _p, _p, _p]),
    "bgemm_f16_workspace_bytes": (_sz, [_i64, _i64, _i64, _int]),
    "bgemm_f16_forward": (_int, [_p, _p, _p, _i64, _i64, _i64, _p, _sz, _int, _int, _p]),
    "bgemm_f16_forward_static": (_int, [_p, _p, _p, _i64, _i64, _i64, _int, _int, _p]),
    "bgemm_chain_workspace_bytes": (_sz, [_int, _p, _int, _i64]),
    "bgemm_chain_forward": (_int, [_int, _p, _p, _int, _p, _p, _i64, _p, _int, _int, _p, _sz, _int, _p]),
    "bgemm_chain_status": (_int, [_p, _p]),
}


class ChainLayer(ctypes.Structure):
    """bgemm_chain_layer: one layer of a chain; every pointer is a device pointer."""
    _fields_ = [("W_tiled", _p), ("sw", _p), ("bias", _p), ("sa", _p), ("next_zero_point", _p),
                ("M", _i64), ("K", _i64), ("reserved", _i64)]

_lib = None


def lib():
    """Loads the shared library once and types every entry point."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise ImportError("%s is missing: build it with `python %s`" %
                              (SO_PATH, os.path.join(_HERE, "_build.py")))
        L = ctypes.CDLL(SO_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        if L.bgemm_abi_version() != ABI_VERSION:
            raise ImportError("%s is ABI version %d, this binding needs %d: rebuild it" %
                              (SO_PATH, L.bgemm_abi_version(), ABI_VERSION))
        _lib = L
    return _lib


class BgemmError(RuntimeError):
    pass


def check(rc):
    """Turns a negative status into the Python exception the reference's asserts map to."""
    if rc == OK:
        return
    msg = lib().bgemm_last_error().decode() or "error %d" % rc
    if rc in (EINVAL, ENULL, EALIGN, EWORKSPACE):
        raise ValueError(msg)
    raise BgemmError(msg)
