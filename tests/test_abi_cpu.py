"""The C-ABI library loads without a GPU, exports every symbol the header declares, and
rejects bad arguments from the host side (no kernel is launched by any call here)."""
import ctypes
import os
import re
import shutil
import subprocess

import pytest

import _lib

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "bgemm_mi355x.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bgemm_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported():
    names = declared_functions()
    assert len(names) >= 12
    L = ctypes.CDLL(_lib.SO_PATH)
    for n in names:
        assert hasattr(L, n), "missing export: %s" % n
    # the binding table and the header list the same entry points
    assert sorted(_lib.SIGNATURES) == names


def test_header_is_plain_c_and_a_c_program_links(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 and as C++11 with -pedantic, and a C program built against it
    links with the library and calls a host-only entry point (what a cgo / JNI / FFI binding does first)."""
    gcc = shutil.which("gcc")
    if not gcc:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    src.write_text('#include <stdio.h>\n#include "bgemm_mi355x.h"\n'
                   'int main(void) { printf("%d %lld\\n", bgemm_abi_version(), (long long)bgemm_tiled_words(33, 257)); return 0; }\n')
    inc = os.path.dirname(HEADER)
    for cc, std in ((gcc, ["-std=c99"]), (shutil.which("g++") or gcc, ["-std=c++11", "-x", "c++"])):
        subprocess.check_call([cc] + std + ["-Wall", "-Wextra", "-Werror", "-pedantic", "-I", inc, "-fsyntax-only", str(src)])
    exe = tmp_path / "use_header"
    libdir = os.path.dirname(_lib.SO_PATH)
    subprocess.check_call([gcc, "-std=c99", "-I", inc, str(src), "-o", str(exe), "-L", libdir, "-l:" + os.path.basename(_lib.SO_PATH),
                           "-Wl,-rpath," + libdir, "-Wl,-rpath-link,/opt/rocm/lib"])
    out = subprocess.check_output([str(exe)], env=dict(os.environ, LD_LIBRARY_PATH="/opt/rocm/lib:" + os.environ.get("LD_LIBRARY_PATH", "")))
    assert out.split() == [str(_lib.ABI_VERSION).encode(), b"1024"]


def test_layout_sizes():
    L = _lib.lib()
    assert L.bgemm_abi_version() == _lib.ABI_VERSION == 10
    assert L.bgemm_tiled_words(1, 1) == 256
    assert L.bgemm_tiled_words(32, 256) == 256
    assert L.bgemm_tiled_words(33, 257) == 4 * 256
    assert L.bgemm_tiled_words(11008, 4096) == 11008 * 4096 // 32
    assert L.bgemm_tiled_words(0, 128) == 0
    # splitK is an upper bound, and only the VALU family (variant 1) splits K across blocks, through a workspace:
    # the matrix-core family splits K among the waves of a block for outputs of few tiles and not at all otherwise
    assert L.bgemm_packed_workspace_bytes(1, 1, 64, 256, 16384, 1, 1) == 0
    assert L.bgemm_packed_workspace_bytes(1, 1, 64, 256, 16384, 4, 1) >= 2 * 64 * 256 * 4
    assert L.bgemm_packed_counter_bytes(1, 1, 64, 256, 16384, 4, 1) >= 4
    assert L.bgemm_packed_counter_bytes(1, 1, 64, 256, 16384, 1, 1) == 0
    assert L.bgemm_packed_workspace_bytes(1, 1, 64, 256, 1024, 4, 1) == 0            # K too short to split
    assert L.bgemm_packed_workspace_bytes(1, 1, 8192, 8192, 65536, 8, 1) == 0        # enough tiles without
    assert L.bgemm_packed_workspace_bytes(3, 2, 100, 270, 40000, 3, 1) >= 2 * 3 * 100 * 270 * 4
    for variant in (0, 2, 3):
        for shape in ((1, 1, 64, 256, 16384), (3, 1, 64, 256, 16384), (1, 1, 11008, 16, 4096), (1, 1, 4096, 128, 4096),
                      (1, 1, 128, 128, 65536), (3, 2, 100, 270, 40000), (1, 1, 8192, 8192, 65536)):
            assert L.bgemm_packed_workspace_bytes(*shape, 8, variant) == 0
            assert L.bgemm_packed_counter_bytes(*shape, 8, variant) == 0
    assert L.bgemm_f16_workspace_bytes(64, 32, 256, 1) >= (64 + 32) * 256 // 8


@pytest.mark.parametrize("kwargs, code", [
    (dict(mode=7), _lib.EINVAL),
    (dict(out_dtype=5), _lib.EINVAL),
    (dict(variant=4), _lib.EINVAL),
    (dict(variant=_lib.force_kernel(9)), _lib.EINVAL),                                   # no such kernel
    (dict(variant=_lib.force_kernel(_lib.KERNEL_MFMA_64x64, _lib.VARIANT_VALU)), _lib.EINVAL),   # the VALU design has one kernel
    (dict(variant=_lib.force_kernel(_lib.KERNEL_SKINNY_STREAM), batch=70000, strideC=64 * 256), _lib.EINVAL),
    (dict(M=-1), _lib.EINVAL),
    (dict(splitK=0), _lib.EINVAL),
    (dict(K=1 << 24), _lib.EINVAL),
    (dict(out=None), _lib.ENULL),
    (dict(W=None), _lib.ENULL),
    (dict(mode=3), _lib.ENULL),                       # BWTA without the second plane
    (dict(W=0x1008), _lib.EALIGN),
    (dict(out=0x3002), _lib.EALIGN),                  # int32 output on a 2-byte boundary
    (dict(out=0x3001, out_dtype=1), _lib.EALIGN),     # fp16 output on an odd address
    # the VALU family on 64 x 256 outputs with a long K splits K across blocks
    (dict(variant=1, splitK=2), _lib.EWORKSPACE),                # no workspace given
    (dict(variant=1, splitK=2, ws=0x10000, ws_bytes=1 << 24), _lib.EWORKSPACE),            # no counters given
    (dict(variant=1, splitK=2, ws=0x10000, ws_bytes=16, cnt=0x20000, cnt_bytes=4096), _lib.EWORKSPACE),
    (dict(variant=1, splitK=2, ws=0x10000, ws_bytes=1 << 24, cnt=0x20000, cnt_bytes=0), _lib.EWORKSPACE),
    (dict(variant=1, splitK=2, ws=0x10004, ws_bytes=1 << 24, cnt=0x20000, cnt_bytes=4096), _lib.EALIGN),
    (dict(strideW=2), _lib.EINVAL),
])
def test_packed_forward_rejects(kwargs, code):
    L = _lib.lib()
    a = dict(mode=1, W=0x1000, X=0x2000, X2=None, out=0x3000, out_dtype=0, batch=1, M=64, N=256, K=16384,
             strideW=0, strideX=0, strideC=0, splitK=1, variant=0, ws=None, ws_bytes=0, cnt=None, cnt_bytes=0,
             stream=None)
    a.update(kwargs)
    rc = L.bgemm_packed_forward(a["mode"], a["W"], a["X"], a["X2"], a["out"], a["out_dtype"], a["batch"], a["M"],
                                a["N"], a["K"], a["strideW"], a["strideX"], a["strideC"], a["splitK"], a["variant"],
                                a["ws"], a["ws_bytes"], a["cnt"], a["cnt_bytes"], a["stream"])
    assert rc == code
    assert L.bgemm_last_error()            # a message was recorded
    with pytest.raises(ValueError):
        _lib.check(rc)


def test_dispatch_of_the_benchmark_configurations():
    """Which kernel each benchmark configuration runs (what the profiles and the bench lines are about):
    the query is host code and needs no GPU."""
    B = _lib
    kid = lambda mode, *rest: B.lib().bgemm_packed_kernel_id(mode, B.OUT_I32, *rest)
    MODE_XOR, MODE_BWTA, MODE_ATTN_X, VARIANT_AUTO, VARIANT_VALU, force_kernel = (
        B.MODE_XOR, B.MODE_BWTA, B.MODE_ATTN_X, B.VARIANT_AUTO, B.VARIANT_VALU, B.force_kernel)
    TILES = (0, 1, 2, 3, 4, 5, 6, 7)
    A = VARIANT_AUTO
    assert kid(MODE_XOR, 1, 8192, 8192, 8192, 1, A) == B.KERNEL_MFMA_256x128
    assert kid(MODE_XOR, 1, 8192, 8192, 16384, 1, A) == B.KERNEL_MFMA_256x128
    assert kid(MODE_XOR, 1, 8192, 8192, 32768, 1, A) == B.KERNEL_MFMA_256x256
    assert kid(MODE_XOR, 1, 11008, 768, 4096, 1, A) == B.KERNEL_MFMA_128x128     # 258 blocks of 256 x 128: one too many
    assert kid(MODE_BWTA, 1, 11008, 128, 4096, 1, A) == B.KERNEL_MFMA_32x256
    assert kid(MODE_XOR, 1, 11008, 512, 8192, 1, A) == B.KERNEL_MFMA_256x128     # 172 blocks: 0.67 a unit is enough
    assert kid(MODE_XOR, 1, 11008, 640, 8192, 1, A) == B.KERNEL_MFMA_128x128     # 258 again
    assert kid(MODE_XOR, 1, 8192, 768, 16384, 1, A) == B.KERNEL_MFMA_256x128
    assert kid(MODE_XOR, 1, 8192, 512, 16384, 1, A) == B.KERNEL_MFMA_128x128     # 4096 pieces: past the four-pieces kernel's 2048
    assert kid(MODE_XOR, 1, 6144, 384, 11008, 1, A) == B.KERNEL_MFMA_128x128     # 144 blocks on a long K
    assert kid(MODE_BWTA, 1, 11008, 64, 4096, 1, A) == B.KERNEL_SKINNY_SPLITK
    assert kid(MODE_XOR, 1, 8192, 2048, 4096, 1, A) == B.KERNEL_MFMA_256x128
    assert kid(MODE_XOR, 1, 8192, 2048, 16384, 4, A) == B.KERNEL_MFMA_256x128
    assert kid(MODE_XOR, 1, 8192, 256, 16384, 1, A) == B.KERNEL_SKINNY_QUAD
    assert kid(MODE_ATTN_X, 192, 64, 512, 512, 1, A) == B.KERNEL_MFMA_64x64
    assert kid(MODE_ATTN_X, 384, 64, 512, 512, 1, A) == B.KERNEL_MFMA_128x64
    assert kid(MODE_XOR, 1, 4096, 2048, 4096, 1, A) == B.KERNEL_MFMA_128x128     # 256 blocks of 256 x 128 on 16 K-tiles: the next tile down
    assert kid(MODE_XOR, 1, 4096, 2048, 8192, 1, A) == B.KERNEL_MFMA_256x128
    # a short K with a 2-byte output takes the tile with 512-byte rows
    assert B.lib().bgemm_packed_kernel_id(MODE_XOR, B.OUT_F16, 192, 512, 512, 64, 1, A) == B.KERNEL_MFMA_32x256
    assert kid(MODE_XOR, 192, 512, 512, 64, 1, A) == B.KERNEL_MFMA_128x128
    assert kid(MODE_XOR, 48, 2048, 1024, 64, 1, A) == B.KERNEL_MFMA_32x256      # 403 MB of int32 from one K-tile
    # int32 rows of a power of two in bytes on a short K: many 32-row blocks instead of few large ones in step
    assert kid(MODE_XOR, 1, 2048, 4096, 1024, 1, A) == B.KERNEL_MFMA_32x256
    assert kid(MODE_XOR, 1, 2000, 4000, 1024, 1, A) == B.KERNEL_MFMA_128x128
    assert kid(MODE_XOR, 1, 2048, 4096, 2048, 1, A) == B.KERNEL_MFMA_128x128
    # 256 x 128: from 132 blocks on 16 K-tiles or more, but not between one block a unit and one and a half
    assert kid(MODE_XOR, 1, 4352, 1024, 8192, 1, A) == B.KERNEL_MFMA_256x128     # 136 blocks
    assert kid(MODE_XOR, 1, 2560, 1536, 8192, 1, A) == B.KERNEL_MFMA_128x128     # 120: every 128 x 128 block has a unit to itself
    assert kid(MODE_XOR, 1, 6144, 2048, 16384, 1, A) == B.KERNEL_MFMA_128x128    # 384
    assert kid(MODE_XOR, 1, 6656, 2048, 16384, 1, A) == B.KERNEL_MFMA_256x128    # 416
    assert kid(MODE_XOR, 1, 9216, 256, 4096, 1, A) == B.KERNEL_MFMA_128x128      # 144 blocks from 16 K-tiles on
    assert kid(MODE_XOR, 1, 9216, 256, 2048, 1, A) == B.KERNEL_MFMA_32x128
    # four to seven K-tiles: split-K in the block for up to two activation tile rows
    assert kid(MODE_XOR, 1, 11008, 40, 1792, 1, A) == B.KERNEL_SKINNY_SPLITK
    assert kid(MODE_XOR, 1, 1024, 384, 1024, 1, A) == B.KERNEL_MFMA_32x128
    assert kid(MODE_XOR, 1, 4096, 128, 784, 1, A) == B.KERNEL_SKINNY_SPLITK       # four tile rows, 512 pieces: an MLP's first layer
    assert kid(MODE_XOR, 1, 6144, 64, 1024, 1, A) == B.KERNEL_MFMA_32x128        # 384 pieces on four K-tiles
    # two bit planes: four pieces a block for one round of blocks, then the pipelined 32 x 256 and 128 x 128 tiles
    assert kid(MODE_BWTA, 1, 8192, 128, 8192, 1, A) == B.KERNEL_SKINNY_QUAD      # 512 blocks
    assert kid(MODE_BWTA, 1, 8192, 160, 8192, 1, A) == B.KERNEL_MFMA_32x256      # 640
    assert kid(MODE_BWTA, 1, 11008, 96, 4096, 1, A) == B.KERNEL_MFMA_32x256      # 129 blocks of 32 x 256
    assert kid(MODE_BWTA, 1, 11008, 256, 8192, 1, A) == B.KERNEL_MFMA_128x128    # 172 blocks of 128 x 128
    # the signed tile takes a ternary operand from more than half a 128 x 256 block a unit on, on the fp4 engine only
    assert kid(MODE_BWTA, 1, 11008, 320, 11008, 1, A) == B.KERNEL_MFMA_128x256T  # 129 blocks
    assert kid(MODE_BWTA, 1, 11008, 320, 11008, 1, B.VARIANT_MFMA) == B.KERNEL_MFMA_32x256    # int8 engine: 258 blocks of 128 x 128, between one a unit and one and a quarter
    assert kid(MODE_BWTA, 1, 22016, 2048, 4096, 1, A) == B.KERNEL_MFMA_128x256T
    assert kid(MODE_BWTA, 1, 4096, 1024, 11008, 1, A) == B.KERNEL_MFMA_128x128   # 128 blocks of the signed tile: level, stays
    assert kid(MODE_BWTA, 1, 8192, 8192, 256, 1, A) != B.KERNEL_MFMA_128x256T    # one K-tile
    assert kid(MODE_ATTN_X, 24, 64, 512, 512, 1, A) == B.KERNEL_MFMA_64x64
    assert kid(MODE_BWTA, 1, 11008, 1, 4096, 8, A) == B.KERNEL_SKINNY_POPC
    assert kid(MODE_BWTA, 1, 11008, 16, 4096, 8, A) == B.KERNEL_SKINNY_SPLITK
    assert kid(MODE_BWTA, 64, 11008, 16, 4096, 1, A) == B.KERNEL_SKINNY_STREAM
    assert kid(MODE_XOR, 1, 4096, 128, 4096, 1, VARIANT_VALU) == B.KERNEL_VALU
    assert kid(MODE_XOR, 70000, 40, 8, 300, 1, A) in TILES        # a batch beyond the decode kernels' grid
    assert kid(MODE_XOR, 1, 64, 64, 64, 1, force_kernel(B.KERNEL_MFMA_256x256)) == B.KERNEL_MFMA_256x256
    assert kid(MODE_XOR, 1, 64, 64, 64, 1, force_kernel(9)) == B.EINVAL    # no such kernel
    assert kid(MODE_XOR, 1, 64, 64, 64, 1, force_kernel(B.KERNEL_MFMA_64x64, VARIANT_VALU)) == B.EINVAL
    assert kid(9, 1, 64, 64, 64, 1, A) == B.EINVAL and kid(MODE_XOR, 1, 64, 0, 64, 1, A) == B.EINVAL


def test_counted_entry_points_reject_without_touching_the_gpu():
    """Argument checks of bgemm_row_popcounts and bgemm_packed_forward_counted are host code: every rejection
    below returns before any launch."""
    B, L = _lib, _lib.lib()
    buf = (ctypes.c_char * 64)()
    p = ctypes.addressof(buf) + (-ctypes.addressof(buf)) % 16
    assert L.bgemm_row_popcounts(None, 1, 32, 256, 0, p, None) == B.ENULL
    assert L.bgemm_row_popcounts(p, 1, 32, 256, 0, None, None) == B.ENULL
    assert L.bgemm_row_popcounts(p + 4, 1, 32, 256, 0, p, None) == B.EALIGN
    assert L.bgemm_row_popcounts(p, 1, 32, 1 << 24, 0, p, None) == B.EINVAL
    assert L.bgemm_row_popcounts(p, 2, 32, 256, 4, p, None) == B.EINVAL              # batch stride below one operand
    assert L.bgemm_row_popcounts(p, 0, 32, 256, 0, None, None) == 0                   # nothing to count
    fwd = lambda mode, cw, cx, variant: L.bgemm_packed_forward_counted(mode, p, p, cw, cx, p, B.OUT_I32, 1, 32, 32, 256,
                                                                        0, 0, 1024, variant, None)
    assert fwd(B.MODE_XOR, None, p, B.VARIANT_AUTO) == B.ENULL
    assert fwd(B.MODE_XOR, p, p + 2, B.VARIANT_AUTO) == B.EALIGN
    assert fwd(B.MODE_BWTA, p, p, B.VARIANT_AUTO) in (B.EINVAL, B.ENULL)             # two bit planes: not this entry point
    assert fwd(B.MODE_XOR, p, p, B.VARIANT_VALU) == B.EINVAL
    assert L.bgemm_packed_forward_counted(B.MODE_XOR, p, p, p, p, p, B.OUT_F32_SCALED, 1, 32, 32, 256, 0, 0, 1024,
                                          B.VARIANT_AUTO, None) == B.EINVAL


def test_decode_entry_states_its_shapes_and_rejects_others():
    L = _lib.lib()
    assert L.bgemm_packed_weight_forward_supported(1, 11008, 1, 4096) == 1
    assert L.bgemm_packed_weight_forward_supported(1, 11008, 4, 4096) == 1
    assert L.bgemm_packed_weight_forward_supported(1, 11008, 5, 4096) == 0           # beyond a few rows: pack kernel first
    assert L.bgemm_packed_weight_forward_supported(3, 11008, 4, 4096) == 1           # ternary planes
    assert L.bgemm_packed_weight_forward_supported(3, 11008, 17, 4096) == 0
    assert L.bgemm_packed_weight_forward_supported(1, 131072, 1, 4096) == 0          # streamed, not split in the block
    assert L.bgemm_packed_weight_forward_supported(9, 64, 1, 64) == 0
    names = ("mode", "W", "x", "dt", "ld", "zp", "out", "od", "M", "N", "K", "v", "sw", "sa", "b", "nz", "st")
    base = dict(mode=1, W=0x1000, x=0x2000, dt=0, ld=4096, zp=None, out=0x3000, od=0, M=64, N=4, K=4096, v=0, sw=None,
                sa=None, b=None, nz=None, st=None)
    call = lambda **k: L.bgemm_packed_weight_forward(*[{**base, **k}[n] for n in names])
    assert call(N=64) == _lib.EINVAL           # not a decode shape
    assert call(dt=7) == _lib.EINVAL
    assert call(ld=100) == _lib.EINVAL         # row stride shorter than K
    assert call(x=None) == _lib.ENULL
    assert call(x=0x2001) == _lib.EALIGN
    assert call(od=2) == _lib.ENULL            # scaled kind without scales
    assert call(v=1) == _lib.EINVAL            # the VALU design has no such kernel
    assert call(N=0) == 0 and call(M=0) == 0   # nothing to do


def test_empty_problems_are_ok_without_launch():
    L = _lib.lib()
    assert L.bgemm_packed_forward(1, None, None, None, None, 0, 0, 64, 64, 256, 0, 0, 0, 1, 0, None, 0, None, 0, None) == 0
    assert L.bgemm_packed_forward(1, None, None, None, None, 0, 1, 0, 64, 256, 0, 0, 0, 1, 0, None, 0, None, 0, None) == 0
    assert L.bgemm_pack_sign_f16(None, 0, 128, 128, None, None) == 0
    assert L.bgemm_f16_forward(None, None, None, 0, 5, 128, None, 0, 1, 1, None) == 0


def test_pack_and_f16_reject():
    L = _lib.lib()
    assert L.bgemm_pack_sign_f16(0x1000, 4, 128, 64, 0x2000, None) == _lib.EINVAL      # ld < K
    assert L.bgemm_pack_sign_f16(None, 4, 128, 128, 0x2000, None) == _lib.ENULL
    assert L.bgemm_pack_sign_f16(0x1000, 4, 128, 128, 0x2004, None) == _lib.EALIGN
    assert L.bgemm_pack_ternary_f16(0x1000, 4, 128, 128, 0x2000, None, None) == _lib.ENULL
    # batched packs: (src, dtype, ternary, zp, outer, inner, rows, K, ld, stride_outer, stride_inner, dst0, dst1, stream)
    assert L.bgemm_pack_batched(0x1000, 0, 0, None, 2, 3, 4, 128, 128, 0, 0, None, None, None) == _lib.ENULL
    assert L.bgemm_pack_batched(0x1000, 7, 0, None, 2, 3, 4, 128, 128, 0, 0, 0x2000, None, None) == _lib.EINVAL  # dtype
    assert L.bgemm_pack_batched(0x1000, 0, 0, None, 2, 3, 4, 128, 128, -8, 0, 0x2000, None, None) == _lib.EINVAL  # stride
    assert L.bgemm_pack_batched(0x1000, 0, 0, None, -1, 3, 4, 128, 128, 0, 0, 0x2000, None, None) == _lib.EINVAL
    assert L.bgemm_pack_batched(0x1000, 0, 1, 0x3000, 1, 1, 4, 128, 128, 0, 0, 0x2000, 0x4000, None) == _lib.EINVAL  # ternary + zero point
    assert L.bgemm_pack_batched(0x1000, 0, 1, None, 1, 1, 4, 128, 128, 0, 0, 0x2000, None, None) == _lib.ENULL     # second plane
    assert L.bgemm_pack_batched(None, 0, 0, None, 0, 3, 4, 128, 128, 0, 0, None, None, None) == 0                  # empty batch
    assert L.bgemm_pack_transposed_batched(0x1000, 0, 2, 3, 64, 128, 32, 0, 0, 0x2000, None) == _lib.EINVAL       # ld < rows
    assert L.bgemm_pack_transposed_batched(0x1000, 2, 2, 3, 64, 128, 64, 0, 0, 0x2000, None) == _lib.EINVAL       # dtype
    assert L.bgemm_pack_transposed_batched(0x1002, 1, 2, 3, 64, 128, 64, 0, 0, 0x2000, None) == _lib.EALIGN       # fp32 source
    assert L.bgemm_pack_transposed_batched(None, 0, 2, 3, 64, 128, 64, 0, 0, 0x2000, None) == _lib.ENULL
    assert L.bgemm_f16_forward(0x1000, 0x2000, 0x3000, 32, 32, 128, None, 0, 1, 3, None) == _lib.EINVAL  # INSTR 3
    assert L.bgemm_f16_forward(0x1000, 0x2000, 0x3000, 32, 32, 128, None, 0, 1, 1, None) == _lib.EWORKSPACE
    assert L.bgemm_f16_forward(0x1000, 0x2000, None, 32, 32, 128, 0x4000, 1 << 20, 1, 1, None) == _lib.ENULL


def test_missing_library_is_loud(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "SO_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError):
        _lib.lib()


def test_shim_rejects_cpu_tensors():
    import torch
    import lowbit_kernel
    x = torch.zeros(32, 128, dtype=torch.half)
    with pytest.raises(ValueError):
        lowbit_kernel.bgemm_linear_forward_cuda(x, x)
    with pytest.raises(NotImplementedError):
        lowbit_kernel.linear_forward_cuda()


def test_cpu_layers_match_reference_cpu_path(oracle):
    """BNNLinear / NNLinear_elastic_signed are plain torch and run anywhere."""
    import torch
    import bgemm_linear
    torch.manual_seed(0)
    x = torch.randn(32, 128)
    lin = bgemm_linear.BNNLinear(128, 64, False)
    y = lin(x)
    sw, sa, zpw, zpa = oracle.cpu_path_layer_scales(x, lin.weight)
    want = oracle.cpu_path_bnn_linear(x, lin.weight, None, sw, sa, zpw, zpa)
    assert torch.equal(y, want)
    el = bgemm_linear.NNLinear_elastic_signed(128, 64, True)
    y2 = el(x)
    xs = ((x - x.mean().item()) / el.sa).half().sign()
    ws = (el.weight - el.weight.mean().item()).half().sign()
    assert torch.equal(y2, oracle.cpu_path_linear(xs, ws) * el.sa * el.sw + el.bias)
    y2.sum().backward()
    assert el.weight.grad is not None and el.sa.grad is not None


def test_packed_file_format_round_trip_and_rejects(tmp_path):
    """The on-disk prepacked format is plain host code: header checks run without a GPU."""
    import numpy as np
    import torch
    import lowbit_kernel as lk
    rows, K = 40, 300
    words = 2 * 2 * 256
    rng = np.random.default_rng(3)
    d0 = torch.from_numpy(rng.integers(-2 ** 31, 2 ** 31 - 1, (3, words), dtype=np.int64).astype(np.int32))
    d1 = torch.from_numpy(rng.integers(-2 ** 31, 2 ** 31 - 1, (3, words), dtype=np.int64).astype(np.int32))
    path = str(tmp_path / "w.bgpk")
    lk.save_packed(path, lk.PackedBits(d0, d1, 3, rows, K))
    assert lk.read_packed_header(path) == (2, 3, rows, K, words)
    back = lk.load_packed(path, device="cpu")
    assert back.batch == 3 and back.rows == rows and back.K == K and back.ternary
    assert torch.equal(back.data, d0) and torch.equal(back.data2, d1)
    raw = bytearray(open(path, "rb").read())
    for mutate, what in ((lambda b: b.__setitem__(0, 0x58), "magic"), (lambda b: b.__setitem__(8, 99), "version"),
                         (lambda b: b.__setitem__(slice(24, 32), (100).to_bytes(8, "little")), "rows vs words")):
        bad = bytearray(raw)
        mutate(bad)
        open(path, "wb").write(bad)
        with pytest.raises(ValueError):
            lk.read_packed_header(path)
    open(path, "wb").write(raw[:-4])          # truncated payload
    with pytest.raises(ValueError):
        lk.load_packed(path, device="cpu")


def test_shim_checks_buffers_before_the_kernel_sees_them(monkeypatch):
    """A wrong output tensor or a hand-built PackedBits is a ValueError, not an out-of-bounds access on the GPU."""
    import torch
    import lowbit_kernel as lk
    monkeypatch.setattr(lk, "_need_cuda", lambda t, name: None)       # the checks themselves are host code
    words = _lib.lib().bgemm_tiled_words(40, 300)
    good = lambda rows: lk.PackedBits(torch.zeros((1, _lib.lib().bgemm_tiled_words(rows, 300)), dtype=torch.int32), None, 1, rows, 300)
    w, x = good(40), good(7)
    for bad_out in (torch.zeros((1, 7, 39), dtype=torch.int32),                 # too small
                    torch.zeros((1, 7, 40), dtype=torch.int16),                 # wrong element type
                    torch.zeros((1, 40, 7), dtype=torch.int32).transpose(1, 2)):    # not contiguous
        with pytest.raises(ValueError):
            lk.bgemm_packed_forward(w, x, out=bad_out)
    for bad in (lk.PackedBits(torch.zeros((1, words - 256), dtype=torch.int32), None, 1, 40, 300),     # a tile short
                lk.PackedBits(torch.zeros((1, words), dtype=torch.int64), None, 1, 40, 300),
                lk.PackedBits(torch.zeros((2, words), dtype=torch.int32), None, 1, 40, 300),
                lk.PackedBits(torch.zeros((1, 2 * words), dtype=torch.int32)[:, ::2], None, 1, 40, 300)):
        with pytest.raises(ValueError):
            lk.bgemm_packed_forward(bad, x)
    with pytest.raises(ValueError):
        lk.bgemm_packed_forward(w, lk.PackedBits(x.data, torch.zeros((1, 256), dtype=torch.int32), 1, 7, 300), _lib.MODE_BWTA)


def test_chain_entry_point_rejects_bad_arguments_on_the_host():
    """bgemm_chain_forward checks its arguments before anything touches a GPU (tests/python/bgemm_linear.py:474-486 is the
    stack of layers it runs; the reference's own launcher asserts and aborts instead, fp6_linear.cu:288-290)."""
    L = _lib.lib()
    layers = (_lib.ChainLayer * 2)()
    for l, (M, K) in enumerate(((512, 256), (64, 512))):
        layers[l].W_tiled, layers[l].sw, layers[l].sa, layers[l].M, layers[l].K = 4096, 4096, 4096, M, K
    call = lambda mode=1, lay=layers, n=2, N=4, out_dtype=0, param=0: L.bgemm_chain_forward(
        mode, lay, 4096, n, 4096, 4096, N, 4096, out_dtype, param, 4096, 1 << 20, 0, None)
    assert call(mode=9) == _lib.EINVAL
    assert call(lay=None) == _lib.ENULL
    assert call(n=0) == _lib.EINVAL and call(n=200) == _lib.EINVAL
    assert call(N=0) == _lib.EINVAL and call(N=33) == _lib.EINVAL and call(mode=3, N=17) == _lib.EINVAL
    assert b"activation rows" in L.bgemm_last_error()
    assert L.bgemm_chain_workspace_bytes(9, layers, 2, 4) == 0
    assert L.bgemm_chain_status(None, None) == _lib.ENULL
