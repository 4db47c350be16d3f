"""Parity of every kernel behind bgemm_packed_forward*, kernel by kernel.

The library picks a kernel per shape, so a test only covers the kernel its shape lands on.  Here every
case either asserts the kernel the library reports for the call (``packed_kernel_id``) or insists on one
(``force_kernel``), so that each tile of the general matrix-core kernel, and each decode-shaped kernel, runs
ragged M / N / K, odd K-tile counts and every output kind against the dense closed forms on de-binarised
operands (the reference drivers' own method, csrc/benchmark.cu:146-204), the epilogue and prologue models of
the oracle, bit for bit.  Output order and fp16 rounding follow kernel_matmul.cuh:529-546.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lowbit_kernel as lk
import _lib as B
from _lib import (MODE_AND, MODE_XOR, MODE_ATTN, MODE_BWTA, MODE_ATTN_X, VARIANT_AUTO, VARIANT_VALU, VARIANT_MFMA,
                  VARIANT_MFMA_F4, force_kernel)

DEV = "cuda:0"
TILES = {"256x256": B.KERNEL_MFMA_256x256, "256x128": B.KERNEL_MFMA_256x128, "128x128": B.KERNEL_MFMA_128x128,
         "64x128": B.KERNEL_MFMA_64x128, "32x128": B.KERNEL_MFMA_32x128, "32x256": B.KERNEL_MFMA_32x256, "128x64": B.KERNEL_MFMA_128x64,
         "64x64": B.KERNEL_MFMA_64x64}
ENGINES = {"fp4": VARIANT_MFMA_F4, "int8": VARIANT_MFMA}


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def pm1(rng, *shape):
    """+-1 fp16 with both zeros mixed in: -0.0 counts as negative, +0.0 as positive."""
    bits = rng.integers(0, 2, shape, dtype=np.int8)
    v = np.where(bits == 1, np.float16(-1), np.float16(1)).astype(np.float16)
    z = rng.random(shape) < 0.01
    return np.where(z, np.where(bits == 1, np.float16(-0.0), np.float16(0.0)), v).astype(np.float16)


def sgn(a):
    return 1.0 - 2.0 * (a.view(np.uint16) >> 15).astype(np.float32)


def dense(mode, w, x):
    """fp32 closed forms (exact below 2^24) on operands de-binarised by sign bit; x [.., N, K], w [.., M, K]."""
    a, b = (1 - sgn(w)) / 2, (1 - sgn(x)) / 2
    wt = np.swapaxes
    if mode == MODE_XOR:
        r = sgn(x) @ wt(sgn(w), -1, -2)
    elif mode == MODE_AND:
        r = b @ wt(a, -1, -2)
    elif mode == MODE_ATTN:
        r = sgn(x) @ wt(1 - a, -1, -2)
    elif mode == MODE_ATTN_X:
        r = (1 - b) @ wt(sgn(w), -1, -2)
    else:
        xs = x.view(np.uint16)
        t = np.where((xs & 0x7FFF) == 0, 0.0, sgn(x)).astype(np.float32)
        r = t @ wt(sgn(w), -1, -2)
    return r.astype(np.int32)


def f16_of(i32):
    with np.errstate(over="ignore"):
        return i32.astype(np.float32).astype(np.float16)


def bits_of(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


def check_all_kinds(oracle, wp, xp, acc, M, N, variant, rng, rows=None, cols=None, mode=MODE_XOR):
    """Every output kind of one GEMM against `acc` (the exact int32 result, or its [rows][:, cols] sample)."""
    def sample(t):
        t = t[0]
        if rows is not None:
            t = t[torch.from_numpy(rows).to(DEV)][:, torch.from_numpy(cols).to(DEV)]
        return t.cpu().numpy()

    got = sample(lk.bgemm_packed_forward(wp, xp, mode, torch.int32, 1, variant))
    assert (got == acc).all(), "int32"
    got = sample(lk.bgemm_packed_forward(wp, xp, mode, torch.half, 1, variant))
    assert (bits_of(got) == bits_of(f16_of(acc))).all(), "fp16"
    for dtype in (np.float32, np.float16):
        sw = rng.uniform(1e-4, 3e-3, M).astype(dtype)
        sa = np.asarray(1.7371, dtype=dtype)
        bias = (0.05 * rng.standard_normal(M)).astype(dtype)
        swc, bc = (sw, bias) if cols is None else (sw[cols], bias[cols])
        for with_bias in (True, False):
            want = oracle.np_scale_epilogue(acc, swc, sa, bc if with_bias else None)
            got = sample(lk.bgemm_packed_forward(wp, xp, mode, variant=variant,
                                                 scale=(to_dev(sw), to_dev(sa.reshape(1)), to_dev(bias) if with_bias else None)))
            assert got.dtype == want.dtype and (bits_of(got) == bits_of(want)).all(), ("scaled", dtype, with_bias)
        # bits kinds: the next layer's operand, the zero point at a value that splits the outputs
        zp = np.asarray(0.011, dtype=dtype)
        out = lk.zeros_packed(N, M, 1, DEV)
        lk.bgemm_packed_forward(wp, xp, mode, variant=variant, bits_out=out,
                                scale=(to_dev(sw), to_dev(sa.reshape(1)), to_dev(bias)), next_zero_point=to_dev(zp.reshape(1)))
        logical = lk.logical_from_tiled(out).cpu().numpy().view(np.uint32)               # [N][ceil(M/32)]
        y = oracle.np_scale_epilogue(acc, swc, sa, bc)
        want_bits = oracle.np_center_to_f16(y, zp).view(np.uint16) >> 15                  # 1 = negative
        got_bits = np.unpackbits(logical.byteswap().view(np.uint8), axis=1)[:, :M]        # MSB-first words
        if rows is not None:
            got_bits = got_bits[rows][:, cols]
        assert (got_bits == want_bits).all(), ("bits", dtype)
        assert 0.2 < want_bits.mean() < 0.8                                               # the zero point does split them
        # nothing but real bits was written
        assert int(np.unpackbits(out.data.cpu().numpy().view(np.uint8)).sum()) == int(np.unpackbits(logical.view(np.uint8)).sum())


# M picks the store path of the general kernel: 520 = 16-byte stores of eight halves / four ints, 516 = four elements a lane,
# 517 = one element a lane; N = 515 leaves a ragged last strip; K = 1275 is five K-tiles (odd: the pipelined
# loops run a zero tile to fill their last pair), the last one ragged
@pytest.mark.parametrize("M", [520, 516, 517])
@pytest.mark.parametrize("engine", list(ENGINES))
@pytest.mark.parametrize("tile", list(TILES))
def test_each_tile_every_output_kind(oracle, tile, engine, M):
    N, K = 515, 1275
    rng = np.random.default_rng(M * 31 + TILES[tile])
    w, x = pm1(rng, M, K), pm1(rng, N, K)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    variant = force_kernel(TILES[tile], ENGINES[engine])
    assert lk.packed_kernel_id(wp, xp, MODE_XOR, 1, variant) == TILES[tile]
    check_all_kinds(oracle, wp, xp, dense(MODE_XOR, w, x), M, N, variant, rng)


@pytest.mark.parametrize("KT", [9, 17])
@pytest.mark.parametrize("M", [520, 517])
@pytest.mark.parametrize("engine", list(ENGINES))
def test_128x128_takes_the_pipelined_loop_from_eight_k_tiles(oracle, engine, M, KT):
    """From eight K-tiles on the 128 x 128 tile runs the hand-pipelined loop (fp16 pairs, which the plain loop stores
    straight from its registers, from sixteen): nine and seventeen K-tiles, the last ragged, every output kind, ragged
    M and N; and with the operands' row popcounts brought along."""
    N, K = 515, KT * 256 - 5
    rng = np.random.default_rng(M * 17 + 5)
    w, x = pm1(rng, M, K), pm1(rng, N, K)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    variant = force_kernel(TILES["128x128"], ENGINES[engine])
    acc = dense(MODE_XOR, w, x)
    check_all_kinds(oracle, wp, xp, acc, M, N, variant, rng)
    lk.row_popcounts(wp), lk.row_popcounts(xp)
    assert (lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1, variant)[0].cpu().numpy() == acc).all()
    # a ternary operand's two planes on the same loop (the tile then has the fragments of 256 x 128 of one plane)
    t = x.copy()
    t[rng.random(t.shape) < 0.3] = 0
    xt, want = lk.pack_ternary(to_dev(t)), dense(MODE_BWTA, w, t)
    assert (lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, variant)[0].cpu().numpy() == want).all()
    goth = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.half, 1, variant)[0].cpu().numpy()
    assert (bits_of(goth) == bits_of(f16_of(want))).all()
    sw, sa = rng.uniform(1e-4, 3e-3, M).astype(np.float32), np.asarray(0.61, dtype=np.float32)
    gots = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, splitK=1, variant=variant, scale=(to_dev(sw), to_dev(sa.reshape(1)), None))[0].cpu().numpy()
    assert (bits_of(gots) == bits_of(oracle.np_scale_epilogue(want, sw, sa, None))).all()


@pytest.mark.parametrize("KT", [9, 17])
@pytest.mark.parametrize("engine", list(ENGINES))
@pytest.mark.parametrize("tile", ["128x128", "32x256"])
def test_two_planes_on_the_pipelined_loop(oracle, tile, engine, KT):
    """A ternary operand on the two tiles whose two-plane form runs the hand-pipelined loop (from eight K-tiles; fp16
    pairs from sixteen): ragged M, N and K, an odd K-tile count, int32, fp16 and the scaled output against the dense
    reference and the oracle's epilogue."""
    rng = np.random.default_rng(TILES[tile] * 100 + KT)
    variant = force_kernel(TILES[tile], ENGINES[engine])
    for M, N in ((520, 515), (517, 130)):
        K = KT * 256 - 5
        w, t = pm1(rng, M, K), pm1(rng, N, K)
        t[rng.random(t.shape) < 0.4] = 0
        wp, xt, want = lk.pack_sign(to_dev(w)), lk.pack_ternary(to_dev(t)), dense(MODE_BWTA, w, t)
        assert (lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, variant)[0].cpu().numpy() == want).all()
        goth = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.half, 1, variant)[0].cpu().numpy()
        assert (bits_of(goth) == bits_of(f16_of(want))).all()
        sw, sa = rng.uniform(1e-4, 3e-3, M).astype(np.float32), np.asarray(0.61, dtype=np.float32)
        gots = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, splitK=1, variant=variant, scale=(to_dev(sw), to_dev(sa.reshape(1)), None))[0].cpu().numpy()
        assert (bits_of(gots) == bits_of(oracle.np_scale_epilogue(want, sw, sa, None))).all()


@pytest.mark.parametrize("K", [512, 16 * 256 + 40])
@pytest.mark.parametrize("tile,N,M", [("128x128", 1024, 512), ("128x128", 512, 1024), ("256x128", 1024, 1024),
                                       ("256x128", 2048, 512), ("256x256", 1024, 2048), ("128x128", 1000, 500), ("128x128", 512, 768), ("128x128", 768, 512)])
def test_tile_grids_that_split_evenly_among_the_xcds(tile, N, M, K):
    """One product on the tall tiles whose tile grid divides by 4 x 2 (short K) or 2 x 4: every XCD walks a sub-rectangle of
    its own; every tile must be computed exactly once (whole output against the dense form), and the two-plane and
    batched calls, which walk the grid the other way, on the same operands."""
    rng = np.random.default_rng(N + M + K)
    w, x = pm1(rng, M, K), pm1(rng, N, K)
    wp, xp, xt = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x)), lk.pack_ternary(to_dev(x))
    for mode, xo in ((MODE_XOR, xp), (MODE_AND, xp)) + (((MODE_BWTA, xt),) if tile == "128x128" else ()):
        want = dense(mode, w, x)
        for dt in (torch.int32, torch.half):
            got = lk.bgemm_packed_forward(wp, xo, mode, dt, 1, force_kernel(TILES[tile]))[0].cpu().numpy()
            assert (got.astype(np.float32) == want.astype(np.float16 if dt == torch.half else np.int32).astype(np.float32)).all(), (mode, dt)
    wp2 = lk.PackedBits(torch.cat([wp.data, wp.data]), None, 2, M, K)
    got2 = lk.bgemm_packed_forward(wp2, xp, MODE_XOR, torch.int32, 1, force_kernel(TILES[tile])).cpu().numpy()
    assert (got2[0] == dense(MODE_XOR, w, x)).all() and (got2[1] == got2[0]).all()


@pytest.mark.parametrize("engine", list(ENGINES))
@pytest.mark.parametrize("tile", list(TILES))
def test_each_tile_every_mode_batched(tile, engine):
    """All five modes on a batch of ragged matrices, one K-tile and an even number of them; tiles built for one bit
    plane refuse the ternary operand."""
    rng = np.random.default_rng(TILES[tile])
    variant = force_kernel(TILES[tile], ENGINES[engine])
    for Bn, M, N, K in ((3, 70, 300, 200), (2, 300, 70, 1000)):
        w, x = pm1(rng, Bn, M, K), pm1(rng, Bn, N, K)
        x[rng.random(x.shape) < 0.3] = 0                          # ternary zeros (+0.0: positive for the sign modes)
        wp, xp, xt = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x)), lk.pack_ternary(to_dev(x))
        for mode in (MODE_AND, MODE_XOR, MODE_ATTN, MODE_ATTN_X):
            got = lk.bgemm_packed_forward(wp, xp, mode, torch.int32, 2, variant).cpu().numpy()
            assert (got == dense(mode, w, x)).all(), mode
        if tile in ("256x256", "256x128"):
            with pytest.raises(ValueError):
                lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, variant)
        else:
            got = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.half, 1, variant).cpu().numpy()
            assert (bits_of(got) == bits_of(f16_of(dense(MODE_BWTA, w, x)))).all()


@pytest.mark.parametrize("engine", list(ENGINES))
@pytest.mark.parametrize("tile", ["128x128", "32x256"])
def test_fp16_pairs_straight_from_the_accumulators(tile, engine):
    """Plain fp16 output with rows of a multiple of eight on the tiles whose waves hold an even number of weight
    tiles: weight rows are dealt in pairs and two halves leave in one store.  Every mode (two bit planes included),
    a ragged last weight tile (M = 328: the block's later tiles do not exist), a ragged last strip, and K of
    one ragged word, two words (both take the two-words-a-fragment loop), one K-tile and three."""
    rng = np.random.default_rng(97 + TILES[tile])
    variant = force_kernel(TILES[tile], ENGINES[engine])
    Bn, M, N = 2, 328, 77
    for K in (40, 64, 200, 600):
        w, x = pm1(rng, Bn, M, K), pm1(rng, Bn, N, K)
        x[rng.random(x.shape) < 0.3] = 0
        wp, xp, xt = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x)), lk.pack_ternary(to_dev(x))
        assert lk.packed_kernel_id(wp, xp, MODE_XOR, 1, variant, torch.half) == TILES[tile]
        for mode in (MODE_AND, MODE_XOR, MODE_ATTN, MODE_ATTN_X, MODE_BWTA):
            got = lk.bgemm_packed_forward(wp, xt if mode == MODE_BWTA else xp, mode, torch.half, 1, variant).cpu().numpy()
            assert (bits_of(got) == bits_of(f16_of(dense(mode, w, x)))).all(), (K, mode)


@pytest.mark.parametrize("engine", list(ENGINES))
@pytest.mark.parametrize("tile", [t for t in TILES if t not in ("256x256", "256x128")])
def test_k_of_at_most_two_words_on_every_tile(tile, engine):
    """K <= 64 expands two words a fragment instead of four (the loop of the tiles that are not hand-pipelined):
    int32, every mode, K = 1, 33 and 64."""
    rng = np.random.default_rng(131 + TILES[tile])
    variant = force_kernel(TILES[tile], ENGINES[engine])
    for K in (1, 33, 64):
        w, x = pm1(rng, 2, 100, K), pm1(rng, 2, 45, K)
        x[rng.random(x.shape) < 0.3] = 0
        wp, xp, xt = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x)), lk.pack_ternary(to_dev(x))
        for mode in (MODE_AND, MODE_XOR, MODE_ATTN, MODE_ATTN_X, MODE_BWTA):
            got = lk.bgemm_packed_forward(wp, xt if mode == MODE_BWTA else xp, mode, torch.int32, 1, variant).cpu().numpy()
            assert (got == dense(mode, w, x)).all(), (K, mode)


@pytest.mark.parametrize("engine", list(ENGINES))
@pytest.mark.parametrize("tile", ["256x256", "256x128", "128x128"])
def test_row_popcounts_brought_by_the_caller(tile, engine):
    """bgemm_row_popcounts against numpy, then bgemm_packed_forward_counted: every mode of one bit plane, int32 and
    fp16, a weight operand shared by a batch of two, ragged M / N / K with an odd K-tile count.  The two pipelined
    tiles must really use the counts (a count raised by one moves that row's XOR outputs by -2); the other tiles
    count for themselves and ignore them."""
    rng = np.random.default_rng(211 + TILES[tile])
    variant = force_kernel(TILES[tile], ENGINES[engine])
    M, N, K = 300, 290, 1275
    w, x = pm1(rng, 1, M, K), pm1(rng, 2, N, K)
    wp, xp = lk.row_popcounts(lk.pack_sign(to_dev(w))), lk.row_popcounts(lk.pack_sign(to_dev(x)))
    for p, a in ((wp, w), (xp, x)):
        assert (p.counts.cpu().numpy() == (a.view(np.uint16) >> 15).sum(-1)).all()
    for mode in (MODE_AND, MODE_XOR, MODE_ATTN, MODE_ATTN_X):
        want = dense(mode, w, x)
        assert (lk.bgemm_packed_forward(wp, xp, mode, torch.int32, 1, variant).cpu().numpy() == want).all(), mode
        got = lk.bgemm_packed_forward(wp, xp, mode, torch.half, 1, variant).cpu().numpy()
        assert (bits_of(got) == bits_of(f16_of(want))).all(), mode
    want = dense(MODE_XOR, w, x)
    wp.counts[0, 7] += 1
    xp.counts[1, 11] += 1
    got = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1, variant).cpu().numpy()
    if tile in ("256x256", "256x128"):
        want[:, :, 7] -= 2
        want[1, 11, :] -= 2
    assert (got == want).all()


def tern(rng, *shape):
    """-1 / 0 / +1 fp16 with both zeros among the zeros."""
    t = rng.integers(-1, 2, shape).astype(np.float16)
    return np.where((t == 0) & (rng.random(shape) < 0.5), np.float16(-0.0), t).astype(np.float16)


# The signed tile (binary weights x ternary activations as signed fp4 operands, one MFMA per 64 k where the two bit planes
# take two): M picks the store path as above, N = 515 leaves a ragged strip, K = five K-tiles (odd: the loop runs whole pairs, the
# last tile of the pair reads as zero bits) and eight, the last one ragged.
@pytest.mark.parametrize("K", [1275, 2048 - 9])
@pytest.mark.parametrize("M", [520, 516, 517])
def test_signed_ternary_tile_every_output_kind(oracle, M, K):
    N = 515
    rng = np.random.default_rng(M * 37 + K)
    w, t = pm1(rng, M, K), tern(rng, N, K)
    wp, xt = lk.pack_sign(to_dev(w)), lk.pack_ternary(to_dev(t))
    variant = force_kernel(B.KERNEL_MFMA_128x256T, VARIANT_MFMA_F4)
    assert lk.packed_kernel_id(wp, xt, MODE_BWTA, 1, variant) == B.KERNEL_MFMA_128x256T
    check_all_kinds(oracle, wp, xt, dense(MODE_BWTA, w, t), M, N, variant, rng, mode=MODE_BWTA)


def test_signed_ternary_tile_batched_and_what_it_refuses():
    """A batch of ragged matrices, one K-tile and several; every ternary value against every weight sign; the tile takes
    nothing but a ternary operand on the fp4 engine."""
    rng = np.random.default_rng(128256)
    variant = force_kernel(B.KERNEL_MFMA_128x256T, VARIANT_MFMA_F4)
    for Bn, M, N, K in ((3, 70, 300, 200), (2, 300, 70, 1000), (1, 257, 129, 256 * 3)):
        w, t = pm1(rng, Bn, M, K), tern(rng, Bn, N, K)
        wp, xt = lk.pack_sign(to_dev(w)), lk.pack_ternary(to_dev(t))
        got = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, variant).cpu().numpy()
        assert (got == dense(MODE_BWTA, w, t)).all()
        got = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.half, 1, variant).cpu().numpy()
        assert (bits_of(got) == bits_of(f16_of(dense(MODE_BWTA, w, t)))).all()
    # all-equal operands: every product -1, 0 or +1 in all of K, whole rows at +-K
    M, N, K = 256, 128, 1024
    for wv in (1.0, -1.0):
        for tv in (1.0, -1.0, 0.0):
            wp = lk.pack_sign(torch.full((M, K), wv, dtype=torch.half, device=DEV))
            xt = lk.pack_ternary(torch.full((N, K), tv, dtype=torch.half, device=DEV))
            got = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, variant)
            assert int(got.min()) == int(got.max()) == int(wv * tv * K)
    xp = lk.pack_sign(to_dev(pm1(rng, N, K)))
    with pytest.raises(ValueError):
        lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1, variant)                                    # one bit plane
    with pytest.raises(ValueError):
        lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, force_kernel(B.KERNEL_MFMA_128x256T, VARIANT_MFMA))   # the int8 engine


@pytest.mark.parametrize("seed", range(12))
def test_signed_ternary_tile_random_shapes(seed):
    """Seeded random shapes, ragged in every dimension (K from one bit to a dozen K-tiles, batches of one to three), sparse
    and dense ternary rows: the forced signed tile against the dense product, int32 and fp16."""
    rng = np.random.default_rng(9100 + seed)
    variant = force_kernel(B.KERNEL_MFMA_128x256T, VARIANT_MFMA_F4)
    for _ in range(4):
        Bn, M, N = int(rng.integers(1, 4)), int(rng.integers(1, 700)), int(rng.integers(1, 400))
        K = int(rng.choice([1, 31, 64, 255, 256, 257, int(rng.integers(1, 3000))]))
        w, t = pm1(rng, Bn, M, K), tern(rng, Bn, N, K)
        t[rng.random(t.shape) < rng.random()] = 0                      # from almost dense to almost empty
        wp, xt = lk.pack_sign(to_dev(w)), lk.pack_ternary(to_dev(t))
        want = dense(MODE_BWTA, w, t)
        got = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, variant).cpu().numpy()
        assert (got == want).all(), (Bn, M, N, K)
        got = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.half, 1, variant).cpu().numpy()
        assert (bits_of(got) == bits_of(f16_of(want))).all(), (Bn, M, N, K)


@pytest.mark.parametrize("M,N,K", [(4096 + 5, 2048 + 3, 17 * 256 - 7), (11008, 512, 4096)])
def test_signed_ternary_tile_where_the_library_picks_it(oracle, M, N, K):
    """No forcing: prefill-sized BWTA products go to the signed tile on the fp4 engine (the library's choice) and to the
    two-plane tiles on the int8 engine; both agree with the dense product on sampled rows and columns, edges included, in
    every output kind, and with each other everywhere."""
    rng = np.random.default_rng(M + N)
    g = torch.Generator(device=DEV).manual_seed(M * 7 + N)
    w16 = (1 - 2 * torch.randint(0, 2, (M, K), generator=g, device=DEV, dtype=torch.int8)).to(torch.half)
    t16 = torch.randint(-1, 2, (N, K), generator=g, device=DEV, dtype=torch.int8).to(torch.half)
    wp, xt = lk.pack_sign(w16), lk.pack_ternary(t16)
    assert lk.packed_kernel_id(wp, xt, MODE_BWTA) == B.KERNEL_MFMA_128x256T
    assert lk.packed_kernel_id(wp, xt, MODE_BWTA, 1, VARIANT_MFMA_F4) == B.KERNEL_MFMA_128x256T
    assert lk.packed_kernel_id(wp, xt, MODE_BWTA, 1, VARIANT_MFMA) != B.KERNEL_MFMA_128x256T
    rows = np.unique(np.concatenate([rng.choice(N, 90, replace=False), [0, N - 1, N - 2, (N // 32) * 32, (N // 128) * 128]]))
    cols = np.unique(np.concatenate([rng.choice(M, 120, replace=False), [0, M - 1, M - 2, (M // 32) * 32, (M // 256) * 256]]))
    rows, cols = rows[rows < N], cols[cols < M]
    wsub = w16[torch.from_numpy(cols).to(DEV)].float().cpu()
    xsub = t16[torch.from_numpy(rows).to(DEV)].float().cpu()
    acc = (xsub @ wsub.T).to(torch.int32).numpy()
    check_all_kinds(oracle, wp, xt, acc, M, N, VARIANT_AUTO, rng, rows, cols, mode=MODE_BWTA)
    out = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32)[0]
    assert torch.equal(out, lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, VARIANT_MFMA)[0])
    assert int(out.to(torch.int64).sum()) == int((w16.double().sum(0) * t16.double().sum(0)).sum().item())


@pytest.mark.parametrize("engine", list(ENGINES))
@pytest.mark.parametrize("M,N,K,want_kernel", [
    (5907, 5903, 129 * 256 - 5, B.KERNEL_MFMA_256x256),      # the tile of the longest K: ragged edges, 129 K-tiles
    (5907, 5903, 33 * 256 - 5, B.KERNEL_MFMA_256x128),       # the 8192^3 kernel: ragged edges, 33 K-tiles
    (8195, 2053, 17 * 256 - 7, B.KERNEL_MFMA_256x128),       # the 8192 x 2048 x 4096 kernel likewise
    (2048, 4127, 5 * 256 - 5, B.KERNEL_MFMA_32x256),         # int32 rows of 8 KiB on a short K: the 32-row tile
])
def test_headline_tiles_where_the_library_picks_them(oracle, engine, M, N, K, want_kernel):
    """No forcing: shapes that the library itself sends to the two large tiles, ragged in M, N and K with an odd
    K-tile count, every output kind, on sampled rows and columns (the edges included)."""
    rng = np.random.default_rng(M + N)
    g = torch.Generator(device=DEV).manual_seed(M * 7 + N)
    w16 = (1 - 2 * torch.randint(0, 2, (M, K), generator=g, device=DEV, dtype=torch.int8)).to(torch.half)
    x16 = (1 - 2 * torch.randint(0, 2, (N, K), generator=g, device=DEV, dtype=torch.int8)).to(torch.half)
    wp, xp = lk.pack_sign(w16), lk.pack_sign(x16)
    variant = ENGINES[engine]
    assert lk.packed_kernel_id(wp, xp, MODE_XOR, 1, variant) == want_kernel
    rows = np.unique(np.concatenate([rng.choice(N, 90, replace=False), [0, N - 1, N - 2, (N // 32) * 32, (N // 256) * 256]]))
    cols = np.unique(np.concatenate([rng.choice(M, 120, replace=False), [0, M - 1, M - 2, (M // 32) * 32, (M // 128) * 128]]))
    rows, cols = rows[rows < N], cols[cols < M]               # (a size that is a whole number of tiles has no ragged tile)
    wsub = w16[torch.from_numpy(cols).to(DEV)].float().cpu()
    xsub = x16[torch.from_numpy(rows).to(DEV)].float().cpu()
    acc = (xsub @ wsub.T).to(torch.int32).numpy()
    check_all_kinds(oracle, wp, xp, acc, M, N, variant, rng, rows, cols)
    # the whole output: parity, range, the checksum of checksums
    out = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1, variant)[0]
    assert int(((out - K) % 2).abs().max()) == 0 and int(out.abs().max()) <= K
    assert int(out.to(torch.int64).sum()) == int((w16.double().sum(0) * x16.double().sum(0)).sum().item())


def test_config3_attention_av_all_192_heads():
    """The batched attention x value configuration at its full size, every element: 16 x 12 heads, attn {0,1} [512,512] x value +-1 [512,64]."""
    rng = np.random.default_rng(3192)
    Bn, S, D = 192, 512, 64
    attn_bits = rng.integers(0, 2, (Bn, S, S), dtype=np.int8)
    v = np.where(rng.integers(0, 2, (Bn, S, D), dtype=np.int8) == 1, np.float16(-1), np.float16(1)).astype(np.float16)
    want = np.matmul(attn_bits.astype(np.float32), v.astype(np.float32)).astype(np.int32)
    attn16 = to_dev((2 * attn_bits - 1).astype(np.float16))          # "1" must have its sign bit clear
    ap, vp = lk.pack_sign(attn16), lk.pack_sign_transposed(to_dev(v))
    assert lk.packed_kernel_id(vp, ap, MODE_ATTN_X) == B.KERNEL_MFMA_64x64
    for variant in (VARIANT_AUTO, VARIANT_MFMA, force_kernel(B.KERNEL_MFMA_128x64)):
        got = lk.bgemm_packed_forward(vp, ap, MODE_ATTN_X, torch.int32, 1, variant).cpu().numpy()
        assert (got == want).all(), variant
        # the reference's orientation (attn as the weight side, INSTR = 2) gives the transpose
        got_t = lk.bgemm_packed_forward(ap, vp, MODE_ATTN, torch.int32, 1, variant).cpu().numpy()
        assert (got_t.transpose(0, 2, 1) == want).all(), variant
    goth = lk.bgemm_packed_forward(vp, ap, MODE_ATTN_X, torch.half).cpu().numpy()
    assert (bits_of(goth) == bits_of(f16_of(want))).all()


def test_narrow_outputs_ragged_batch():
    """The 128 x 64 tile where the library picks it, ragged in every dimension."""
    rng = np.random.default_rng(77)
    Bn, M, N, K = 350, 50, 300, 700
    w, x = pm1(rng, Bn, M, K), pm1(rng, Bn, N, K)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    assert lk.packed_kernel_id(wp, xp, MODE_XOR) == B.KERNEL_MFMA_128x64
    for mode in (MODE_XOR, MODE_ATTN_X):
        assert (lk.bgemm_packed_forward(wp, xp, mode).cpu().numpy() == dense(mode, w, x)).all()
    got = lk.bgemm_packed_forward(wp, xp, MODE_AND, torch.half, 1, VARIANT_MFMA).cpu().numpy()
    assert (bits_of(got) == bits_of(f16_of(dense(MODE_AND, w, x)))).all()


@pytest.mark.parametrize("engine", list(ENGINES))
def test_stream_kernel_up_to_four_rows_one_store_a_row(engine):
    """The streaming decode kernel writes a row's 64 outputs of a wave's two weight tiles as one store when there are
    at most four rows: every row count from 1 to 5 (5: the other path), sign and ternary activations, a weight matrix
    whose last tile pair is incomplete (M = 100: tiles 2 and 3, the last with four rows) and one with an odd number
    of tiles (M = 90), int32 and fp16."""
    rng = np.random.default_rng(977)
    variant = force_kernel(B.KERNEL_SKINNY_STREAM, ENGINES[engine])
    for M in (100, 90, 128):
        Bn, K = 1100, 300
        w = pm1(rng, Bn, M, K)
        wp = lk.pack_sign(to_dev(w))
        for N in (1, 2, 3, 4, 5):
            x = pm1(rng, 1, N, K)
            x[rng.random(x.shape) < 0.3] = 0
            xp, xt = lk.pack_sign(to_dev(x)), lk.pack_ternary(to_dev(x))
            for mode, xop in ((MODE_XOR, xp), (MODE_BWTA, xt)):
                assert lk.packed_kernel_id(wp, xop, mode, 1, variant) == B.KERNEL_SKINNY_STREAM
                want = dense(mode, w, x)
                got = lk.bgemm_packed_forward(wp, xop, mode, torch.int32, 1, variant).cpu().numpy()
                assert (got == want).all(), (M, N, mode)
                got = lk.bgemm_packed_forward(wp, xop, mode, torch.half, 1, variant).cpu().numpy()
                assert (bits_of(got) == bits_of(f16_of(want))).all(), (M, N, mode)


@pytest.mark.parametrize("N,want_kernel", [(256, B.KERNEL_SKINNY_QUAD), (2048, B.KERNEL_MFMA_256x128),
                                           # 192 and 256 blocks of 128 x 128 on 64 K-tiles (three K-tiles in flight)
                                           (320, B.KERNEL_MFMA_128x128), (512, B.KERNEL_MFMA_128x128)])
def test_config5_sweep_long_k(N, want_kernel):
    """The K = 16384 points of configuration 5's sweep, split-K 1 / 2 / 4: sampled rows and columns against the
    closed form, identities over the whole output, and agreement between the split-K values and the designs."""
    M, K = 8192, 16384
    g = torch.Generator(device=DEV).manual_seed(N)
    w16 = (1 - 2 * torch.randint(0, 2, (M, K), generator=g, device=DEV, dtype=torch.int8)).to(torch.half)
    x16 = (1 - 2 * torch.randint(0, 2, (N, K), generator=g, device=DEV, dtype=torch.int8)).to(torch.half)
    wp, xp = lk.pack_sign(w16), lk.pack_sign(x16)
    assert lk.packed_kernel_id(wp, xp, MODE_XOR) == want_kernel
    out = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1)[0]
    rng = np.random.default_rng(N)
    rows, cols = rng.choice(N, 64, replace=False), rng.choice(M, 96, replace=False)
    want = (x16[torch.from_numpy(rows).to(DEV)].float().cpu() @ w16[torch.from_numpy(cols).to(DEV)].float().cpu().T).to(torch.int32)
    assert torch.equal(out[torch.from_numpy(rows).to(DEV)][:, torch.from_numpy(cols).to(DEV)].cpu(), want)
    assert int(((out - K) % 2).abs().max()) == 0 and int(out.abs().max()) <= K
    assert int(out.to(torch.int64).sum()) == int((w16.double().sum(0) * x16.double().sum(0)).sum().item())
    for splitK in (2, 4):
        assert torch.equal(lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, splitK)[0], out), splitK
    for variant in (VARIANT_MFMA, VARIANT_VALU):
        assert torch.equal(lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 4, variant)[0], out), variant


KERNELS_FOR_LONG_K = {
    "mfma 32x128": (B.KERNEL_MFMA_32x128, 32), "mfma 256x256": (B.KERNEL_MFMA_256x256, 32),
    "mfma 128x64": (B.KERNEL_MFMA_128x64, 32), "split-K in the block": (B.KERNEL_SKINNY_SPLITK, 32),
    "four pieces": (B.KERNEL_SKINNY_QUAD, 32), "stream": (B.KERNEL_SKINNY_STREAM, 16), "popcount": (B.KERNEL_SKINNY_POPC, 1),
}


@pytest.mark.parametrize("kernel", list(KERNELS_FOR_LONG_K))
def test_k_just_under_2_to_24_every_term_at_its_maximum(kernel):
    """K = 2^24 - 32 with every bit set: the range term, both popcount terms and the AND-dot all lie between 2^23 and
    2^24, where a signed 24-bit multiply would misread them.  Closed forms for all-ones / all-zero / half-set
    operands in every mode; every kernel with an epilogue of its own, both engines, and the VALU design."""
    kid, N = KERNELS_FOR_LONG_K[kernel]
    K = (1 << 24) - 32
    W = K // 32
    ones = torch.full((32, W), -1, dtype=torch.int32, device=DEV)              # every sign bit set: all -1
    half = ones[:N].clone()
    half[:, ::2] = 0                                                            # every other word clear
    pb = (W // 2) * 32                                                          # W is odd: one more word clear than set
    zeros = torch.zeros((32, W), dtype=torch.int32, device=DEV)                 # all +1
    w1, w0 = lk.tile_from_logical(ones, K), lk.tile_from_logical(zeros, K)
    x1, xh = lk.tile_from_logical(ones[:N].contiguous(), K), lk.tile_from_logical(half, K)
    tern = lambda p: lk.PackedBits(p.data, p.data.clone(), 1, p.rows, p.K)     # nonzero = sign plane: every set bit is a -1
    variants = [force_kernel(kid, VARIANT_MFMA_F4)] + ([force_kernel(kid, VARIANT_MFMA)] if kid != B.KERNEL_SKINNY_POPC else [])
    if kernel == "mfma 32x128":
        variants.append(VARIANT_VALU)
    two_planes = kid not in (B.KERNEL_MFMA_256x256,)
    for variant in variants:
        def run(w, x, mode):
            out = lk.bgemm_packed_forward(w, x, mode, torch.int32, 1, variant)
            lo, hi = int(out.min()), int(out.max())
            assert lo == hi, (mode, lo, hi)
            return lo
        assert run(w1, x1, MODE_AND) == K and run(w1, x1, MODE_XOR) == K
        assert run(w1, x1, MODE_ATTN) == 0 and run(w1, x1, MODE_ATTN_X) == 0
        assert run(w0, x1, MODE_AND) == 0 and run(w0, x1, MODE_XOR) == -K
        assert run(w0, x1, MODE_ATTN) == -K and run(w0, x1, MODE_ATTN_X) == 0
        assert run(w1, xh, MODE_AND) == pb and run(w1, xh, MODE_XOR) == 2 * pb - K
        assert run(w1, xh, MODE_ATTN_X) == -(K - pb) and run(w0, xh, MODE_ATTN) == K - 2 * pb
        if two_planes:
            assert run(w1, tern(x1), MODE_BWTA) == K and run(w0, tern(x1), MODE_BWTA) == -K
            assert run(w1, tern(xh), MODE_BWTA) == pb


def test_signed_ternary_tile_k_just_under_2_to_24():
    """K = 2^24 - 32 on the signed tile: sums of +1 or -1 over all of K reach +-K, the last integers the fp32
    accumulator holds exactly; all-zero activations give 0, and rows whose nonzero entries are every other word (all
    negative) give the count of those entries with the weight's sign."""
    K = (1 << 24) - 32
    W = K // 32
    ones = torch.full((32, W), -1, dtype=torch.int32, device=DEV)
    zeros = torch.zeros((32, W), dtype=torch.int32, device=DEV)
    half = ones.clone()
    half[:, ::2] = 0
    pb = (W // 2) * 32
    w_neg, w_pos = lk.tile_from_logical(ones, K), lk.tile_from_logical(zeros, K)
    p1, p0, ph = lk.tile_from_logical(ones, K), lk.tile_from_logical(zeros, K), lk.tile_from_logical(half, K)
    tern = lambda nz, sg: lk.PackedBits(nz.data, sg.data.clone(), 1, nz.rows, nz.K)      # planes: nonzero, sign & nonzero
    variant = force_kernel(B.KERNEL_MFMA_128x256T, VARIANT_MFMA_F4)

    def run(w, x):
        out = lk.bgemm_packed_forward(w, x, MODE_BWTA, torch.int32, 1, variant)
        lo, hi = int(out.min()), int(out.max())
        assert lo == hi, (lo, hi)
        return lo
    assert run(w_neg, tern(p1, p1)) == K and run(w_pos, tern(p1, p1)) == -K          # t = -1 everywhere
    assert run(w_neg, tern(p1, p0)) == -K and run(w_pos, tern(p1, p0)) == K          # t = +1 everywhere
    assert run(w_neg, tern(p0, p0)) == 0
    assert run(w_neg, tern(ph, ph)) == pb and run(w_pos, tern(ph, p0)) == pb


KERNELS_FOR_SCALES = dict({"mfma " + t: (TILES[t], 96) for t in TILES},
                          **{"split-K in the block": (B.KERNEL_SKINNY_SPLITK, 96), "four pieces": (B.KERNEL_SKINNY_QUAD, 96),
                             "stream": (B.KERNEL_SKINNY_STREAM, 20), "popcount": (B.KERNEL_SKINNY_POPC, 2), "valu": (None, 96)})


@pytest.mark.parametrize("M", [1024, 1028, 1027])      # eight, four and one element(s) a lane in the general kernel's store
@pytest.mark.parametrize("kernel", list(KERNELS_FOR_SCALES))
def test_scaled_and_bits_kinds_with_per_row_scales_from_denormal_to_overflow(oracle, kernel, M):
    """`half(acc) * sw * sa (+ bias)` (tests/python/bgemm_linear.py:482-484) and the sign bits of its centred fp16 value
    (the next layer's `(x - zpa).to(torch.half)`, :479-482) with per-row scales from fp16's denormal range (a layer of
    M >= 13 000 output rows has sw = |W|_1 / numel there) to overflow: every kernel family, every scaled and bits kind,
    against the oracle's step-by-step rounding, bit for bit (NaN for NaN)."""
    kid, N = KERNELS_FOR_SCALES[kernel]
    K = 1024
    rng = np.random.default_rng(M * 7 + N)
    w, x = pm1(rng, M, K), pm1(rng, N, K)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    variant = VARIANT_VALU if kid is None else force_kernel(kid, VARIANT_MFMA_F4)
    acc = dense(MODE_XOR, w, x)
    for lo, hi in ((-24, -14), (-24, 6)):
        for dtype in (np.float16, np.float32):
            with np.errstate(over="ignore"):
                sw = (np.exp2(rng.integers(lo, hi + 1, M)) * (1 + rng.random(M)) * rng.choice([-1.0, 1.0], M)).astype(dtype)
                bias = (rng.standard_normal(M) * np.exp2(rng.integers(-24, 4, M))).astype(dtype)
            for sa_v in (0.7371, 61.0):
                sa = np.asarray(sa_v, dtype=dtype)
                for b in (None, bias):
                    sc = (to_dev(sw), to_dev(sa.reshape(1)), None if b is None else to_dev(b))
                    y = oracle.np_scale_epilogue(acc, sw, sa, b)
                    got = lk.bgemm_packed_forward(wp, xp, MODE_XOR, variant=variant, scale=sc)[0].cpu().numpy()
                    same = (bits_of(got) == bits_of(y)) | (np.isnan(got) & np.isnan(y))
                    assert got.dtype == y.dtype and same.all(), ("scaled", lo, hi, dtype, sa_v, b is not None, int((~same).sum()))
                    # the bits kinds: zero points a few fp16 denormal steps either side of zero, and none
                    for zp_steps in (None, 0, 3, -2, 40):
                        zp = None if zp_steps is None else np.asarray(zp_steps * 2.0 ** -24, dtype=dtype)
                        out = lk.bgemm_packed_forward(wp, xp, MODE_XOR, variant=variant, bits_out=lk.zeros_packed(N, M, 1, DEV),
                                                      scale=sc, next_zero_point=None if zp is None else to_dev(zp.reshape(1)))
                        with np.errstate(invalid="ignore", over="ignore"):
                            c = oracle.np_center_to_f16(y, dtype(0) if zp is None else zp)
                        want_bits = c.view(np.uint16) >> 15
                        logical = lk.logical_from_tiled(out).cpu().numpy().view(np.uint32)
                        got_bits = np.unpackbits(logical.byteswap().view(np.uint8), axis=1)[:, :M]
                        ok = (got_bits == want_bits) | np.isnan(c)          # the sign of a NaN (inf - inf) is not defined
                        assert ok.all(), ("bits", lo, hi, dtype, sa_v, b is not None, zp_steps, int((~ok).sum()))
