"""Parity of the HIP path against the CPU oracle, through the C ABI (ctypes shim).

Bar: bit-exact for int32 outputs; fp16 outputs equal the exact integer rounded to nearest
even (tolerance 0 ulp).  Sizes the oracle finishes in seconds are compared element by element;
the benchmark's full sizes are checked on sampled rows plus size-independent identities.
"""
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lowbit_kernel as lk
from _lib import (MODE_AND, MODE_XOR, MODE_ATTN, MODE_BWTA, MODE_ATTN_X, VARIANT_AUTO, VARIANT_VALU, VARIANT_MFMA,
                  VARIANT_MFMA_F4)
import _lib

DEV = "cuda:0"
VARIANTS = [VARIANT_VALU, VARIANT_MFMA, VARIANT_MFMA_F4]


def rand_f16(rng, rows, K, zeros=True):
    x = rng.standard_normal((rows, K)).astype(np.float16)
    if zeros and K > 4:
        idx = rng.integers(0, K, size=max(1, K // 16))
        x[:, idx] = np.float16(0.0)
        x[::2, idx[: len(idx) // 2]] = np.float16(-0.0)
    return x


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def f16_of(i32):
    with np.errstate(over="ignore"):
        return i32.astype(np.float32).astype(np.float16)


def oracle_all_modes(oracle, w, x):
    K = w.shape[1]
    Wp, Xp = oracle.c_pack_sign(w), oracle.c_pack_sign(x)
    nz, sg = oracle.c_pack_ternary(x)
    return {
        MODE_AND: oracle.c_bgemm_packed(0, Wp, Xp, K),
        MODE_XOR: oracle.c_bgemm_packed(1, Wp, Xp, K),
        MODE_ATTN: oracle.c_bgemm_packed(2, Wp, Xp, K),
        MODE_ATTN_X: np.ascontiguousarray(oracle.c_bgemm_packed(2, Xp, Wp, K).T),
        MODE_BWTA: oracle.c_bwta_packed(Wp, nz, sg, K),
    }


# ------------------------------------------------------------------ packing
def test_pack_known_answers(golden_dir):
    kat = json.load(open(os.path.join(golden_dir, "pack_kat.json")))
    for case in kat["sign"]:
        h = torch.tensor([case["halves"]], dtype=torch.int32).to(torch.int16).view(torch.half).to(DEV)
        got = lk.binary_weight_prepacking(h).cpu().numpy().view(np.uint32)
        assert [int(v) for v in got[0]] == case["words"]
        tiled = lk.pack_sign(h)
        assert [int(v) for v in lk.logical_from_tiled(tiled).cpu().numpy().view(np.uint32)[0]] == case["words"]
    for case in kat["ternary"]:
        h = torch.tensor([case["halves"]], dtype=torch.int32).to(torch.int16).view(torch.half).to(DEV)
        p = lk.pack_ternary(h)
        assert [int(v) for v in lk.logical_from_tiled(p, 0).cpu().numpy().view(np.uint32)[0]] == case["nz"]
        assert [int(v) for v in lk.logical_from_tiled(p, 1).cpu().numpy().view(np.uint32)[0]] == case["sg"]


@pytest.mark.parametrize("rows,K", [(1, 1), (3, 31), (5, 33), (32, 256), (33, 257), (7, 784), (100, 4096),
                                    (64, 520), (11008, 128)])
def test_pack_matches_oracle(oracle, rows, K):
    rng = np.random.default_rng(rows * 7919 + K)
    x = rand_f16(rng, rows, K)
    xd = to_dev(x)
    want = oracle.c_pack_sign(x)
    assert (lk.binary_weight_prepacking(xd).cpu().numpy().view(np.uint32) == want).all()
    tiled = lk.pack_sign(xd)
    assert tiled.data.numel() == ((rows + 31) // 32) * ((K + 255) // 256) * 256
    assert (lk.logical_from_tiled(tiled).cpu().numpy().view(np.uint32) == want).all()
    # logical -> tiled re-layout gives the same tiled words, padding included (all zero)
    again = lk.tile_from_logical(to_dev(want.view(np.int32)), K)
    assert torch.equal(again.data, tiled.data)
    nz, sg = oracle.c_pack_ternary(x)
    t = lk.pack_ternary(xd)
    assert (lk.logical_from_tiled(t, 0).cpu().numpy().view(np.uint32) == nz).all()
    assert (lk.logical_from_tiled(t, 1).cpu().numpy().view(np.uint32) == sg).all()


def test_pack_strided_and_unaligned(oracle):
    """Row stride > K and 2-byte-aligned starts go through the C ABI directly (the shim copies)."""
    import _lib
    L = _lib.lib()
    rng = np.random.default_rng(11)
    big = rand_f16(rng, 40, 1000)
    bd = to_dev(big)
    st = torch.cuda.current_stream().cuda_stream
    for (r0, r1, k0, k1) in [(0, 40, 0, 1000), (3, 37, 1, 778), (5, 6, 7, 8), (0, 33, 8, 520)]:
        rows, K = r1 - r0, k1 - k0
        want = oracle.c_pack_sign(big[r0:r1, k0:k1])
        src = bd.data_ptr() + 2 * (r0 * 1000 + k0)
        tiled = torch.empty(L.bgemm_tiled_words(rows, K), dtype=torch.int32, device=DEV)
        _lib.check(L.bgemm_pack_sign_f16(src, rows, K, 1000, tiled.data_ptr(), st))
        got = lk.logical_from_tiled(lk.PackedBits(tiled.view(1, -1), None, 1, rows, K))
        assert (got.cpu().numpy().view(np.uint32) == want).all()
        logical = torch.empty((rows, (K + 31) // 32), dtype=torch.int32, device=DEV)
        _lib.check(L.bgemm_pack_sign_f16_logical(src, rows, K, 1000, logical.data_ptr(), st))
        assert (logical.cpu().numpy().view(np.uint32) == want).all()


@pytest.mark.parametrize("B,K,R,pad", [(1, 1, 1, 0), (1, 300, 70, 0), (3, 512, 64, 0), (2, 1000, 33, 7), (5, 40, 200, 0)])
def test_pack_transposed_equals_pack_of_the_transpose(B, K, R, pad):
    """[B, K, R] sources packed as they lie = the ordinary pack of their transposes (ragged K and R, a row stride
    larger than R, a batch, -0.0 and NaN sign bits)."""
    g = torch.Generator(device=DEV).manual_seed(K * 7 + R)
    big = torch.randn((B, K, R + pad), generator=g, device=DEV, dtype=torch.half)
    big[:, ::3, ::5] = -0.0
    big[:, 1::7, 2::3] = float("nan")
    x = big[:, :, :R]                                         # row stride R + pad
    want = lk.pack_sign(x.transpose(1, 2).contiguous())
    got = lk.pack_sign_transposed(x)
    assert (got.batch, got.rows, got.K) == (B, R, K) and torch.equal(got.data, want.data)
    assert torch.equal(lk.pack_sign_transposed(x[0]).data, lk.pack_sign(x[0].T.contiguous()).data)
    # a source whose last dimension is strided is copied first, same bits
    assert torch.equal(lk.pack_sign_transposed(want_src := x.transpose(1, 2).contiguous().transpose(1, 2)).data, want.data)


@pytest.mark.parametrize("B,H,S,d", [(2, 3, 40, 64), (1, 2, 33, 72), (3, 1, 5, 300), (16, 12, 128, 64)])
@pytest.mark.parametrize("dtype", [torch.half, torch.float32])
def test_pack_batched_strided_views_match_oracle(oracle, B, H, S, d, dtype):
    """[B, H, S, d] views of a [B, S, H*d] tensor (what attention's head split produces) are packed where they lie, one
    launch: every matrix's tiled block equals the oracle's pack of that matrix; sign, ternary, centred, transposed;
    ragged rows (each matrix padded to whole tiles on its own), few tiles and many."""
    g = torch.Generator(device=DEV).manual_seed(B * 1000 + S)
    flat = torch.randn((B, S, H * d), generator=g, device=DEV, dtype=dtype)
    flat[:, ::3, ::5] = -0.0
    flat[:, 1::4, 1::7] = 0.0
    flat[:, 2::5, 3::11] = 1e-9 if dtype == torch.float32 else 6e-8      # fp32: rounds to +0.0 in fp16
    view = flat.view(B, S, H, d).permute(0, 2, 1, 3)
    assert not view.is_contiguous() or H == 1
    host = view.to(torch.half).cpu().numpy()
    got = lk.pack_sign(view)
    assert (got.batch, got.rows, got.K) == (B * H, S, d)
    tern = lk.pack_ternary(view)

    def logical(data, b):
        return lk.logical_from_tiled(lk.PackedBits(data[b:b + 1], None, 1, S, d)).cpu().numpy().view(np.uint32)

    for b in range(0, B * H, 1 if B * H <= 6 else 37):
        m = host[b // H, b % H]
        assert (logical(got.data, b) == oracle.c_pack_sign(m)).all(), b
        nz, sg = oracle.c_pack_ternary(m)
        assert (logical(tern.data, b) == nz).all() and (logical(tern.data2, b) == sg).all(), b
    # the same bits as the pack of a contiguous fp16 copy, padding words included
    assert torch.equal(got.data, lk.pack_sign(view.to(torch.half).contiguous()).data)
    assert torch.equal(tern.data, lk.pack_ternary(view.to(torch.half).contiguous()).data)
    assert torch.equal(tern.data2, lk.pack_ternary(view.to(torch.half).contiguous()).data2)
    # centred
    zp = flat.float().mean().to(dtype).reshape(1)
    want_c = lk.pack_sign((view - zp).to(torch.half).contiguous())
    assert torch.equal(lk.pack_sign(view, zero_point=zp).data, want_c.data)
    # transposed: the view read as [.., K = S, rows = d]
    got_t = lk.pack_sign_transposed(view)
    assert (got_t.batch, got_t.rows, got_t.K) == (B * H, d, S)
    assert torch.equal(got_t.data, lk.pack_sign(view.to(torch.half).transpose(-1, -2).contiguous()).data)
    # 3-D slices with a batch stride and a row stride of their own
    sl = flat[:, 1:, 8:8 + d]
    assert torch.equal(lk.pack_sign(sl).data, lk.pack_sign(sl.to(torch.half).contiguous()).data)
    assert torch.equal(lk.pack_sign_transposed(sl).data, lk.pack_sign(sl.to(torch.half).transpose(-1, -2).contiguous()).data)


# ------------------------------------------------------------------ packed GEMM, small and ragged
SMALL = [(1, 1, 1), (8, 5, 32), (33, 7, 40), (32, 32, 128), (10, 3, 784), (64, 1, 256), (65, 17, 300),
         (130, 70, 1000), (256, 256, 512), (40, 200, 2304),
         (260, 70, 2500), (100, 40, 2304), (33, 128, 4096)]      # two to four activation tile rows, K split in the block


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("M,N,K", SMALL)
def test_packed_small_all_modes(oracle, variant, M, N, K):
    rng = np.random.default_rng(M * 1000003 + N * 1009 + K)
    w, x = rand_f16(rng, M, K, zeros=False), rand_f16(rng, N, K)
    want = oracle_all_modes(oracle, w, x)
    wp, xp, xt = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x)), lk.pack_ternary(to_dev(x))
    for mode in (MODE_AND, MODE_XOR, MODE_ATTN, MODE_ATTN_X, MODE_BWTA):
        xin = xt if mode == MODE_BWTA else xp
        for splitK in (1, 2, 5):
            got = lk.bgemm_packed_forward(wp, xin, mode, torch.int32, splitK, variant)[0].cpu().numpy()
            assert (got == want[mode]).all(), (mode, splitK)
        goth = lk.bgemm_packed_forward(wp, xin, mode, torch.half, 3, variant)[0].cpu().numpy()
        assert (goth.view(np.uint16) == f16_of(want[mode]).view(np.uint16)).all(), mode


def test_packed_golden_dense(golden_dir):
    d = np.load(os.path.join(golden_dir, "dense_kat.npz"))
    names = {MODE_AND: "and", MODE_XOR: "xor", MODE_ATTN: "attn", MODE_ATTN_X: "attnx", MODE_BWTA: "bwta"}
    for i in range(int(d["n_cases"])):
        w = to_dev(d["w%d" % i].view(np.float16))
        x = to_dev(d["x%d" % i].view(np.float16))
        wp, xp, xt = lk.pack_sign(w), lk.pack_sign(x), lk.pack_ternary(x)
        for variant in VARIANTS:
            for mode, nm in names.items():
                got = lk.bgemm_packed_forward(wp, xt if mode == MODE_BWTA else xp, mode, torch.int32, 1, variant)
                assert (got[0].cpu().numpy() == d["%s%d" % (nm, i)]).all(), (i, nm, variant)


# ------------------------------------------------------------------ benchmark configurations
def dense_ref(mode, w, x):
    """Closed forms in fp32 on the CPU (exact: K < 2^24); the reference drivers' own method."""
    a = torch.from_numpy((w.view(np.uint16) >> 15).astype(np.float32))
    xs = x.view(np.uint16)
    b = torch.from_numpy((xs >> 15).astype(np.float32))
    if mode == MODE_XOR:
        r = (1 - 2 * b) @ (1 - 2 * a).T
    elif mode == MODE_AND:
        r = b @ a.T
    elif mode == MODE_ATTN:
        r = (1 - 2 * b) @ (1 - a).T
    elif mode == MODE_ATTN_X:
        r = (1 - b) @ (1 - 2 * a).T
    else:
        t = torch.from_numpy(np.where((xs & 0x7FFF) == 0, 0, np.where(xs >> 15, -1, 1)).astype(np.float32))
        r = t @ (1 - 2 * a).T
    return r.to(torch.int32).numpy()


def test_config1_bgemm_1024(oracle):
    g = torch.Generator().manual_seed(1001)
    a_bits = torch.randint(0, 2, (1024, 1024), generator=g).numpy()
    b_bits = torch.randint(0, 2, (1024, 64), generator=g).numpy()
    w16, x16 = oracle.bits_to_f16(a_bits), oracle.bits_to_f16(b_bits.T)
    want = oracle.c_bgemm_packed(1, oracle.c_pack_sign(w16), oracle.c_pack_sign(x16), 1024)
    wp, xp = lk.pack_sign(to_dev(w16)), lk.pack_sign(to_dev(x16))
    for variant in VARIANTS:
        for splitK in (1, 2, 4):
            got = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, splitK, variant)[0].cpu().numpy()
            assert (got == want).all()
    out = lk.bgemm_linear_forward_cuda(to_dev(x16), to_dev(w16), 1, 1).cpu().numpy()
    assert (out.view(np.uint16) == f16_of(want).view(np.uint16)).all()


@pytest.mark.parametrize("N", [1, 4, 16])
def test_config4_decode_bwta(N):
    rng = np.random.default_rng(4000 + N)
    M, K = 11008, 4096
    w = np.where(rng.integers(0, 2, (M, K)) == 1, np.float16(-1), np.float16(1)).astype(np.float16)
    t = rng.choice(np.array([-1, 0, 0, 1], dtype=np.float16), size=(N, K)).astype(np.float16)
    want = dense_ref(MODE_BWTA, w, t)
    wp, xt = lk.pack_sign(to_dev(w)), lk.pack_ternary(to_dev(t))
    for variant in [VARIANT_AUTO] + VARIANTS:
        for splitK in (1, 2, 4, 8):
            got = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, splitK, variant)[0].cpu().numpy()
            assert (got == want).all(), (variant, splitK)
    goth = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.half, 8)[0].cpu().numpy()
    assert (goth.view(np.uint16) == f16_of(want).view(np.uint16)).all()


@pytest.mark.parametrize("M,N,K", [(11008, 17, 4096), (11008, 40, 4096), (4096, 100, 4096), (1000, 130, 2304), (70, 250, 1000),
                                   (16400, 20, 6200)])      # one tile row of two planes on the four-pieces kernel
def test_decode_batches_of_ternary_rows(M, N, K):
    """More than 16 ternary rows (a batch of decode steps): the two bit planes are taken 16 rows at a time by the
    kernel that splits K inside a block, also over ragged M, N and K; same integers as the dense reference, and the
    same through the other kernel families."""
    rng = np.random.default_rng(M + N)
    w = np.where(rng.integers(0, 2, (M, K)) == 1, np.float16(-1), np.float16(1)).astype(np.float16)
    t = rng.choice(np.array([-1, 0, 0, 1], dtype=np.float16), size=(N, K)).astype(np.float16)
    want = dense_ref(MODE_BWTA, w, t)
    wp, xt = lk.pack_sign(to_dev(w)), lk.pack_ternary(to_dev(t))
    if M == 16400:
        assert lk.packed_kernel_id(wp, xt, MODE_BWTA) == _lib.KERNEL_SKINNY_QUAD
    for variant in [VARIANT_AUTO] + VARIANTS:
        got = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32, 1, variant)[0].cpu().numpy()
        assert (got == want).all(), variant
    goth = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.half, 8)[0].cpu().numpy()
    assert (goth.view(np.uint16) == f16_of(want).view(np.uint16)).all()
    # a batch of weight matrices against shared rows
    wp3 = lk.PackedBits(torch.cat([wp.data, wp.data.flip(1)], 0), None, 2, M, K)
    got3 = lk.bgemm_packed_forward(wp3, xt, MODE_BWTA, torch.int32)
    assert (got3[0].cpu().numpy() == want).all()
    assert torch.equal(got3[1], lk.bgemm_packed_forward(lk.PackedBits(wp.data.flip(1).contiguous(), None, 1, M, K), xt, MODE_BWTA, torch.int32)[0])


@pytest.mark.parametrize("batch,M,N,K", [(1, 4040, 270, 6200), (4, 1000, 250, 6200), (1, 8192, 256, 8192),
                                         (1, 4096, 384, 12288), (1, 4096, 512, 8192)])      # the last two: four / two K ways, several blocks a CU
def test_split_k_in_block_four_pieces_a_block(oracle, batch, M, N, K):
    """Outputs of one to two thousand 32 x 32 pieces over a long K: a block takes two weight row tiles and two
    activation tile rows (odd tile counts, ragged M, N and K, batches); every one-plane mode, both engines,
    every output kind, against the dense reference and the oracle's epilogue."""
    rng = np.random.default_rng(batch + M + N + K)
    w = rand_f16(rng, batch * M, K).reshape(batch, M, K)
    x = rand_f16(rng, batch * N, K).reshape(batch, N, K)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    xt = lk.pack_ternary(to_dev(x))
    assert lk.packed_kernel_id(wp, xp, MODE_XOR, 8) == _lib.KERNEL_SKINNY_QUAD
    # two planes take this kernel up to 512 blocks (one round); past that the general kernel's tiles: forced below
    blocks2 = batch * -(-(-(-M // 32)) // 2) * -(-N // 32)
    assert (lk.packed_kernel_id(wp, xt, MODE_BWTA, 8) == _lib.KERNEL_SKINNY_QUAD) == (blocks2 <= 512)
    for mode in (MODE_XOR, MODE_AND, MODE_ATTN, MODE_ATTN_X, MODE_BWTA):     # ternary: the two planes of a tile row are the block's two operands
        want = np.stack([dense_ref(mode, w[b], x[b]) for b in range(batch)])
        xo = xt if mode == MODE_BWTA else xp
        for variant in (VARIANT_AUTO, VARIANT_MFMA, _lib.force_kernel(_lib.KERNEL_SKINNY_QUAD)):
            got = lk.bgemm_packed_forward(wp, xo, mode, torch.int32, 8, variant).cpu().numpy()
            assert (got == want).all(), (mode, variant)
        for variant in (VARIANT_AUTO, _lib.force_kernel(_lib.KERNEL_SKINNY_QUAD)):
            goth = lk.bgemm_packed_forward(wp, xo, mode, torch.half, 1, variant).cpu().numpy()
            assert (goth.view(np.uint16) == f16_of(want).view(np.uint16)).all(), (mode, variant)
    acc = np.stack([dense_ref(MODE_XOR, w[b], x[b]) for b in range(batch)])
    acct = np.stack([dense_ref(MODE_BWTA, w[b], x[b]) for b in range(batch)]).reshape(batch * N, M)
    swt, sat = rng.uniform(1e-4, 3e-3, M).astype(np.float32), np.asarray(0.61, dtype=np.float32)
    gott = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, scale=(to_dev(swt), to_dev(sat.reshape(1)), None)).cpu().numpy()
    assert (_bits(gott.reshape(batch * N, M)) == _bits(oracle.np_scale_epilogue(acct, swt, sat, None))).all()
    for dtype in (np.float32, np.float16):
        sw = rng.uniform(1e-4, 3e-3, M).astype(dtype)
        sa = np.asarray(1.7371, dtype=dtype)
        bias = rng.standard_normal(M).astype(dtype)
        scale = (to_dev(sw), to_dev(sa.reshape(1)), to_dev(bias))
        y = oracle.np_scale_epilogue(acc.reshape(batch * N, M), sw, sa, bias)
        got = lk.bgemm_packed_forward(wp, xp, MODE_XOR, scale=scale).cpu().numpy()
        assert (_bits(got.reshape(batch * N, M)) == _bits(y)).all(), dtype
        zp = np.asarray(0.013, dtype=dtype)
        out = lk.bgemm_packed_forward(wp, xp, MODE_XOR, scale=scale, bits_out=lk.zeros_packed(N, M, batch, DEV),
                                      next_zero_point=to_dev(zp.reshape(1)))
        wantb = oracle.c_pack_sign(oracle.np_center_to_f16(y, zp))
        for b in range(batch):
            one = lk.PackedBits(out.data[b:b + 1], None, 1, N, M)
            assert (lk.logical_from_tiled(one).cpu().numpy().view(np.uint32) == wantb[b * N:(b + 1) * N]).all(), (dtype, b)


def test_config3_attention_av_batched():
    rng = np.random.default_rng(3000)
    B, S, D = 24, 512, 64                      # 24 of the 192 heads element by element
    attn_bits = rng.integers(0, 2, (B, S, S))  # {0,1}, 1 = attend
    v = np.where(rng.integers(0, 2, (B, S, D)) == 1, np.float16(-1), np.float16(1)).astype(np.float16)
    attn16 = (2 * attn_bits - 1).astype(np.float16)            # "1" must have its sign bit clear
    want = np.einsum("bqk,bkd->bqd", attn_bits.astype(np.float32), v.astype(np.float32)).astype(np.int32)
    vt = np.ascontiguousarray(v.transpose(0, 2, 1))            # [B, D, S_k]
    ap, vp = lk.pack_sign(to_dev(attn16)), lk.pack_sign(to_dev(vt))
    for variant in [VARIANT_AUTO] + VARIANTS:
        # weight side = value^T (M = D), activation side = attn (N = S_q): output [B, S_q, D] directly
        got = lk.bgemm_packed_forward(vp, ap, MODE_ATTN_X, torch.int32, 1, variant).cpu().numpy()
        assert (got == want).all()
        # the reference's orientation (attn as the weight side, INSTR=2) gives the transpose
        got_t = lk.bgemm_packed_forward(ap, vp, MODE_ATTN, torch.int32, 1, variant).cpu().numpy()
        assert (got_t.transpose(0, 2, 1) == want).all()


@pytest.mark.parametrize("M,N,K,splitK", [(8192, 256, 4096, 1), (8192, 256, 4096, 4), (8192, 2048, 4096, 2),
                                          (4096, 128, 4096, 1), (4096, 128, 784, 1), (10, 128, 4096, 4)])
def test_config5_sweep_mid(M, N, K, splitK):
    rng = np.random.default_rng(M + N + K + splitK)
    w = np.where(rng.integers(0, 2, (M, K)) == 1, np.float16(-1), np.float16(1)).astype(np.float16)
    x = np.where(rng.integers(0, 2, (N, K)) == 1, np.float16(-1), np.float16(1)).astype(np.float16)
    want = dense_ref(MODE_XOR, w, x)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    for variant in VARIANTS:
        got = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, splitK, variant)[0].cpu().numpy()
        assert (got == want).all(), variant


def test_config5_full_8192_sampled_and_identities():
    M = N = K = 8192
    g = torch.Generator(device=DEV).manual_seed(5000)
    wbits = torch.randint(0, 2, (M, K), generator=g, device=DEV, dtype=torch.int8)
    xbits = torch.randint(0, 2, (N, K), generator=g, device=DEV, dtype=torch.int8)
    w16 = (1 - 2 * wbits).to(torch.half)
    x16 = (1 - 2 * xbits).to(torch.half)
    wp, xp = lk.pack_sign(w16), lk.pack_sign(x16)
    out = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1, VARIANT_MFMA)[0]
    # (1) sampled rows/columns against the fp32 closed form on the CPU
    rs = np.random.default_rng(5).choice(M, 96, replace=False)
    cs = np.random.default_rng(6).choice(N, 80, replace=False)
    wsub = w16[torch.from_numpy(rs).to(DEV)].float().cpu()
    xsub = x16[torch.from_numpy(cs).to(DEV)].float().cpu()
    want = (xsub @ wsub.T).to(torch.int32)
    got = out[torch.from_numpy(cs).to(DEV)][:, torch.from_numpy(rs).to(DEV)].cpu()
    assert torch.equal(got, want)
    # (2) identities over the whole output: parity, range, checksum of checksums
    assert int(((out - K) % 2).abs().max()) == 0 and int(out.abs().max()) <= K
    col_sum = (1 - 2 * wbits).to(torch.float64).sum(0)               # sum_m s(w[m,k])
    row_sum = (1 - 2 * xbits).to(torch.float64).sum(0)               # sum_n s(x[n,k])
    assert int(out.to(torch.int64).sum()) == int((col_sum * row_sum).sum().item())
    # (3) split-K and the VALU design agree bit for bit with the MFMA design
    assert torch.equal(lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 4, VARIANT_MFMA)[0], out)
    assert torch.equal(lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1, VARIANT_VALU)[0], out)
    assert torch.equal(lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1, VARIANT_MFMA_F4)[0], out)
    assert torch.equal(lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 2, VARIANT_MFMA_F4)[0], out)
    # (4) C(w, w) has K on the diagonal; negating the weights negates the output
    assert int(lk.bgemm_packed_forward(wp, wp, MODE_XOR, torch.int32)[0].diagonal().min()) == K
    assert torch.equal(lk.bgemm_packed_forward(lk.pack_sign(-w16), xp, MODE_XOR, torch.int32)[0], -out)


@pytest.mark.parametrize("variant", [VARIANT_MFMA, VARIANT_MFMA_F4, VARIANT_VALU])
def test_large_k_accumulators_stay_exact(variant):
    """Worst case for the accumulators: every bit set, so the AND-dot equals K.  K = 2^22 keeps the fp4
    engine's fp32 accumulator far above the point where a narrower internal adder would lose bits."""
    K = 1 << 22
    ones = torch.full((32, K // 32), -1, dtype=torch.int32, device=DEV)         # all sign bits set
    half_ones = ones.clone()
    half_ones[:, ::2] = 0                                                        # every other word clear
    wp, xp = lk.tile_from_logical(ones, K), lk.tile_from_logical(half_ones, K)
    assert int(lk.bgemm_packed_forward(wp, wp, MODE_AND, torch.int32, 1, variant).min()) == K
    assert int(lk.bgemm_packed_forward(wp, wp, MODE_XOR, torch.int32, 1, variant).min()) == K
    got = lk.bgemm_packed_forward(wp, xp, MODE_AND, torch.int32, 3, variant)
    assert int(got.min()) == K // 2 and int(got.max()) == K // 2
    assert int(lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1, variant).abs().max()) == 0


# ------------------------------------------------------------------ drop-in fp16 entry point
@pytest.mark.parametrize("M,N,K", [(32, 32, 128), (64, 96, 640), (800, 128, 128), (10, 128, 4096), (33, 5, 100)])
@pytest.mark.parametrize("INSTR", [0, 1, 2])
def test_dropin_matches_reference_call(oracle, M, N, K, INSTR):
    rng = np.random.default_rng(M * 31 + N * 17 + K + INSTR)
    w, x = rand_f16(rng, M, K), rand_f16(rng, N, K)
    for splitK in (1, 3):
        want_h, _ = oracle.c_bgemm_f16(x, w, splitK, INSTR)
        got = lk.bgemm_linear_forward_cuda(to_dev(x), to_dev(w), splitK, INSTR)
        assert got.dtype == torch.half and tuple(got.shape) == (N, M)
        assert (got.cpu().numpy().view(np.uint16) == want_h.view(np.uint16)).all()


def test_dropin_rounds_to_nearest_even(oracle):
    K = 4224
    w = -np.ones((32, K), dtype=np.float16)
    x = np.ones((32, K), dtype=np.float16)
    x[:, :4099] = -1
    got = lk.bgemm_linear_forward_cuda(to_dev(x), to_dev(w), 1, 0).cpu().numpy()
    assert (got == np.float16(4100)).all()
    want_h, _ = oracle.c_bgemm_f16(x, w, 1, 0)
    assert (got.view(np.uint16) == want_h.view(np.uint16)).all()


def test_dropin_weight_cache_is_opt_in_and_follows_the_tensor():
    """With the cache on, the drop-in call packs a weight tensor once; a write through torch (version counter)
    or another tensor object gets a fresh pack; results never differ from the uncached call."""
    torch.manual_seed(9)
    x = torch.randn(5, 300, device=DEV, dtype=torch.half)
    w = torch.randn(70, 300, device=DEV, dtype=torch.half)
    plain = lk.bgemm_linear_forward_cuda(x, w, 1, 1)
    assert len(lk._weight_cache) == 0                                  # off by default
    lk.set_weight_cache(2)
    try:
        for instr in (0, 1, 2):
            assert torch.equal(lk.bgemm_linear_forward_cuda(x, w, 1, instr), lk.bgemm_linear_forward_cuda(x, w.clone(), 1, instr))
        assert torch.equal(lk.bgemm_linear_forward_cuda(x, w, 4, 1), plain)
        packed = lk._weight_cache[id(w)][3]
        assert lk.bgemm_linear_forward_cuda(x, w, 1, 1) is not None and lk._weight_cache[id(w)][3] is packed   # reused
        w.neg_()                                                        # in-place write: must be packed again
        assert torch.equal(lk.bgemm_linear_forward_cuda(x, w, 1, 1), -plain)
        assert lk._weight_cache[id(w)][3] is not packed
        for _ in range(4):                                              # other tensors push old entries out
            lk.bgemm_linear_forward_cuda(x, torch.randn_like(w), 1, 1)
        assert len(lk._weight_cache) <= 2
        with pytest.raises(ValueError):
            lk.bgemm_linear_forward_cuda(x, w, 1, 3)
    finally:
        lk.set_weight_cache(0)
    assert len(lk._weight_cache) == 0


def test_dropin_argument_errors():
    x = torch.zeros(32, 128, dtype=torch.half, device=DEV)
    with pytest.raises(TypeError):
        lk.bgemm_linear_forward_cuda(x.float(), x)
    with pytest.raises(ValueError):
        lk.bgemm_linear_forward_cuda(x, x[:, :64])
    with pytest.raises(ValueError):
        lk.bgemm_linear_forward_cuda(x, x, 1, 3)
    with pytest.raises(ValueError):
        lk.bgemm_linear_forward_cuda(x, x, 0, 1)


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("M,N,K,splits", [(130, 170, 16384, (2,)), (100, 200, 40000, (3, 5, 8)), (300, 260, 24800, (2, 4))])
def test_split_k_handover_long_k(oracle, variant, M, N, K, splits):
    """Shapes with few output tiles and a long K, where K is really split: across blocks in the VALU family (K is
    only split while every range keeps 24 K-tiles; partial tiles through the workspace, tickets), among the waves
    of a block, without a workspace, in the matrix-core family.  All modes and output kinds."""
    import _lib
    rng = np.random.default_rng(M + N + K)
    w, x = rand_f16(rng, M, K), rand_f16(rng, N, K)
    Wp, Xp = oracle.c_pack_sign(w), oracle.c_pack_sign(x)
    nz, sg = oracle.c_pack_ternary(x)
    want = {MODE_XOR: oracle.c_bgemm_packed(1, Wp, Xp, K), MODE_ATTN: oracle.c_bgemm_packed(2, Wp, Xp, K),
            MODE_BWTA: oracle.c_bwta_packed(Wp, nz, sg, K)}
    wp, xp, xt = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x)), lk.pack_ternary(to_dev(x))
    L = _lib.lib()
    for sk in splits:
        assert (L.bgemm_packed_workspace_bytes(MODE_BWTA, 1, M, N, K, sk, variant) > 0) == (variant == VARIANT_VALU)
        for mode in (MODE_XOR, MODE_ATTN, MODE_BWTA):
            got = lk.bgemm_packed_forward(wp, xt if mode == MODE_BWTA else xp, mode, torch.int32, sk, variant)
            assert (got[0].cpu().numpy() == want[mode]).all(), (mode, sk)
        goth = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.half, sk, variant)[0].cpu().numpy()
        assert (goth.view(np.uint16) == f16_of(want[MODE_XOR]).view(np.uint16)).all()
    sw = rng.uniform(1e-4, 3e-3, M).astype(np.float32)
    gots = lk.bgemm_packed_forward(wp, xp, MODE_XOR, splitK=splits[-1], variant=variant,
                                   scale=(to_dev(sw), torch.full((1,), 0.75, device=DEV), None))[0].cpu().numpy()
    assert (_bits(gots) == _bits(oracle.np_scale_epilogue(want[MODE_XOR], sw, np.float32(0.75), None))).all()


def test_split_k_workspace_left_clean():
    rng = np.random.default_rng(77)
    w, x = rand_f16(rng, 96, 16384, zeros=False), rand_f16(rng, 200, 16384, zeros=False)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    first = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 4, VARIANT_MFMA)
    for variant in VARIANTS:
        for _ in range(3):
            assert torch.equal(lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 4, variant), first)
    torch.cuda.synchronize()
    assert lk._counters
    for buf in lk._counters.values():
        assert int(buf.count_nonzero()) == 0


# ------------------------------------------------------------------ fused layer prologue / epilogue
def _bits(a):
    return a.view(np.uint32 if a.dtype == np.float32 else np.uint16)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("rows,K", [(5, 33), (64, 784), (33, 1000), (128, 4096)])
def test_pack_centered_matches_oracle(oracle, dtype, rows, K):
    rng = np.random.default_rng(rows * 7 + K)
    x = rng.standard_normal((rows, K)).astype(dtype)
    zp = np.asarray(x.mean(), dtype=dtype)
    x[0, 0], x[-1, -1] = zp, np.nextafter(zp, np.asarray(-9, dtype))       # exactly at / just below the zero point
    want = oracle.c_pack_sign(oracle.np_center_to_f16(x, zp))
    got = lk.logical_from_tiled(lk.pack_sign(to_dev(x), zero_point=to_dev(zp.reshape(1))))
    assert (got.cpu().numpy().view(np.uint32) == want).all()
    # zero_point = 0 is the plain sign pack of the rounded source
    got0 = lk.logical_from_tiled(lk.pack_sign(to_dev(x), zero_point=torch.zeros(1, device=DEV)))
    assert (got0.cpu().numpy().view(np.uint32) == oracle.c_pack_sign(x.astype(np.float16))).all()


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("M,N,K,splitK,with_bias", [(96, 40, 784, 1, True), (10, 128, 4096, 3, True),
                                                    (4096, 128, 784, 1, False), (260, 7, 300, 2, True),
                                                    (130, 70, 2500, 1, True)])
def test_scaled_epilogue_matches_oracle(oracle, variant, dtype, M, N, K, splitK, with_bias):
    rng = np.random.default_rng(M + N + K)
    w, x = rand_f16(rng, M, K), rand_f16(rng, N, K)
    sw = rng.uniform(1e-4, 3e-3, M).astype(dtype)
    sa = np.asarray(1.7371, dtype=dtype)
    bias = rng.standard_normal(M).astype(dtype) if with_bias else None
    acc = oracle.c_bgemm_packed(1, oracle.c_pack_sign(w), oracle.c_pack_sign(x), K)
    want = oracle.np_scale_epilogue(acc, sw, sa, bias)
    got = lk.bgemm_packed_forward(lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x)), MODE_XOR, splitK=splitK,
                                  variant=variant,
                                  scale=(to_dev(sw), to_dev(sa.reshape(1)), to_dev(bias) if with_bias else None))
    got = got[0].cpu().numpy()
    assert got.dtype == want.dtype and (_bits(got) == _bits(want)).all()


def test_scaled_epilogue_empty_k_and_errors():
    sw, sa, b = torch.full((8,), 0.5, device=DEV), torch.ones(1, device=DEV), torch.arange(8.0, device=DEV)
    w0 = lk.PackedBits(torch.empty((1, 0), dtype=torch.int32, device=DEV), None, 1, 8, 0)
    x0 = lk.PackedBits(torch.empty((1, 0), dtype=torch.int32, device=DEV), None, 1, 3, 0)
    out = lk.bgemm_packed_forward(w0, x0, MODE_XOR, scale=(sw, sa, b))
    assert torch.equal(out[0], b.expand(3, 8))                         # 0 * sw * sa + bias
    out = lk.bgemm_packed_forward(w0, x0, MODE_XOR, out_dtype=torch.half)
    assert torch.equal(out, torch.zeros_like(out))
    w = lk.pack_sign(torch.randn(8, 64, device=DEV))
    x = lk.pack_sign(torch.randn(3, 64, device=DEV))
    with pytest.raises(ValueError):
        lk.bgemm_packed_forward(w, x, MODE_XOR, scale=(sw[:4], sa, b))
    with pytest.raises(ValueError):
        lk.bgemm_packed_forward(w, x, MODE_XOR, scale=(sw, sa, b.half()))


# ------------------------------------------------------------------ decode step on unpacked activations
@pytest.mark.parametrize("variant", [VARIANT_AUTO, VARIANT_MFMA, VARIANT_MFMA_F4])
@pytest.mark.parametrize("M,N,K", [(11008, 1, 4096), (4100, 4, 1000), (300, 2, 40), (64, 4, 2500), (1000, 3, 256), (33, 1, 8), (500, 16, 512),
                                   # several rounds of K-tiles a wave (rows requested a round ahead); sixteen ways a block
                                   (8200, 4, 6400), (4096, 4, 11008), (1000, 3, 8200), (1000, 2, 11008)])
def test_decode_step_packs_its_own_activations(variant, M, N, K):
    """One launch on fp16 / fp32 activations = pack launch + packed GEMM, bit for bit: every mode, ternary planes,
    zero point, strided rows, scaled output."""
    g = torch.Generator(device=DEV).manual_seed(M + 7 * N + K)
    w = torch.randn((M, K), generator=g, device=DEV, dtype=torch.half)
    wide = torch.randn((N, K + 24), generator=g, device=DEV, dtype=torch.float32)
    wide[:, ::4] = 0
    wide[:, 1::9] = -0.0
    wp = lk.pack_sign(w)
    for dt in (torch.half, torch.float32):
        x = wide.to(dt)[:, 8:8 + K]                       # row stride K + 24, rows not 16-byte aligned for odd K
        for mode in (MODE_XOR, MODE_AND, MODE_ATTN, MODE_ATTN_X, MODE_BWTA):
            if mode == MODE_BWTA and N > 16:
                continue
            xp = lk.pack_ternary(x) if mode == MODE_BWTA else lk.pack_sign(x)
            want = lk.bgemm_packed_forward(wp, xp, mode, torch.int32, 1, variant)[0]
            assert torch.equal(lk.bgemm_packed_weight_forward(wp, x, mode, torch.int32, variant=variant), want), (dt, mode)
        zp = x.mean().reshape(1)
        sw = (torch.rand(M, generator=g, device=DEV) + 0.5).to(dt)
        sa, bias = torch.tensor([0.37], device=DEV, dtype=dt), torch.randn(M, generator=g, device=DEV).to(dt)
        want = lk.bgemm_packed_forward(wp, lk.pack_sign(x, zero_point=zp), MODE_XOR, splitK=1, variant=variant, scale=(sw, sa, bias))[0]
        got = lk.bgemm_packed_weight_forward(wp, x, MODE_XOR, scale=(sw, sa, bias), x_zero_point=zp, variant=variant)
        assert got.dtype == dt and torch.equal(got, want), dt
    assert torch.equal(lk.bgemm_packed_weight_forward(wp, x, MODE_XOR, torch.half), lk.bgemm_packed_forward(wp, lk.pack_sign(x), MODE_XOR, torch.half)[0])


@pytest.mark.parametrize("batch,M,N,K", [(1, 11008, 1, 4096), (1, 4100, 2, 1000), (3, 70, 2, 5000), (1, 33, 1, 8), (2, 1000, 1, 11008)])
def test_one_or_two_rows_on_the_vector_alu(oracle, batch, M, N, K):
    """One or two activation vectors (rows x bit planes) take the AND-popcount kernel: every mode against the dense
    reference (batches, ragged M and K, one to 43 K-tiles), fp16, the layer epilogue and the bits output against
    the oracle, and the same from unpacked fp16 / fp32 rows with a zero point."""
    rng = np.random.default_rng(batch + M + N + K)
    w = rand_f16(rng, batch * M, K).reshape(batch, M, K)
    x = rand_f16(rng, batch * N, K).reshape(batch, N, K)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    for mode in (MODE_XOR, MODE_AND, MODE_ATTN, MODE_ATTN_X, MODE_BWTA):
        if mode == MODE_BWTA and N > 1:
            continue                                    # two ternary rows are four vectors: the matrix-core kernel's
        want = np.stack([dense_ref(mode, w[b], x[b]) for b in range(batch)])
        xo = lk.pack_ternary(to_dev(x)) if mode == MODE_BWTA else xp
        for splitK in (1, 8):
            got = lk.bgemm_packed_forward(wp, xo, mode, torch.int32, splitK).cpu().numpy()
            assert (got == want).all(), (mode, splitK)
        goth = lk.bgemm_packed_forward(wp, xo, mode, torch.half, 1).cpu().numpy()
        assert (goth.view(np.uint16) == f16_of(want).view(np.uint16)).all(), mode
        if batch == 1:                                  # the same from the rows as they are
            for dt in (torch.half, torch.float32):
                got1 = lk.bgemm_packed_weight_forward(lk.PackedBits(wp.data, None, 1, M, K), to_dev(x[0]).to(dt), mode, torch.int32)
                assert (got1.cpu().numpy() == want[0]).all(), (mode, dt)
    acc = np.stack([dense_ref(MODE_XOR, w[b], x[b]) for b in range(batch)]).reshape(batch * N, M)
    for dtype in (np.float32, np.float16):
        sw = rng.uniform(1e-4, 3e-3, M).astype(dtype)
        sa = np.asarray(1.7371, dtype=dtype)
        bias = rng.standard_normal(M).astype(dtype)
        scale = (to_dev(sw), to_dev(sa.reshape(1)), to_dev(bias))
        y = oracle.np_scale_epilogue(acc, sw, sa, bias)
        got = lk.bgemm_packed_forward(wp, xp, MODE_XOR, scale=scale).cpu().numpy()
        assert (_bits(got.reshape(batch * N, M)) == _bits(y)).all(), dtype
        zp = np.asarray(0.013, dtype=dtype)
        out = lk.bgemm_packed_forward(wp, xp, MODE_XOR, scale=scale, bits_out=lk.zeros_packed(N, M, batch, DEV),
                                      next_zero_point=to_dev(zp.reshape(1)))
        wantb = oracle.c_pack_sign(oracle.np_center_to_f16(y, zp))
        for b in range(batch):
            one = lk.PackedBits(out.data[b:b + 1], None, 1, N, M)
            assert (lk.logical_from_tiled(one).cpu().numpy().view(np.uint32) == wantb[b * N:(b + 1) * N]).all(), (dtype, b)
    if batch == 1:      # unpacked rows with a zero point: the sign bits of (x - zp).half(), as the centring pack forms them
        xd = to_dev(x[0]).float()
        zpt = xd.mean().reshape(1)
        want = lk.bgemm_packed_forward(wp, lk.pack_sign(xd, zero_point=zpt), MODE_XOR, torch.int32, 1, VARIANT_MFMA)[0]
        assert torch.equal(lk.bgemm_packed_weight_forward(wp, xd, MODE_XOR, torch.int32, x_zero_point=zpt), want)


def test_decode_step_larger_batches_fall_back_to_two_launches():
    g = torch.Generator(device=DEV).manual_seed(3)
    w = torch.randn((500, 700), generator=g, device=DEV, dtype=torch.half)
    x = torch.randn((77, 700), generator=g, device=DEV, dtype=torch.half)
    wp = lk.pack_sign(w)
    assert torch.equal(lk.bgemm_packed_weight_forward(wp, x, MODE_XOR), lk.bgemm_packed_forward(wp, lk.pack_sign(x), MODE_XOR)[0])
    xt = torch.sign(x[:20])
    assert torch.equal(lk.bgemm_packed_weight_forward(wp, xt, MODE_BWTA), lk.bgemm_packed_forward(wp, lk.pack_ternary(xt), MODE_BWTA)[0])
    with pytest.raises(ValueError):
        lk.bgemm_packed_weight_forward(wp, x[:, :100], MODE_XOR)


# ------------------------------------------------------------------ random shapes through every path
@pytest.mark.parametrize("seed", range(96))
def test_random_shapes_modes_kinds(seed):
    """Seeded random shapes (ragged in every dimension, batches, K from one bit to twenty K-tiles), every
    mode, every kernel design, int32 and fp16 stores, any splitK: bit-exact against the +-1 / {0,1} matmul."""
    rng = np.random.default_rng(7000 + seed)
    B = int(rng.choice([1, 1, 2, 5]))
    M = int(rng.choice([rng.integers(1, 64), rng.integers(64, 1500), rng.integers(1500, 6000)]))
    N = int(rng.choice([rng.integers(1, 17), rng.integers(17, 200), rng.integers(200, 900)]))
    K = int(rng.choice([rng.integers(1, 256), rng.integers(256, 2048), rng.integers(2048, 5200)]))
    mode = int(rng.choice([MODE_AND, MODE_XOR, MODE_ATTN, MODE_ATTN_X, MODE_BWTA]))
    variant = int(rng.choice([VARIANT_AUTO, VARIANT_VALU, VARIANT_MFMA, VARIANT_MFMA_F4]))
    splitK = int(rng.choice([1, 2, 3, 8]))
    dt = torch.half if rng.integers(0, 2) else torch.int32
    g = torch.Generator(device=DEV).manual_seed(seed)
    w = torch.randn((B, M, K), generator=g, device=DEV, dtype=torch.half)
    x = torch.randn((B, N, K), generator=g, device=DEV, dtype=torch.half)
    x[:, :, ::3] = 0
    ws, xs = torch.where(torch.signbit(w), -1.0, 1.0), torch.where(torch.signbit(x), -1.0, 1.0)
    want = {MODE_XOR: lambda: xs @ ws.transpose(1, 2),
            MODE_AND: lambda: (xs < 0).float() @ (ws < 0).float().transpose(1, 2),
            MODE_ATTN: lambda: xs @ (ws > 0).float().transpose(1, 2),
            MODE_ATTN_X: lambda: (xs > 0).float() @ ws.transpose(1, 2),
            MODE_BWTA: lambda: torch.sign(x.float()) @ ws.transpose(1, 2)}[mode]()
    xin = lk.pack_ternary(x) if mode == MODE_BWTA else lk.pack_sign(x)
    got = lk.bgemm_packed_forward(lk.pack_sign(w), xin, mode, dt, splitK, variant)
    case = (B, M, N, K, mode, variant, splitK, dt)
    assert tuple(got.shape) == (B, N, M), case
    assert torch.equal(got, want.to(torch.int32) if dt == torch.int32 else want.half()), case


# ------------------------------------------------------------------ skinny shapes with many row tiles
@pytest.mark.parametrize("B,M,N,K", [(40, 4100, 5, 300),      # 5160 row tiles: one per wave, ragged M and K
                                     (70, 4000, 16, 2304),    # 8750 row tiles: two per wave, nine K-tiles
                                     (1, 262144 + 40, 1, 256),# one tall matrix, odd number of row tiles
                                     (33, 8000, 32, 1000)])   # 32 binary activation rows
def test_skinny_streaming_batched(B, M, N, K):
    g = torch.Generator(device=DEV).manual_seed(B * 31 + N)
    w = torch.randn((B, M, K), generator=g, device=DEV, dtype=torch.half)
    x = torch.randn((N, K), generator=g, device=DEV, dtype=torch.half)
    x[:, ::5] = 0
    wp, xp, xt = lk.pack_sign(w), lk.pack_sign(x), lk.pack_ternary(x)
    ws, xs = torch.where(torch.signbit(w), -1.0, 1.0), torch.where(torch.signbit(x), -1.0, 1.0)
    want = {
        MODE_XOR: xs @ ws.transpose(1, 2),
        MODE_AND: (xs < 0).float() @ (ws < 0).float().transpose(1, 2),
        MODE_ATTN: xs @ (ws > 0).float().transpose(1, 2),
        MODE_ATTN_X: (xs > 0).float() @ ws.transpose(1, 2),
        MODE_BWTA: torch.sign(x.float()) @ ws.transpose(1, 2),
    }
    for mode in ([MODE_XOR, MODE_AND, MODE_ATTN, MODE_ATTN_X] + ([MODE_BWTA] if N <= 16 else [])):
        got = lk.bgemm_packed_forward(wp, xt if mode == MODE_BWTA else xp, mode, torch.int32)
        assert tuple(got.shape) == (B, N, M) and torch.equal(got, want[mode].to(torch.int32)), mode
    variants = {v: lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.half, 1, v) for v in (VARIANT_MFMA, VARIANT_MFMA_F4)}
    for v, got in variants.items():
        assert torch.equal(got, want[MODE_XOR].half()), v


def test_packed_file_round_trip_on_device(tmp_path):
    """Weights prepacked once, written to disk, read back: same bits, same GEMM."""
    rng = np.random.default_rng(77)
    w, x = rand_f16(rng, 300, 1000), rand_f16(rng, 9, 1000)
    wp, xt = lk.pack_sign(to_dev(w)), lk.pack_ternary(to_dev(x))
    pw, px = str(tmp_path / "w.bgpk"), str(tmp_path / "x.bgpk")
    lk.save_packed(pw, wp)
    lk.save_packed(px, xt)
    wp2, xt2 = lk.load_packed(pw, DEV), lk.load_packed(px, DEV)
    assert torch.equal(wp2.data, wp.data) and torch.equal(xt2.data, xt.data) and torch.equal(xt2.data2, xt.data2)
    a = lk.bgemm_packed_forward(wp, xt, MODE_BWTA, torch.int32)
    b = lk.bgemm_packed_forward(wp2, xt2, MODE_BWTA, torch.int32)
    assert torch.equal(a, b) and (a[0].cpu().numpy() == dense_ref(MODE_BWTA, w, x)).all()


# ------------------------------------------------------------------ binary layer feeding a binary layer: bits out
@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("M,N,K,splitK,batch", [(96, 40, 784, 1, 1),        # general kernel, ragged everything
                                                 (300, 128, 4096, 1, 1),     # skinny split-K, four tile rows
                                                 (4100, 5, 300, 1, 3),       # skinny split-K, one tile row, batched
                                                 (260, 70, 24800, 4, 1),     # cross-block split-K
                                                 (512, 256, 512, 1, 2),      # whole tiles, batched
                                                 (10, 128, 4096, 1, 1)])     # a single weight row tile
def test_bits_output_is_next_layers_operand(oracle, variant, dtype, M, N, K, splitK, batch):
    """The GEMM writes the next binary layer's packed operand directly: the bits must be those of
    pack_sign((half(acc) * sw * sa + bias - zp).half()) evaluated op by op."""
    rng = np.random.default_rng(M * 3 + N * 5 + K)
    w = rng.standard_normal((batch, M, K)).astype(np.float16)
    x = rng.standard_normal((batch, N, K)).astype(np.float16)
    sw = rng.uniform(1e-4, 3e-3, M).astype(dtype)
    sa = np.asarray(1.7371, dtype=dtype)
    bias = (0.05 * rng.standard_normal(M)).astype(dtype)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    for zp_val in (None, 0.013):
        zp = None if zp_val is None else np.asarray(zp_val, dtype=dtype)
        out = lk.zeros_packed(N, M, batch, DEV)
        got = lk.bgemm_packed_forward(wp, xp, MODE_XOR, splitK=splitK, variant=variant, bits_out=out,
                                      scale=(to_dev(sw), to_dev(sa.reshape(1)), to_dev(bias)),
                                      next_zero_point=None if zp is None else to_dev(zp.reshape(1)))
        assert got is out
        for b in range(batch):
            acc = oracle.c_bgemm_packed(1, oracle.c_pack_sign(w[b]), oracle.c_pack_sign(x[b]), K)
            y = oracle.np_scale_epilogue(acc, sw, sa, bias)
            want = oracle.c_pack_sign(oracle.np_center_to_f16(y, dtype(0) if zp is None else zp))
            one = lk.PackedBits(out.data[b:b + 1], None, 1, N, M)
            assert (lk.logical_from_tiled(one).cpu().numpy().view(np.uint32) == want).all(), (zp_val, b)
        # the padding of the tiled buffer is left as it was: zero
        words = out.data.cpu().numpy().view(np.uint32)
        logical_bits = sum(int(np.unpackbits(lk.logical_from_tiled(lk.PackedBits(out.data[b:b + 1], None, 1, N, M))
                                             .cpu().numpy().view(np.uint8)).sum()) for b in range(batch))
        assert int(np.unpackbits(words.view(np.uint8)).sum()) == logical_bits


def test_bits_output_chains_two_layers_and_empty_k(oracle):
    """Two binary layers with nothing but bits in between equal the op-by-op chain; K = 0 gives the bits of the bias."""
    rng = np.random.default_rng(99)
    N, K, H, M = 128, 784, 512, 96
    x = to_dev(rng.standard_normal((N, K)).astype(np.float16))
    w1, w2 = to_dev(rng.standard_normal((H, K)).astype(np.float16)), to_dev(rng.standard_normal((M, H)).astype(np.float16))
    sw1 = (w1.float().norm(1, 1) / w1.numel()).half()
    sa, zp = torch.full((1,), 1.25, device=DEV).half(), torch.full((1,), 0.001, device=DEV).half()
    w1p, w2p = lk.pack_sign(w1), lk.pack_sign(w2)
    # op by op: fp16 activations materialised, then centred and packed
    h = lk.bgemm_packed_forward(w1p, lk.pack_sign(x), MODE_XOR, scale=(sw1, sa, None))[0]
    want = lk.bgemm_packed_forward(w2p, lk.pack_sign(h, zero_point=zp), MODE_XOR, torch.int32)
    # fused: layer 1 writes layer 2's operand
    hb = lk.bgemm_packed_forward(w1p, lk.pack_sign(x), MODE_XOR, scale=(sw1, sa, None), bits_out=lk.zeros_packed(N, H, 1, DEV),
                                 next_zero_point=zp)
    got = lk.bgemm_packed_forward(w2p, hb, MODE_XOR, torch.int32)
    assert torch.equal(got, want)
    # K = 0: acc = 0, so the bits are those of (bias - zp)
    bias = to_dev(rng.standard_normal(70).astype(np.float32))
    e = lambda r: lk.PackedBits(torch.empty((1, 0), dtype=torch.int32, device=DEV), None, 1, r, 0)
    ob = lk.bgemm_packed_forward(e(70), e(9), MODE_XOR, bits_out=lk.zeros_packed(9, 70, 1, DEV),
                                 scale=(torch.ones(70, device=DEV), torch.ones(1, device=DEV), bias),
                                 next_zero_point=torch.full((1,), 0.25, device=DEV))
    wantb = oracle.c_pack_sign(np.tile((bias.cpu().numpy() - np.float32(0.25)).astype(np.float16), (9, 1)))
    assert (lk.logical_from_tiled(ob).cpu().numpy().view(np.uint32) == wantb).all()


@pytest.mark.parametrize("M,N,K", [(1024, 512, 1024), (520, 300, 2304), (1032, 96, 8192), (4096, 256, 6144),      # the last: four pieces a block
                                   (1028, 512, 1024), (1027, 512, 1024)])     # rows stored four elements and one element at a time
def test_scaled_fp16_matches_torchs_fp16_kernels_from_denormal_to_overflow(M, N, K):
    """The fp16 scaled kind against torch's own fp16 elementwise kernels on the int32 result (what the layers of
    tests/python/bgemm_linear.py compute after the kernel, one rounded operation at a time): per-row scales from the
    denormal range to overflow, both signs, activation scales, with and without a bias; bit for bit, NaN for NaN."""
    g = torch.Generator(device=DEV).manual_seed(M + N + K)
    rng = np.random.default_rng(M + N + K)
    w, x = rand_f16(rng, M, K), rand_f16(rng, N, K)
    wp, xp = lk.pack_sign(to_dev(w)), lk.pack_sign(to_dev(x))
    acc = lk.bgemm_packed_forward(wp, xp, MODE_XOR, torch.int32, 1)[0]
    for lo, hi in ((-24, -14), (-14, -6), (-6, 0), (0, 6), (-24, 6)):
        e = torch.randint(lo, hi + 1, (M,), generator=g, device=DEV).float()
        sign = torch.where(torch.rand(M, generator=g, device=DEV) < 0.5, -1.0, 1.0).half()
        sw = (torch.exp2(e) * (1 + torch.rand(M, generator=g, device=DEV))).half() * sign
        for sa_v in (0.7371, 3.1e-3, 61.0):
            sa = torch.tensor([sa_v], device=DEV).half()
            be = torch.randint(-20, 12, (M,), generator=g, device=DEV).float()
            for bias in (None, (torch.randn(M, generator=g, device=DEV) * torch.exp2(be)).half()):
                got = lk.bgemm_packed_forward(wp, xp, MODE_XOR, scale=(sw, sa, bias))[0]
                want = acc.half() * sw * sa
                if bias is not None:
                    want = want + bias
                same = (got.view(torch.int16) == want.view(torch.int16)) | (got.isnan() & want.isnan())
                assert bool(same.all()), (lo, hi, sa_v, bias is not None, int((~same).sum()))


def test_bits_output_drops_row_popcounts_of_the_operand_it_overwrites(oracle):
    """An operand that carried row popcounts and is then rewritten through bits_out must not feed the stale counts to
    the counted kernel (XOR's rank-one terms would be those of the old bits)."""
    rng = np.random.default_rng(5)
    N, K, H, M = 256, 512, 1024, 512
    x, w1, w2 = rand_f16(rng, N, K), rand_f16(rng, H, K), rand_f16(rng, M, H)
    w1p, w2p, xp = lk.pack_sign(to_dev(w1)), lk.pack_sign(to_dev(w2)), lk.pack_sign(to_dev(x))
    lk.row_popcounts(w2p)
    hb = lk.zeros_packed(N, H, 1, DEV)
    lk.row_popcounts(hb)                             # counts of the all-zero buffer
    sw, sa = torch.ones(H, device=DEV), torch.ones(1, device=DEV)
    lk.bgemm_packed_forward(w1p, xp, MODE_XOR, scale=(sw, sa, None), bits_out=hb)
    assert hb.counts is None
    got = lk.bgemm_packed_forward(w2p, hb, MODE_XOR, torch.int32)[0].cpu().numpy()
    acc1 = oracle.c_bgemm_packed(1, oracle.c_pack_sign(w1), oracle.c_pack_sign(x), K)
    h = oracle.np_center_to_f16(oracle.np_scale_epilogue(acc1, np.ones(H, np.float32), np.float32(1)), np.float32(0))
    want = oracle.c_bgemm_packed(1, oracle.c_pack_sign(w2), oracle.c_pack_sign(h), H)
    assert (got == want).all()
    lk.row_popcounts(hb)                             # counted again: the counted kernel agrees
    assert (lk.bgemm_packed_forward(w2p, hb, MODE_XOR, torch.int32)[0].cpu().numpy() == want).all()
