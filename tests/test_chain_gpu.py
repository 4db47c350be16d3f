"""The chain of dependent decode-shaped layers in one launch (bgemm_chain_forward) against the oracle run layer by
layer: acc = the mode's integer product (ptx_mma.cuh:196-250; ternary: bgemm_linear.py:222-241), y = half(acc) * sw * sa
(+ bias) step by step (bgemm_linear.py:482-484), next operand = bits of half(y - zp) (:479-482).  Bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lowbit_kernel as lk
from _lib import MODE_XOR, MODE_BWTA, MODE_ATTN

DEV = "cuda:0"


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def make_chain(rng, dims, dtype, with_bias=True, with_zp=True):
    """Random layers dims[0] -> dims[1] -> ...; scales sized so that the scaled outputs straddle the zero points."""
    layers = []
    for l in range(len(dims) - 1):
        K, M = dims[l], dims[l + 1]
        w = rng.standard_normal((M, K)).astype(np.float16)
        sw = (rng.uniform(0.5, 2.0, M) / np.sqrt(K)).astype(dtype) * rng.choice([-1, 1], M).astype(dtype)
        sa = np.asarray(rng.uniform(0.5, 1.5), dtype=dtype)
        bias = (0.3 * rng.standard_normal(M)).astype(dtype) if with_bias and l % 2 == 0 else None
        zp = np.asarray(0.11 * rng.standard_normal(), dtype=dtype) if with_zp and l % 3 != 2 else None
        layers.append((w, sw, sa, bias, zp))
    return layers


def oracle_chain(oracle, mode, layers, x, last_kind):
    """x: fp16 [N][K0] whose signs / ternary values are the first operand.  Returns the last layer's output."""
    h = x
    for l, (w, sw, sa, bias, zp) in enumerate(layers):
        K = w.shape[1]
        wp = oracle.c_pack_sign(w)
        if mode == MODE_BWTA:
            nz, sg = oracle.c_pack_ternary(h)
            acc = oracle.c_bwta_packed(wp, nz, sg, K)
        else:
            acc = oracle.c_bgemm_packed(mode, wp, oracle.c_pack_sign(h), K)
        if l + 1 == len(layers):
            if last_kind == "i32":
                return acc
            if last_kind == "f16":
                with np.errstate(over="ignore"):
                    return acc.astype(np.float32).astype(np.float16)
            return oracle.np_scale_epilogue(acc, sw, sa, bias)
        y = oracle.np_scale_epilogue(acc, sw, sa, bias)
        h = oracle.np_center_to_f16(y, sw.dtype.type(0) if zp is None else zp)


def device_chain(mode, layers, out_dtype, flags):
    dl = []
    for w, sw, sa, bias, zp in layers:
        dl.append((lk.pack_sign(to_dev(w)), to_dev(sw), to_dev(sa.reshape(1)), None if bias is None else to_dev(bias),
                   None if zp is None else to_dev(zp.reshape(1))))
    return lk.DecodeChain(dl, mode, out_dtype, flags)


def operand(mode, x):
    return lk.pack_ternary(to_dev(x)) if mode == MODE_BWTA else lk.pack_sign(to_dev(x))


def same(got, want):
    got = got.cpu().numpy()
    if want.dtype == np.int32:
        return got.dtype == np.int32 and (got == want).all()
    v = np.uint16 if want.dtype == np.float16 else np.uint32
    return got.dtype == want.dtype and ((got.view(v) == want.view(v)) | (np.isnan(got) & np.isnan(want))).all()


def ternary_input(rng, N, K):
    x = rng.standard_normal((N, K)).astype(np.float16)
    x[rng.random((N, K)) < 0.5] = 0
    x[:, ::13] = np.float16(-0.0)
    return x


# flags: bits 8.. = number of blocks (so that small layers put two and three row tiles on a block), low bits 1 / 2 = one /
# two exchange levels
@pytest.mark.parametrize("flags", [(8 << 8) | 1, (8 << 8) | 2, (16 << 8) | 2, (5 << 8) | 1])
@pytest.mark.parametrize("mode,N", [(MODE_XOR, 1), (MODE_XOR, 5), (MODE_XOR, 32), (MODE_BWTA, 1), (MODE_BWTA, 3), (MODE_BWTA, 16), (MODE_ATTN, 7)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_small_chain_every_tile_count_and_exchange(oracle, mode, N, dtype, flags):
    """Ragged layers (M not a multiple of 32, K not of 256), one to three row tiles a block, one and two exchange
    levels, every mode family, with and without bias and zero point, all three kinds of last output."""
    G = flags >> 8
    rng = np.random.default_rng(N * 100 + mode * 7 + (flags & 0xfff))
    dims = [300, 32 * G * 2, 257, 32 * min(G, 8) * 3, 96, 40] if G >= 8 else [300, 320, 257, 480, 40]
    layers = make_chain(rng, dims, dtype)
    x = ternary_input(rng, N, dims[0])
    for out_dtype, kind in ((torch.int32, "i32"), (torch.half, "f16"), (None, "scaled")):
        want = oracle_chain(oracle, mode, layers, x, kind)
        chain = device_chain(mode, layers, out_dtype, flags)
        for rep in range(3):          # the tags move on from call to call
            got = chain(operand(mode, x))
            chain.check(N)
            assert same(got, want), (kind, rep)


@pytest.mark.parametrize("mode,N", [(MODE_BWTA, 1), (MODE_BWTA, 4), (MODE_BWTA, 16), (MODE_XOR, 2), (MODE_XOR, 32)])
@pytest.mark.parametrize("flags", [0, 1, 2])
def test_llama_mlp_chain_on_every_compute_unit(oracle, mode, N, flags):
    """BASELINE configuration 4's matrix as the layers of a model see it: up W[11008,4096] -> down W[4096,11008] ->
    up -> down, one block per compute unit, fp16 parameters, int32 out."""
    rng = np.random.default_rng(N + mode)
    layers = make_chain(rng, [4096, 11008, 4096, 11008, 4096], np.float16)
    x = ternary_input(rng, N, 4096)
    want = oracle_chain(oracle, mode, layers, x, "i32")
    chain = device_chain(mode, layers, torch.int32, flags)
    for rep in range(2):
        got = chain(operand(mode, x))
        chain.check(N)
        assert same(got, want), rep


def test_chain_equals_layer_by_layer_launches(oracle):
    """The same stack through bgemm_packed_forward with bits between the layers (one launch a layer)."""
    rng = np.random.default_rng(77)
    dims, N = [1024, 2048, 1024, 512], 8
    layers = make_chain(rng, dims, np.float16)
    x = rng.standard_normal((N, dims[0])).astype(np.float16)
    chain = device_chain(MODE_XOR, layers, None, 0)
    got = chain(lk.pack_sign(to_dev(x)))
    chain.check(N)
    hp = lk.pack_sign(to_dev(x))
    for l, (w, sw, sa, bias, zp) in enumerate(chain.layers):
        if l + 1 < len(layers):
            hp = lk.bgemm_packed_forward(w, hp, MODE_XOR, scale=(sw, sa, bias), bits_out=lk.zeros_packed(N, w.rows, 1, DEV), next_zero_point=zp)
        else:
            want = lk.bgemm_packed_forward(w, hp, MODE_XOR, scale=(sw, sa, bias))[0]
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_chain_rejects_what_it_cannot_run():
    rng = np.random.default_rng(3)
    with pytest.raises(ValueError):
        device_chain(MODE_XOR, make_chain(rng, [256, 512, 256], np.float16), None, 0)(lk.pack_sign(to_dev(rng.standard_normal((40, 256)).astype(np.float16))))
    bad = make_chain(rng, [256, 512], np.float16) + make_chain(rng, [480, 64], np.float16)        # 512 written, 480 read
    with pytest.raises(ValueError):
        device_chain(MODE_XOR, bad, None, 0)(lk.pack_sign(to_dev(rng.standard_normal((4, 256)).astype(np.float16))))
    with pytest.raises(ValueError):          # K beyond one block's LDS operand
        device_chain(MODE_XOR, make_chain(rng, [32768, 64], np.float16), None, 0)(lk.pack_sign(to_dev(rng.standard_normal((4, 32768)).astype(np.float16))))


def test_a_wait_that_runs_out_of_budget_ends_the_launch_and_is_reported(oracle):
    """The time-out path, forced from the host: with flags & 8 the first block publishes nothing and the budget is a
    millisecond, so every block gives up waiting for it and leaves (no wave spins on); the status call reports it once,
    and the same workspace then runs the chain correctly."""
    import _lib
    rng = np.random.default_rng(11)
    layers = make_chain(rng, [512, 2048, 512], np.float16)
    x = rng.standard_normal((4, 512)).astype(np.float16)
    want = oracle_chain(oracle, MODE_XOR, layers, x, "i32")
    chain = device_chain(MODE_XOR, layers, torch.int32, 0)
    xp = lk.pack_sign(to_dev(x))
    assert same(chain(xp), want)
    chain.check(4)
    chain.flags = 8
    chain(xp)
    with pytest.raises(_lib.BgemmError, match="budget"):
        chain.check(4)
    chain.flags = 0
    chain.check(4)                      # reported once
    for rep in range(2):
        assert same(chain(xp), want)
        chain.check(4)
