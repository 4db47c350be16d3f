"""bgemm_f16_forward_static (the drop-in call with the library's own scratch array instead of a workspace):
through the C ABI, against bgemm_f16_forward on the same inputs, bit for bit, on two calls in a row, the
second smaller than the first (the array keeps the first call's contents)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import _lib

DEV = "cuda:0"


def both(L, x, w, splitK, instr):
    N, K = x.shape
    M = w.shape[0]
    stream = torch.cuda.current_stream().cuda_stream
    want = torch.full((N, M), float("nan"), dtype=torch.half, device=DEV)
    got = torch.full((N, M), float("nan"), dtype=torch.half, device=DEV)
    ws = torch.empty(max(L.bgemm_f16_workspace_bytes(M, N, K, splitK), 1), dtype=torch.uint8, device=DEV)
    _lib.check(L.bgemm_f16_forward(w.data_ptr(), x.data_ptr(), want.data_ptr(), M, N, K, ws.data_ptr(), ws.numel(),
                                   splitK, instr, stream))
    _lib.check(L.bgemm_f16_forward_static(w.data_ptr(), x.data_ptr(), got.data_ptr(), M, N, K, splitK, instr, stream))
    torch.cuda.synchronize()
    return got, want


def test_static_scratch_call_equals_the_workspace_call_twice_in_a_row(oracle):
    L = _lib.lib()
    g = torch.Generator(device=DEV).manual_seed(7)
    # ragged everything, zeros of both signs; the second call is smaller in every dimension, so its tiles
    # land on what the first call left in the array
    for (M, N, K), instr, splitK in (((1000, 300, 3000), 1, 2), ((130, 70, 1000), 2, 1), ((33, 5, 100), 0, 3)):
        x = torch.randn((N, K), generator=g, device=DEV).half()
        w = torch.randn((M, K), generator=g, device=DEV).half()
        x[:, ::9] = 0.0
        x[::2, ::18] = -0.0
        got, want = both(L, x, w, splitK, instr)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K)
        ref, _ = oracle.c_bgemm_f16(x.cpu().numpy(), w.cpu().numpy(), splitK, instr)
        assert (got.cpu().numpy().view(np.uint16) == ref.view(np.uint16)).all(), (M, N, K)


def test_static_scratch_call_states_its_limit_and_takes_empty_problems():
    L = _lib.lib()
    # 16384 x 16384 bits on either side: 64 MiB of packed operands, beyond the array
    assert L.bgemm_f16_workspace_bytes(16384, 16384, 16384, 1) > _lib.STATIC_SCRATCH_BYTES
    rc = L.bgemm_f16_forward_static(0x1000, 0x2000, 0x3000, 16384, 16384, 16384, 1, 1, None)
    assert rc == _lib.EWORKSPACE and b"scratch" in L.bgemm_last_error()
    assert L.bgemm_f16_forward_static(None, None, None, 0, 5, 128, 1, 1, None) == 0
    assert L.bgemm_f16_forward_static(0x1000, 0x2000, 0x3000, 32, 32, 128, 1, 7, None) == _lib.EINVAL
    # K = 0: the empty sum, no scratch touched
    out = torch.full((3, 8), 5.0, dtype=torch.half, device=DEV)
    _lib.check(L.bgemm_f16_forward_static(None, None, out.data_ptr(), 8, 3, 0, 1, 1, torch.cuda.current_stream().cuda_stream))
    assert torch.equal(out, torch.zeros_like(out))
    # the largest shape the array takes: 8192 x 8192 against 8192 x 8192
    assert L.bgemm_f16_workspace_bytes(8192, 8192, 8192, 1) <= _lib.STATIC_SCRATCH_BYTES
