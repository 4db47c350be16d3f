"""The layer mirror on the GPU: same numbers as the reference CPU path (torch matmul on +-1
tensors) fed identical operands, compared bit for bit (tolerance 0)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import bgemm_linear as bl
import lowbit_kernel as lk

DEV = "cuda:0"


def test_bgemm_linear_function_vs_sign_matmul():
    torch.manual_seed(0)
    x, w = torch.randn(64, 768, device=DEV), torch.randn(96, 768, device=DEV)
    out = bl.bgemm_linear.apply(x, w)
    want = (x.half().sign().float() @ w.half().sign().float().T)
    assert out.dtype == torch.half and torch.equal(out.float(), want.half().float())
    out_and = bl.bgemm_linear.apply(x, w, 'and')
    assert torch.equal(out_and.float(), ((x < 0).float() @ (w < 0).float().T).half().float())


def test_bgemm_matmul_and_attn_matmul():
    torch.manual_seed(1)
    q, k = torch.randn(32, 768, device=DEV), torch.randn(32, 768, device=DEV)
    attn = bl.bgemm_matmul.apply(q, k.transpose(-1, -2))
    assert torch.equal(attn.float(), torch.matmul(q.sign(), k.sign().T).half().float())
    # a genuinely contiguous [K, M] right operand also works (the reference mis-reads it); it is packed as it lies
    kt = k.T.contiguous()
    assert torch.equal(bl.bgemm_matmul.apply(q, kt), attn)
    assert torch.equal(bl.bgemm_matmul.apply(q.reshape(4, 8, 768), kt), attn.reshape(4, 8, 32))     # leading dimensions
    assert torch.equal(bl.bgemm_matmul.apply(q, kt, 'and').float(), ((q < 0).float() @ (k < 0).float().T).half().float())
    a = torch.randn(128, 256, device=DEV)
    v = torch.randn(256, 64, device=DEV)
    out = bl.bgemm_attn_matmul.apply(a, v)
    want = (a >= 0).float() @ v.sign()
    assert tuple(out.shape) == (128, 64) and torch.equal(out.float(), want.half().float())


def test_batched_attention_pair_bert_shape():
    """Q K^T then A V over [batch, heads, seq, head_dim] in one launch each (the reference is 2-D only)."""
    torch.manual_seed(5)
    B, H, S, D = 2, 12, 512, 64
    q, k, v = (torch.randn(B, H, S, D, device=DEV) for _ in range(3))
    scores = bl.bgemm_matmul.apply(q, k.transpose(-1, -2))
    pm = lambda t: torch.where(torch.signbit(t.half()), -1.0, 1.0)
    want = torch.matmul(pm(q), pm(k).transpose(-1, -2))
    assert scores.dtype == torch.half and tuple(scores.shape) == (B, H, S, S)
    assert torch.equal(scores.float(), want.half().float())
    attn = torch.randn(B, H, S, S, device=DEV)                    # zero-centred: "1" where the sign bit is clear
    ctx = bl.bgemm_attn_matmul.apply(attn, v)
    # operands are read off the sign bit, as the kernel does: among millions of halves a few round to +-0.0,
    # which torch.sign would map to 0
    want = torch.matmul((~torch.signbit(attn.half())).float(), torch.where(torch.signbit(v.half()), -1.0, 1.0))
    assert tuple(ctx.shape) == (B, H, S, D) and torch.equal(ctx.float(), want.half().float())
    # each slice equals the 2-D call
    assert torch.equal(ctx[1, 3], bl.bgemm_attn_matmul.apply(attn[1, 3], v[1, 3]))
    # gradients flow with batched shapes
    qg = q.clone().requires_grad_(True)
    kt = k.transpose(-1, -2).clone().requires_grad_(True)
    bl.bgemm_matmul.apply(qg, kt).float().sum().backward()
    assert qg.grad.shape == q.shape and kt.grad.shape == kt.shape
    g = torch.ones(S, S, device=DEV)
    assert torch.allclose(qg.grad[0, 0].float(), g @ k[0, 0].half().sign().float(), atol=0)   # backward uses torch.sign


@pytest.mark.parametrize("dtype", [torch.float32, torch.half])
def test_attention_pair_reads_head_split_views_where_they_lie(dtype):
    """The [B, H, S, d] operands of BERT are `permute(0, 2, 1, 3)` views of [B, S, H*d] projections
    (bert.py:216-234).  The pair takes the views as they are, fp32 or fp16, with or without gradients, and gives what
    it gives for contiguous fp16 copies; ragged S and d included."""
    torch.manual_seed(9)
    for (B, H, S, D) in ((2, 12, 128, 64), (2, 3, 50, 40)):
        split = lambda t: t.view(B, S, H, D).permute(0, 2, 1, 3)
        q, k, v = (split(torch.randn(B, S, H * D, device=DEV, dtype=dtype)) for _ in range(3))
        attn = torch.randn(B, H, S, S, device=DEV, dtype=dtype)
        dense = lambda t: t.to(torch.half).contiguous()
        with torch.no_grad():
            scores = bl.bgemm_matmul.apply(q, k.transpose(-1, -2))
            ctx = bl.bgemm_attn_matmul.apply(attn, v)
            assert torch.equal(scores, bl.bgemm_matmul.apply(dense(q), dense(k).transpose(-1, -2)))
            assert torch.equal(ctx, bl.bgemm_attn_matmul.apply(dense(attn), dense(v)))
        pm = lambda t: torch.where(torch.signbit(t.half()), -1.0, 1.0)
        assert torch.equal(scores.float(), torch.matmul(pm(q), pm(k).transpose(-1, -2)).half().float())
        assert torch.equal(ctx.float(), torch.matmul((~torch.signbit(attn.half())).float(), pm(v)).half().float())
        # with gradients the operands are saved as fp16 and the outputs are the same
        qg, vg = q.detach().clone().requires_grad_(True), v.detach().clone().requires_grad_(True)
        assert torch.equal(bl.bgemm_matmul.apply(qg, k.transpose(-1, -2)), scores)
        assert torch.equal(bl.bgemm_attn_matmul.apply(attn, vg), ctx)


def test_bgemm_linear_backward_shapes_and_values():
    torch.manual_seed(2)
    x = torch.randn(32, 128, device=DEV, requires_grad=True)
    w = torch.randn(16, 128, device=DEV, requires_grad=True)
    bl.bgemm_linear_bireal.apply(x, w).float().sum().backward()
    g = torch.ones(32, 16, device=DEV)
    assert torch.allclose(w.grad, (g.T @ x.detach().half().sign().float()), atol=0)
    dx = 2 - 2 * x.detach().half().float().abs().clamp(max=1)
    # the backward runs in fp16 like the reference's (saved tensors are halves): fp16 tolerance
    assert torch.allclose(x.grad, (g @ w.detach().half().sign().float()) * dx, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("cls", [bl.BGEMMLinear, bl.BGEMMLinear_bireal])
def test_bgemm_linear_module_vs_bnn(oracle, cls):
    torch.manual_seed(3)
    x = torch.randn(128, 784, device=DEV)
    lin = cls(784, 4096, bias=True).to(DEV)
    y = lin(x)
    sw, sa, zpw, zpa = oracle.cpu_path_layer_scales(x, lin.weight)
    # reference CPU path (torch matmul on +-1 tensors).  Operands are de-binarised by the sign bit, as
    # the kernel reads them: the fp16 cast flushes a few tiny negatives to -0.0, which BinActive would
    # map to +1 (bgemm_linear.py:606-607) and the reference kernel to -1 (ptx_mma.cuh:375).
    xh, wh = (x - zpa).half(), (lin.weight - zpw).half()
    pm = lambda t: torch.where(torch.signbit(t), -1.0, 1.0).cpu()
    acc = oracle.cpu_path_linear(pm(xh), pm(wh)).to(DEV)
    bin_active = oracle.cpu_path_bin_active
    differs = (bin_active(wh.float()).cpu() != pm(wh)) | False
    assert bool((differs == ((wh == 0) & torch.signbit(wh)).cpu()).all())
    want = acc.half() * sw * sa + lin.bias.view(1, -1)
    assert torch.equal(y, want)
    # ragged batch (the reference asserts batch % 32 == 0)
    assert torch.equal(lin(x[:5]), want[:5])


@pytest.mark.parametrize("dtype", [torch.float32, torch.half])
@pytest.mark.parametrize("bias", [True, False])
def test_fused_inference_forward_equals_composed_ops(dtype, bias):
    """Under no_grad the module centres+packs x in one pass, reuses the packed weight and scales in
    the GEMM's store; the result must equal the op-by-op forward (bgemm_linear.py:479-484) bit for bit."""
    torch.manual_seed(7)
    lin = bl.BGEMMLinear(784, 300, bias=bias).to(DEV).to(dtype)
    x = torch.randn(3, 50, 784, device=DEV).to(dtype)
    y_ops = lin(x)                                   # grad mode: separate torch kernels around the GEMM
    assert y_ops.requires_grad
    with torch.no_grad():
        assert lin._fusable(x)
        y_fused = lin(x)
        lin.fuse_inference = False
        y_plain = lin(x)
        lin.fuse_inference = True
    assert y_fused.dtype == y_ops.dtype == dtype and y_fused.shape == y_ops.shape
    assert torch.equal(y_fused, y_ops.detach()) and torch.equal(y_fused, y_plain)
    # the packed weight is cached until the weight changes
    wp = lin._packed_weight()
    assert lin._packed_weight() is wp
    with torch.no_grad():
        lin.weight.neg_()
        assert lin._packed_weight() is not wp
        lin.fuse_inference = False
        want = lin(x)
        lin.fuse_inference = True
        assert torch.equal(lin(x), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.half])
def test_chain_keeps_only_bits_between_layers(dtype):
    """784 -> 4096 -> 4096 -> 10 with the hidden activations never stored: same output as layer by layer."""
    torch.manual_seed(11)
    chain = bl.BGEMMChain(bl.BGEMMLinear(784, 4096, bias=True), bl.BGEMMLinear(4096, 4096, bias=False),
                          bl.BGEMMLinear(4096, 10, bias=True)).to(DEV).to(dtype)
    x = torch.randn(128, 784, device=DEV).to(dtype)
    with torch.no_grad():
        first = chain(x)                       # initialises the scales layer by layer
        assert chain._fusable(x)
        fused = chain(x)
        h = x
        for layer in chain:
            h = layer(h)
    assert fused.dtype == dtype and tuple(fused.shape) == (128, 10)
    assert torch.equal(fused, h) and torch.equal(fused, first)
    x2 = torch.randn(3, 7, 784, device=DEV).to(dtype)      # another batch shape, leading dimensions
    with torch.no_grad():
        h = x2
        for layer in chain:
            h = layer(h)
        assert torch.equal(chain(x2), h)
    assert chain(x).requires_grad                          # with gradients: the ordinary path


@pytest.mark.parametrize("dtype", [torch.float32, torch.half])
def test_decode_rows_take_one_launch_and_follow_parameter_updates(dtype):
    """Inputs of one to four rows go through the kernel that packs its own activations; the cached parameter
    views must follow in-place updates, replaced parameters and dtype changes."""
    torch.manual_seed(21)
    lin = bl.BGEMMLinear(1000, 300, bias=True).to(DEV).to(dtype)
    big = torch.randn(64, 1000, device=DEV).to(dtype)
    with torch.no_grad():
        lin(big)                                             # initialises the scales
        lin.fuse_inference = False
        want = lin(big)
        lin.fuse_inference = True
        for n in (1, 2, 4, 5):
            assert torch.equal(lin(big[:n]), want[:n]), n
        assert torch.equal(lin(big[:3].reshape(3, 1, 1000)), want[:3].reshape(3, 1, 300))
        lin.sw.mul_(2.0); lin.bias.add_(1.0)                 # in place
        lin.fuse_inference = False
        want = lin(big[:2])
        lin.fuse_inference = True
        assert torch.equal(lin(big[:2]), want)
        lin.sa = torch.nn.Parameter(lin.sa.detach() * 3)     # replaced
        lin.fuse_inference = False
        want = lin(big[:2])
        lin.fuse_inference = True
        assert torch.equal(lin(big[:2]), want)
    other = torch.half if dtype == torch.float32 else torch.float32
    lin = lin.to(other)
    lin.zpa = lin.zpa.to(other)
    with torch.no_grad():
        x = big[:1].to(other)
        lin.fuse_inference = False
        want = lin(x)
        lin.fuse_inference = True
        assert lin(x).dtype == other and torch.equal(lin(x), want)


def test_elastic_module_matches_cpu_twin():
    torch.manual_seed(4)
    x = torch.randn(64, 256, device=DEV)
    a = bl.BGEMMLinear_elastic_signed(256, 128).to(DEV)
    b = bl.NNLinear_elastic_signed(256, 128).to(DEV)
    b.load_state_dict(a.state_dict())
    ya, yb = a(x), b(x)
    # the twin ternarises exact zeros to 0 while the kernel reads the sign bit; none occur here
    assert torch.equal(ya.float(), yb.float())
    ya.float().sum().backward()
    assert a.weight.grad is not None and a.sa.grad is not None and a.sw.grad is not None


@pytest.mark.filterwarnings("ignore:Synchronization debug mode")
@pytest.mark.parametrize("dtype", [torch.float32, torch.half])
def test_elastic_inference_runs_on_packed_operands_without_host_reads(dtype):
    """Under no_grad the elastic layer centres and packs x in one pass and packs the weight once; the outputs are
    those of the op-by-op forward, also for ragged shapes, after updates of the weight and the scales, and for a
    negative sa (which the packed path leaves to the op-by-op one)."""
    torch.manual_seed(6)
    for (n, k, m) in ((64, 256, 128), (37, 300, 70), (1, 784, 10)):
        lin = bl.BGEMMLinear_elastic_signed(k, m).to(DEV).to(dtype)
        x = torch.randn(n, k, device=DEV, dtype=dtype) + 0.25
        want = lin(x).detach()                               # records gradients: the op-by-op forward
        with torch.no_grad():
            got = lin(x)
            assert got.dtype == want.dtype and torch.equal(got, want)
            assert torch.equal(lin(x.reshape(1, n, k)), want.reshape(1, n, m))
            # steady state: no host read-back in the forward
            torch.cuda.set_sync_debug_mode("error")
            try:
                again = lin(x)
            finally:
                torch.cuda.set_sync_debug_mode("default")
            assert torch.equal(again, want)
            lin.weight.mul_(-0.5).add_(0.01)
            lin.sw.mul_(1.5)
            lin.sa.mul_(0.75)
            lin.fuse_inference = False
            want2 = lin(x)
            lin.fuse_inference = True
            assert not torch.equal(want2, want) and torch.equal(lin(x), want2)
            lin.sa.neg_()
            lin.fuse_inference = False
            want3 = lin(x)
            lin.fuse_inference = True
            assert torch.equal(lin(x), want3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.half])
def test_graphed_inference_replays_equal_eager(dtype):
    """A chain captured into a HIP graph gives, replay after replay and with eager work in between, what the eager
    forward gives for the same input; scales changed in place are seen; another shape is refused."""
    torch.manual_seed(12)
    chain = bl.BGEMMChain(bl.BGEMMLinear(300, 256, bias=True), bl.BGEMMLinear(256, 512), bl.BGEMMLinear(512, 10, bias=True)).to(DEV).to(dtype)
    xs = [torch.randn(64, 300, device=DEV, dtype=dtype) for _ in range(4)]
    with torch.no_grad():
        chain(xs[0])                                  # first call initialises the layers
        fast = bl.GraphedInference(chain, xs[0])
        for i in (1, 2, 0, 3, 1):
            want = chain(xs[i])                       # eager launches between the replays
            got = fast(xs[i])
            assert got.dtype == want.dtype and torch.equal(got, want), i
        chain[1].sw.mul_(0.5)
        chain[2].bias.add_(1.0)
        assert torch.equal(fast(xs[2]), chain(xs[2]))
        with pytest.raises(ValueError):
            fast(xs[0][:32])
    # a decode step (one row: the kernel that packs its own activations) captures too
    lin = bl.BGEMMLinear(4096, 1000, bias=True).to(DEV).to(dtype)
    with torch.no_grad():
        lin(torch.randn(8, 4096, device=DEV, dtype=dtype))
        x1 = torch.randn(1, 4096, device=DEV, dtype=dtype)
        step = bl.GraphedInference(lin, x1)
        for _ in range(3):
            x1 = torch.randn(1, 4096, device=DEV, dtype=dtype)
            assert torch.equal(step(x1), lin(x1))
    # a single layer and the attention block capture the same way
    import attention_demo
    block = attention_demo.BinarySelfAttention(128, 4).to(DEV)
    x = torch.randn(2, 64, 128, device=DEV)
    with torch.no_grad():
        block(x)
        fast = bl.GraphedInference(lambda t: block(t)[0], x)
        for _ in range(3):
            x = torch.randn(2, 64, 128, device=DEV)
            assert torch.equal(fast(x), block(x)[0])


def test_config2_mlp_forward_bitwise(oracle):
    """Benchmark configuration 2: 784 -> 4096 -> 4096 -> 10, batch 128, fp16 outputs vs the CPU chain."""
    g = torch.Generator().manual_seed(1002)
    dims = [784, 4096, 4096, 10]
    x = torch.randn(128, 784, generator=g).half()
    Ws = [torch.randn(dims[i + 1], dims[i], generator=g).half() for i in range(3)]
    h_gpu, h_cpu = x.to(DEV), x.clone()
    for W in Ws:
        sw = (W.float().norm(1, 1) / W.numel()).half()
        sa = (2 * h_cpu.float().abs().mean()).half()
        # GPU: binary kernel then fp16 scaling, left to right as the reference layer does
        acc_gpu = lk.bgemm_linear_forward_cuda(h_gpu, W.to(DEV), 1, 1)
        h_gpu = acc_gpu * sw.to(DEV) * sa.to(DEV)
        # CPU reference path: torch matmul on +-1 tensors (sign-bit rule), fp16 rounding of the exact sum
        sx = torch.where(torch.signbit(h_cpu), -1.0, 1.0)
        swt = torch.where(torch.signbit(W), -1.0, 1.0)
        acc_cpu = oracle.cpu_path_linear(sx, swt).half()
        h_cpu = acc_cpu * sw * sa
        assert torch.equal(acc_gpu.cpu(), acc_cpu)
        assert torch.equal(h_gpu.cpu(), h_cpu)
    assert tuple(h_gpu.shape) == (128, 10)


@pytest.mark.parametrize("cls", [bl.BGEMMLinear, bl.BGEMMLinear_elastic_signed])
def test_packed_weight_cache_follows_the_parameter_and_can_be_dropped(cls):
    """Updates through the parameter are seen (version counter); a write through ``.data`` is not, and train() /
    eval(), load_state_dict and invalidate_packed_weight() drop the cached bits."""
    torch.manual_seed(11)
    lin = cls(256, 64).to(DEV)
    x = torch.randn(8, 256, device=DEV)
    lin(x)                                           # initialises the scales
    with torch.no_grad():
        y0 = lin(x).clone()
        lin.weight.neg_()                            # through the parameter: the cache follows
        y1 = lin(x).clone()
        lin.weight.data.neg_()                       # behind the version counter: stale bits until told
        stale = lin(x).clone()
        lin.invalidate_packed_weight()
        y2 = lin(x).clone()
    assert not torch.equal(y0, y1) and torch.equal(stale, y1) and torch.equal(y2, y0)
    with torch.no_grad():
        lin.weight.data.neg_()
        lin.eval()                                   # a change of mode drops the cache as well
        assert torch.equal(lin(x), y1)
        sd = {k: v.clone() for k, v in lin.state_dict().items()}
        sd["weight"] = -sd["weight"]
        lin.weight.data.mul_(3.0)                    # (same signs: the bits would not change)
        lin.load_state_dict(sd)
        assert torch.equal(lin(x), y0)


def test_packed_weight_cache_follows_the_weights_zero_point():
    """The cached bits are those of (weight - zpw) (bgemm_linear.py:482): an in-place update of zpw alone packs again."""
    torch.manual_seed(12)
    lin = bl.BGEMMLinear(256, 64).to(DEV)
    x = torch.randn(8, 256, device=DEV)
    lin(x)
    with torch.no_grad():
        y0 = lin(x).clone()
        lin.zpw.add_(0.5)                            # moves about two fifths of the signs
        y1 = lin(x).clone()
        lin.fuse_inference = False
        want = lin(x)
    assert not torch.equal(y0, y1) and torch.equal(y1, want)
