"""Binary Linear / matmul layers over the MI355X BGEMM library.

Host-side mirror of the reference's layer file (tests/python/bgemm_linear.py): the same
class and function names, argument meaning and forward arithmetic, calling
``lowbit_kernel.bgemm_linear_forward_cuda`` exactly where the reference does.  Supersets:
any batch size (the reference asserts ``x.shape[0] % 32 == 0``, bgemm_linear.py:475),
inputs with leading batch dimensions, non-contiguous operands, and, when no gradient is being
recorded, a fused forward for BGEMMLinear / BGEMMLinear_bireal: the centred weight is bit-packed
once and cached, ``x - zpa`` is centred and packed in one pass, and ``* sw * sa (+ bias)`` is
applied in the GEMM's store, rounded step by step as the separate torch kernels would.
"""
import math

import torch
import torch.nn as nn

import lowbit_kernel

__all__ = ['BNNLinear', 'BGEMMLinear', 'BGEMMChain', 'BGEMMLinear_elastic_signed', 'bgemm_matmul', 'bgemm_attn_matmul',
           'BGEMMLinear_bireal', 'NNLinear_elastic_signed', 'bgemm_linear', 'bgemm_linear_bireal',
           'bgemm_linear_elastic_signed', 'nn_linear_elastic_signed', 'BinActive', 'ternary']


def _instr(instruction):
    return lowbit_kernel.AND_POP if instruction == 'and' else lowbit_kernel.XOR_POP


def _kernel_2d(x, w, instr):
    """fp16 [..., K] x fp16 [M, K] -> fp16 [..., M] through the drop-in entry point."""
    lead = x.shape[:-1]
    out = lowbit_kernel.bgemm_linear_forward_cuda(x.reshape(-1, x.shape[-1]), w, 1, instr)
    return out.reshape(*lead, w.shape[0])


def _linear_grads(grad_out, x_sign, w_sign):
    """Straight-through gradients of out = x_sign @ w_sign.T (bgemm_linear.py:149-165)."""
    g = grad_out.to(x_sign.dtype)
    grad_x = g @ w_sign
    grad_w = g.reshape(-1, g.shape[-1]).T @ x_sign.reshape(-1, x_sign.shape[-1])
    return grad_x, grad_w


def _matrices(t):
    """Up to two leading dimensions are handed to the pack as they are (strides and all); more are folded."""
    return t if t.dim() <= 4 else t.reshape(-1, *t.shape[-2:])


def _pack_right(mat):
    """The right-hand operand of ``a @ mat`` (``mat`` is [..., K, M]) as a packed operand of M rows.  A transposed
    view of row-major [..., M, K] matrices (``k.transpose(-1, -2)``) is packed from those rows; anything else is
    packed as it lies by the transposing pack.  No copy either way (bgemm_linear.py:25, :60 copy), also for
    the strided [B, H, S, d] views of attention."""
    rows = mat.transpose(-1, -2)
    if rows.stride(-1) == 1 and rows.stride(-2) >= rows.shape[-1]:
        return lowbit_kernel.pack_sign(_matrices(rows))
    return lowbit_kernel.pack_sign_transposed(_matrices(mat))


def _batched_packed(x_rows, right, mode):
    """x_rows [..., N, K] @ right [..., K, M] with equal leading dimensions -> fp16 [..., N, M]: one launch over
    all leading dimensions on the batched packed entry point (no per-matrix Python loop)."""
    lead = x_rows.shape[:-2]
    if right.shape[:-2] != lead:
        raise ValueError("leading dimensions differ: %s vs %s" % (tuple(x_rows.shape), tuple(right.shape)))
    xp = lowbit_kernel.pack_sign(_matrices(x_rows))
    out = lowbit_kernel.bgemm_packed_forward(_pack_right(right), xp, mode, torch.half)
    return out.reshape(*lead, x_rows.shape[-2], right.shape[-1])


class bgemm_matmul(torch.autograd.Function):
    """matA [.., N, K] @ matB [K, M] with both operands binarised by sign (bgemm_linear.py:9-42).
    A matB with leading dimensions ([B, H, K, M], as K^T in attention) is a batched matmul."""

    @staticmethod
    def forward(ctx, matA, matB, instruction='xor'):
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            matA, matB = matA.to(torch.half), matB.to(torch.half)
            ctx.save_for_backward(matA, matB)
        # otherwise the pack reads fp32 operands itself: rounding to fp16 keeps the sign bit
        mode = lowbit_kernel.MODE_AND if instruction == 'and' else lowbit_kernel.MODE_XOR
        if matB.dim() > 2:
            return _batched_packed(matA, matB, mode)
        lead = matA.shape[:-1]
        out = lowbit_kernel.bgemm_packed_forward(_pack_right(matB), lowbit_kernel.pack_sign(matA.reshape(-1, matA.shape[-1])),
                                                 mode, torch.half, splitK=8)[0]
        return out.reshape(*lead, matB.shape[-1])

    @staticmethod
    def backward(ctx, grad_output):
        matA, matB = ctx.saved_tensors
        if matB.dim() > 2:
            g = grad_output.to(matA.dtype)
            return g @ matB.sign().transpose(-1, -2), matA.sign().transpose(-1, -2) @ g, None
        grad_a, grad_bt = _linear_grads(grad_output, matA.sign(), matB.sign().transpose(-1, -2))
        return grad_a, grad_bt.transpose(-1, -2), None


class bgemm_attn_matmul(torch.autograd.Function):
    """attn [S_q, S_k] ({0,1}: 1 where the sign bit is clear) @ value [S_k, d] ({-1,1})
    (bgemm_linear.py:45-86).  The kernel sees attn as the weight-side operand with INSTR=2."""

    @staticmethod
    def forward(ctx, input1, input2, instruction="attn_mm"):
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            input1, input2 = input1.to(torch.half), input2.to(torch.half)
            ctx.save_for_backward(input1, input2)
        # attn stays as it lies (activation side, {0,1}), the value operand is packed as it lies by the
        # transposing pack, and the result comes out as [..., S_q, d] directly: none of the reference's
        # three transposes (bgemm_linear.py:58-61)
        if input1.dim() > 2:
            return _batched_packed(input1, input2, lowbit_kernel.MODE_ATTN_X)
        return lowbit_kernel.bgemm_packed_forward(_pack_right(input2), lowbit_kernel.pack_sign(input1),
                                                  lowbit_kernel.MODE_ATTN_X, torch.half, splitK=8)[0]

    @staticmethod
    def backward(ctx, grad_output):
        attn, value = ctx.saved_tensors
        a01 = (attn.sign() + 1) / 2
        a01 = torch.where(a01 == 0, torch.ones_like(a01), a01)     # as the reference does (:70-71)
        v = value.sign()
        g = grad_output.to(v.dtype)
        return (g @ v.transpose(-1, -2)) / 2, a01.transpose(-1, -2) @ g, None


class bgemm_linear(torch.autograd.Function):
    """out = sign(input) @ sign(weight).T on the binary kernel (bgemm_linear.py:131-165)."""

    @staticmethod
    def forward(ctx, input, weight, instruction='xor'):
        input, weight = input.to(torch.half), weight.to(torch.half)
        ctx.save_for_backward(input, weight)
        return _kernel_2d(input, weight, _instr(instruction))

    @staticmethod
    def backward(ctx, grad_output):
        x, w = ctx.saved_tensors
        grad_x, grad_w = _linear_grads(grad_output, x.sign(), w.sign())
        return grad_x, grad_w, None


class bgemm_linear_bireal(torch.autograd.Function):
    """As bgemm_linear with the Bi-Real surrogate 2 - 2|x| on the input gradient (:168-219)."""

    @staticmethod
    def forward(ctx, input, weight, instruction='xor'):
        input, weight = input.to(torch.half), weight.to(torch.half)
        ctx.save_for_backward(input, weight)
        return _kernel_2d(input, weight, _instr(instruction))

    @staticmethod
    def backward(ctx, grad_output):
        x, w = ctx.saved_tensors
        grad_x, grad_w = _linear_grads(grad_output, x.sign(), w.sign())
        return grad_x * (2 - 2 * x.abs().clamp(max=1)), grad_w, None


def ternary(x, is_act=True):
    """The reference's ternariser is plain sign (bgemm_linear.py:222-241)."""
    return x.sign()


def calculate_gradient_signed(qx, grad, grad_scale, is_act):
    """Scale gradient of the elastic quantiser (bgemm_linear.py:519-535)."""
    if is_act:
        small, big = (qx < -1).float(), (qx > 1).float()
        middle = 1.0 - small - big
        inner = big - small + middle * (ternary(qx, True) - qx)
    else:
        inner = ternary(qx, False)
    return grad, (inner * grad * grad_scale).sum(dim=-1).unsqueeze(dim=0)


def _elastic_prepare(input, weight, sa):
    # the means stay on the device: subtracting the 0-dim tensor gives the values that subtracting its
    # `.item()` gives (bgemm_linear.py:357-358) without the two host synchronisations
    x = input - input.mean()
    w = weight - weight.mean()
    return x / sa, w


def _elastic_backward(ctx, grad_output, surrogate, clip):
    x, w = ctx.saved_tensors
    grad_x, grad_w = _linear_grads(grad_output, ternary(x, True), ternary(w, False))
    grad_x, grad_sa = calculate_gradient_signed(x, grad_x, ctx.other, True)
    _, grad_sw = calculate_gradient_signed(w, grad_w, ctx.other, False)
    grad_x = grad_x * surrogate(x.abs().clamp(max=clip))
    grad_w = grad_w * surrogate(w.abs().clamp(max=clip))
    return grad_x, grad_w, grad_sa, grad_sw, None, None


class nn_linear_elastic_signed(torch.autograd.Function):
    """The CPU-runnable path: ternary(x) @ ternary(w).T in torch (bgemm_linear.py:243-347)."""

    @staticmethod
    def forward(ctx, input, weight, sa, sw, grad_scale, instruction="xor"):
        x, w = _elastic_prepare(input, weight, sa)
        ctx.other = grad_scale
        ctx.save_for_backward(x, w)
        xt, wt = ternary(x.to(torch.half), True), ternary(w.to(torch.half), False)
        return (xt @ wt.T) * sa * sw

    @staticmethod
    def backward(ctx, grad_output):
        return _elastic_backward(ctx, grad_output, lambda t: 2 * torch.exp(-t ** 2), 1)


class bgemm_linear_elastic_signed(torch.autograd.Function):
    """Elastic-scale binary linear on the kernel (bgemm_linear.py:350-457)."""

    @staticmethod
    def forward(ctx, input, weight, sa, sw, grad_scale, instruction="xor"):
        x, w = _elastic_prepare(input, weight, sa)
        ctx.other = grad_scale
        ctx.save_for_backward(x, w)
        out = _kernel_2d(x.to(torch.half), w.to(torch.half), _instr(instruction))
        return out * sa * sw

    @staticmethod
    def backward(ctx, grad_output):
        return _elastic_backward(ctx, grad_output, lambda t: 2 / torch.cosh(t) ** 2, 4)


class BinActive(torch.autograd.Function):
    """sign with 0 -> +1, identity gradient (bgemm_linear.py:599-616)."""

    @staticmethod
    def forward(ctx, input):
        s = input.sign()
        return torch.where(s == 0, torch.ones_like(s), s)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output.clone()


class _ScaledBinaryLinear(nn.Linear):
    """Shared state of the binary Linear modules: lazily initialised scales and zero points
    (bgemm_linear.py:466-472): sw = |w|_1 per output row / numel, sa = 2 mean|x|."""

    def __init__(self, in_channels, out_channels, bias=False):
        super().__init__(in_channels, out_channels, bias)
        self.initialized = False

    def _initialize(self, x, w):
        assert not self.initialized, 'already initialized.'
        self.sw = nn.Parameter(w.norm(1, 1).div(w.nelement()), requires_grad=True)
        self.sa = nn.Parameter(2 * x.abs().mean(), requires_grad=True)
        self.grad_scale = 1.0 / math.sqrt(x.numel())
        self.zpw = torch.mean(w).detach()
        self.zpa = torch.mean(x).detach()
        self.initialized = True

    def _add_bias(self, out):
        if self.bias is not None:
            out += self.bias.view(1, -1).expand_as(out)
        return out

    # The inference paths keep the weight's packed bits, keyed on the weight tensor's version counter, storage and
    # type.  The counter only sees writes made through the tensor itself: an update through ``weight.data``
    # (``p.data.copy_(...)``, ``p.data.clamp_()``, as some BNN training loops do) leaves it unchanged.  The cache is
    # therefore also dropped whenever the module changes mode (train() / eval()) or loads a state dict, and
    # invalidate_packed_weight() drops it by hand after such a write.
    def invalidate_packed_weight(self):
        """Forget the cached packed weight: the next inference forward packs the float weight again."""
        self.__dict__.pop("_wp", None)
        self.__dict__.pop("_wp_key", None)

    def train(self, mode=True):
        self.invalidate_packed_weight()
        return super().train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        self.invalidate_packed_weight()
        return super()._load_from_state_dict(*args, **kwargs)


class BGEMMLinear(_ScaledBinaryLinear):
    """out = bgemm(x - zpa, w - zpw) * sw * sa (+ bias)  (bgemm_linear.py:460-486).

    Under ``torch.no_grad()`` the forward is fused (``fuse_inference``) and multiplies with a cached packed copy of
    the weight.  The cache follows every update made through the parameter or the weight's zero point ``zpw``
    (optimizer steps, ``copy_``, ``+=``) and is
    dropped by ``train()`` / ``eval()`` and ``load_state_dict``; after a write through ``weight.data`` call
    ``invalidate_packed_weight()``."""
    _fn = bgemm_linear
    fuse_inference = True

    def _fusable(self, x):
        dt = self.weight.dtype
        return (self.fuse_inference and not torch.is_grad_enabled() and x.is_cuda and dt in (torch.float32, torch.half)
                and x.dtype == dt and self.sw.dtype == dt and self.sa.dtype == dt
                and (self.bias is None or self.bias.dtype == dt))

    def _weight_key(self):
        # the packed bits are those of (weight - zpw): an in-place update of the zero point alone (a calibration pass,
        # an optimizer group of its own) must pack again as well
        return (self.weight._version, self.weight.data_ptr(), self.weight.dtype, id(self.zpw), self.zpw._version,
                self.zpw.data_ptr())

    def _packed_weight(self):
        key = self._weight_key()
        if getattr(self, "_wp_key", None) != key:
            self._wp = lowbit_kernel.pack_sign(self.weight.detach(), zero_point=self.zpw)
            self._wp_key = key
        return self._wp

    def use_packed_weight(self, packed):
        """Install an already packed, centred weight (for instance one read from a file) as the operand of the
        inference path; it is used until the float weight changes."""
        if (packed.rows, packed.K) != tuple(self.weight.shape):
            raise ValueError(f"packed weight is {packed.rows}x{packed.K} bits, the layer is {tuple(self.weight.shape)}")
        self._wp, self._wp_key = packed, self._weight_key()

    def _inference_state(self):
        """Detached views of the parameters for the inference path, rebuilt only when a parameter is replaced or
        moved (new object or new storage); in-place updates show through the views."""
        key = (id(self.sw), self.sw.data_ptr(), id(self.sa), self.sa.data_ptr(), id(self.bias),
               None if self.bias is None else self.bias.data_ptr(), id(self.zpa), self.zpa.data_ptr(), self.weight.dtype)
        st = self.__dict__.get("_inf")
        if st is None or st[0] != key:
            dt = self.weight.dtype
            sw, sa = self.sw.detach().contiguous(), self.sa.detach().reshape(1)
            bias = None if self.bias is None else self.bias.detach().contiguous()
            zpa = self.zpa.detach().to(dt).reshape(1)
            same = self.zpa.dtype == dt           # otherwise zpa above is a copy: refresh it on every call
            st = self.__dict__["_inf"] = (key, sw, sa, bias, zpa if same else None)
        return st

    def _fused_forward(self, x):
        lead = x.shape[:-1]
        _, sw, sa, bias, zpa = self._inference_state()
        if zpa is None:
            zpa = self.zpa.detach().to(x.dtype).reshape(1)
        x2 = x.reshape(-1, x.shape[-1])
        wp = self._packed_weight()
        # a few rows (a decode step): one launch, the kernel centres and packs x itself; more rows: one pack
        # launch, then the GEMM (the library only splits K where the output tiles alone leave CUs idle)
        if x2.shape[0] <= 4 and x2.is_contiguous() and lowbit_kernel.decode_shape_supported(lowbit_kernel.MODE_XOR, wp.rows, x2.shape[0], wp.K):
            out = lowbit_kernel.decode_linear_launch(wp, x2, sw, sa, bias, zpa)
        else:
            out = lowbit_kernel.bgemm_packed_weight_forward(wp, x2, lowbit_kernel.MODE_XOR, scale=(sw, sa, bias), x_zero_point=zpa)
        return out.reshape(*lead, self.weight.shape[0])

    def forward(self, x):
        if not self.initialized:
            self._initialize(x, self.weight)
        if self._fusable(x):
            return self._fused_forward(x)
        out = self._fn.apply(x - self.zpa, self.weight - self.zpw) * self.sw * self.sa
        return self._add_bias(out)


class BGEMMChain(nn.Sequential):
    """BGEMMLinear layers applied back to back (the binarisation is the only nonlinearity between them).
    When no gradient is recorded the activations between layers exist only as bits: every GEMM but the last
    writes the next layer's centred, sign-packed operand straight from its accumulators, so a chain of L
    layers is L + 1 launches and never stores a hidden activation.  Same results as calling the layers one
    after the other, bit for bit.  Not in the reference, which has no layer container."""

    def _fusable(self, x):
        layers = list(self)
        return (len(layers) > 0 and all(isinstance(l, BGEMMLinear) and l.initialized and l._fn is not None for l in layers)
                and all(l._fusable(x) for l in layers)
                and all(a.weight.shape[0] == b.weight.shape[1] for a, b in zip(layers, layers[1:])))

    def forward(self, x):
        if not self._fusable(x):
            return super().forward(x)          # also the first call, which initialises the layers' scales
        layers = list(self)
        lead = x.shape[:-1]
        xp = lowbit_kernel.pack_sign(x.reshape(-1, x.shape[-1]), zero_point=layers[0].zpa)
        if not hasattr(self, "_bits"):
            self._bits = {}
        for i, layer in enumerate(layers):
            scale = (layer.sw.detach(), layer.sa.detach().reshape(1), None if layer.bias is None else layer.bias.detach())
            if i + 1 == len(layers):
                out = lowbit_kernel.bgemm_packed_forward(layer._packed_weight(), xp, lowbit_kernel.MODE_XOR, splitK=8, scale=scale)
                return out.reshape(*lead, layer.weight.shape[0])
            key = (i, xp.rows, x.device)
            if key not in self._bits:      # zero-filled once: the GEMM writes real bits only, the padding stays zero
                self._bits[key] = lowbit_kernel.zeros_packed(xp.rows, layer.weight.shape[0], 1, x.device)
            xp = lowbit_kernel.bgemm_packed_forward(layer._packed_weight(), xp, lowbit_kernel.MODE_XOR, splitK=8, scale=scale,
                                                    bits_out=self._bits[key],
                                                    next_zero_point=layers[i + 1].zpa.detach().reshape(1))


class GraphedInference:
    """``module(x)`` under ``no_grad`` captured once into a HIP graph and replayed per call: the launches of a
    binary layer, chain or block are a few microseconds each, less than it costs to issue them from Python, so a
    replay (one call into the runtime) is what makes a small model run at the speed of its kernels.

    The capture fixes the input's shape and dtype, the packed weights and every buffer: parameters updated in
    place afterwards (scales, biases) are seen, a changed or replaced weight is not (capture again).  The
    returned tensor is the graph's own output buffer, overwritten by the next call.  Not in the reference."""

    def __init__(self, module, example):
        if not example.is_cuda:
            raise ValueError("the example input must be on the GPU")
        self.module = module
        self._x = example.detach().clone()
        with torch.no_grad():
            side = torch.cuda.Stream(device=example.device)
            side.wait_stream(torch.cuda.current_stream(example.device))
            with torch.cuda.stream(side):
                for _ in range(2):                 # initialises scales, packs weights, grows cached buffers
                    module(self._x)
                side.synchronize()
                self._graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(self._graph, stream=side):
                    self._y = module(self._x)
            torch.cuda.current_stream(example.device).wait_stream(side)

    def __call__(self, x):
        if x.shape != self._x.shape or x.dtype != self._x.dtype or x.device != self._x.device:
            raise ValueError("captured for %s %s on %s, got %s %s on %s" % (tuple(self._x.shape), self._x.dtype,
                             self._x.device, tuple(x.shape), x.dtype, x.device))
        self._x.copy_(x)
        self._graph.replay()
        return self._y


class BGEMMLinear_bireal(BGEMMLinear):
    """BGEMMLinear with the Bi-Real backward (bgemm_linear.py:489-516)."""
    _fn = bgemm_linear_bireal


class BGEMMLinear_elastic_signed(_ScaledBinaryLinear):
    """Learned-scale binary linear (bgemm_linear.py:538-564).

    When no gradient is being recorded the forward runs on packed operands: the kernel only sees the sign bits of
    ``(x - mean(x)) / sa`` and ``w - mean(w)`` (bgemm_linear.py:357-373), and for a positive ``sa`` the division
    does not change a sign, so the activations are centred and packed in one pass and the weight's bits are
    packed once per weight version; the scaling stays in torch, in the reference's order ``out * sa * sw``."""
    _fn = bgemm_linear_elastic_signed
    fuse_inference = True

    def __init__(self, in_channels, out_channels, bias=True):
        super().__init__(in_channels, out_channels, bias)

    def _fusable(self, x):
        if not (self.fuse_inference and self._fn is bgemm_linear_elastic_signed and not torch.is_grad_enabled()
                and x.is_cuda and x.dtype in (torch.float32, torch.half) and self.weight.dtype in (torch.float32, torch.half)):
            return False
        key = (id(self.sa), self.sa._version, self.sa.data_ptr())
        if self.__dict__.get("_sa_key") != key:          # one read-back per update of sa, none per forward
            self._sa_positive, self._sa_key = bool((self.sa.detach() > 0).all()), key
        return self._sa_positive

    def _packed_weight(self):
        w = self.weight
        key = (w._version, w.data_ptr(), w.dtype)
        if self.__dict__.get("_wp_key") != key:
            self._wp = lowbit_kernel.pack_sign(w.detach(), zero_point=w.detach().mean().reshape(1))
            self._wp_key = key
        return self._wp

    def _fused_forward(self, x):
        x2 = x.reshape(-1, x.shape[-1])
        xp = lowbit_kernel.pack_sign(x2, zero_point=x.mean().reshape(1))
        out = lowbit_kernel.bgemm_packed_forward(self._packed_weight(), xp, lowbit_kernel.MODE_XOR, torch.half, splitK=8)[0]
        return (out * self.sa * self.sw).reshape(*x.shape[:-1], self.weight.shape[0])

    def forward(self, x):
        if not self.initialized:
            self._initialize(x, self.weight)
        if self._fusable(x):
            return self._add_bias(self._fused_forward(x))
        return self._add_bias(self._fn.apply(x, self.weight, self.sa, self.sw, self.grad_scale))


class NNLinear_elastic_signed(BGEMMLinear_elastic_signed):
    """Same layer on the torch CPU/GPU matmul path (bgemm_linear.py:569-595)."""
    _fn = nn_linear_elastic_signed


class BNNLinear(_ScaledBinaryLinear):
    """Dense torch baseline: F.linear(BinActive(x - zpa), BinActive(w - zpw)) * sw * sa (:619-645)."""

    def forward(self, x):
        if not self.initialized:
            self._initialize(x, self.weight)
        bw = BinActive.apply(self.weight - self.zpw)
        bx = BinActive.apply(x - self.zpa)
        return nn.functional.linear(bx, bw, self.bias) * self.sw * self.sa
