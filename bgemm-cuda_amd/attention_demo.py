"""A binarised BERT self-attention block on the binary layers and the batched attention pair.

The reference vendors a quantised BERT whose self-attention still multiplies with ``torch.matmul``
(tests/python/bert/bert.py:222-262: Q K^T at :245-246, probabilities x V at :259); its README lists
wiring the binary kernels in as open work.  This block is that wiring, forward and backward:
the four projections are ``BGEMMLinear`` layers, the scores are ``bgemm_matmul(q, k^T)`` on the
sign bits of Q and K, and the context is ``bgemm_attn_matmul(a, v)`` with the probabilities binarised
to {0,1} (1 where a probability is at least the uniform level 1/S, its row's mean) and V to {-1,+1}.  ``kernels=False``
evaluates the same block with dense torch matmuls on the de-binarised tensors, which is what the
tests compare against, bit for bit.

    python attention_demo.py            # times one BERT-base block, kernels against dense torch
"""
import math
import time

import torch
import torch.nn as nn

from bgemm_linear import BGEMMLinear, GraphedInference, bgemm_attn_matmul, bgemm_matmul


def _pm1(t):
    """{-1,+1} by the sign bit (what the kernels read: -0.0 counts as negative)."""
    return torch.where(torch.signbit(t), -1.0, 1.0).to(t.dtype)


class BinarySelfAttention(nn.Module):
    """hidden -> heads x head_size attention with binary operands everywhere a matmul happens
    (bert.py:177-262 with both matmuls on the binary kernels)."""

    def __init__(self, hidden_size=768, num_attention_heads=12, kernels=True):
        super().__init__()
        if hidden_size % num_attention_heads:
            raise ValueError("hidden size %d is not a multiple of %d heads" % (hidden_size, num_attention_heads))
        self.num_attention_heads = num_attention_heads
        self.attention_head_size = hidden_size // num_attention_heads
        self.kernels = kernels
        self.query = BGEMMLinear(hidden_size, hidden_size, bias=True)
        self.key = BGEMMLinear(hidden_size, hidden_size, bias=True)
        self.value = BGEMMLinear(hidden_size, hidden_size, bias=True)
        self.dense = BGEMMLinear(hidden_size, hidden_size, bias=True)
        self.LayerNorm = nn.LayerNorm(hidden_size, eps=1e-12)

    def transpose_for_scores(self, x):
        return x.view(*x.shape[:-1], self.num_attention_heads, self.attention_head_size).permute(0, 2, 1, 3)

    def forward(self, hidden_states, attention_mask=None):
        q = self.transpose_for_scores(self.query(hidden_states))
        k = self.transpose_for_scores(self.key(hidden_states))
        v = self.transpose_for_scores(self.value(hidden_states))
        if self.kernels:
            scores = bgemm_matmul.apply(q, k.transpose(-1, -2))
        else:
            scores = torch.matmul(_pm1(q.half()).float(), _pm1(k.half()).float().transpose(-1, -2)).half()
        # the scores are small integers held in fp16 (the kernel's output type); the elementwise work between the
        # two matmuls stays in fp16 storage, which is a third of the memory traffic of an fp32 round trip
        scores = scores / math.sqrt(self.attention_head_size)
        if attention_mask is not None:
            scores = scores + attention_mask.to(scores.dtype)
        probs = torch.softmax(scores, dim=-1)
        centred = probs - 1.0 / probs.shape[-1]                     # {0,1}: at least the uniform level 1/S
        if self.kernels:
            context = bgemm_attn_matmul.apply(centred, v)
        else:
            context = torch.matmul((~torch.signbit(centred.half())).float(), _pm1(v.half()).float()).half()
        context = context.permute(0, 2, 1, 3).reshape(*hidden_states.shape[:-1], -1).to(hidden_states.dtype)
        out = self.dense(context)
        return self.LayerNorm(out + hidden_states), scores


def main():
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    block = BinarySelfAttention().to(dev)
    x = torch.randn(16, 512, 768, device=dev)
    with torch.no_grad():
        block(x)                                     # initialises the layers' scales
        for kernels in (True, False):
            block.kernels = kernels
            for _ in range(3):
                block(x)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(20):
                block(x)
            torch.cuda.synchronize()
            print("%-28s %.2f ms per block forward (batch 16, 512 tokens, BERT-base sizes)"
                  % ("binary kernels:" if kernels else "dense torch on +-1 tensors:", (time.perf_counter() - t0) / 20 * 1e3))
        block.kernels = True
        fast = GraphedInference(lambda t: block(t)[0], x)          # the same forward as one captured graph
        for _ in range(3):
            fast(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            fast(x)
        torch.cuda.synchronize()
        print("%-28s %.2f ms per block forward" % ("binary kernels, one graph:", (time.perf_counter() - t0) / 20 * 1e3))


if __name__ == "__main__":
    main()
