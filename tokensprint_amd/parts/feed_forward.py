"""Dense feed-forwards.

SwiGLU: down(silu(gate(h)) * up(h)), no bias
(engine/nn/layers.py:61-66).  Gate and up run as one product over row-concatenated
weights, with the activation applied as the product is written where the kernel
can, and by a separate kernel over both halves otherwise."""

from __future__ import annotations

import torch

from tokensprint_amd.kernels.stream import StreamProducts, fused_rmsnorm_of
from tokensprint_amd.parts.base import FEED_FORWARDS, FeedForward, TensorDecl, register


@register(FEED_FORWARDS, "swiglu")
class SwiGLU(StreamProducts, FeedForward):
    """params: prefix, inner_dim."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.prefix = params["prefix"]
        self.inner = int(params["inner_dim"])
        self.w_gate_up = self.w_down = None

    def tensors(self):
        H, I, pre = self.ctx.width, self.inner, self.prefix
        return {pre + "gate_proj.weight": TensorDecl((I, H)),
                pre + "up_proj.weight": TensorDecl((I, H)),
                pre + "down_proj.weight": TensorDecl((H, I))}

    def load(self, get):
        pre = self.prefix
        g, u = get(pre + "gate_proj.weight"), get(pre + "up_proj.weight")
        if g.dtype != u.dtype:
            raise ValueError(f"{pre}: gate and up weights are stored in different dtypes")
        self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = get(pre + "down_proj.weight")

    def stream_hint(self, norm):
        return self.first_product_hint(norm, self.w_gate_up, silu_mul=True)

    def forward_from_stream(self, resid, delta, norm, batch, hint=None):
        fused = fused_rmsnorm_of(norm)
        if fused is None:
            return super().forward_from_stream(resid, delta, norm, batch)
        act, resid = self.ops.norm_linear(resid, delta, fused[0], fused[1], self.w_gate_up,
                                          self.ctx.dtype, silu_mul=True)
        return self.last_product(act, self.w_down, resid, hint), resid

    def forward(self, h, batch):
        act = self.ops.linear_silu_mul(h, self.w_gate_up, self.ctx.dtype)
        return self.ops.linear(act, self.w_down, self.ctx.dtype)


@register(FEED_FORWARDS, "polynorm_mlp")
class PolyNormMLP(FeedForward):
    """down(act(up(h))) with the PolyNorm activation: with N(v) = v / rms(v) over a
    token's inner values (eps inside the root) and powers taken element by element,
    act(z) = a N(z) + b N(z^2) + c N(z^3) + e; (a, b, c, e) is the tensor '<prefix>act'.
    The activation is computed in float32 on the product's float32 sums.

    params: prefix, inner_dim, eps."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.prefix = params["prefix"]
        self.inner = int(params["inner_dim"])
        self.eps = float(params["eps"])
        self.w_up = self.w_down = self.coef = None

    def tensors(self):
        W, I, pre = self.ctx.width, self.inner, self.prefix
        return {pre + "up": TensorDecl((I, W)), pre + "down": TensorDecl((W, I)),
                pre + "act": TensorDecl((4,), role="vector", init=(0.1, 0.6))}

    def load(self, get):
        pre = self.prefix
        self.w_up, self.w_down, self.coef = get(pre + "up"), get(pre + "down"), get(pre + "act")

    def forward(self, h, batch):
        z = self.ops.linear(h, self.w_up, torch.float32)
        act = self.ops.polynorm(z, self.coef, self.eps, self.ctx.dtype)
        return self.ops.linear(act, self.w_down, torch.float32)
