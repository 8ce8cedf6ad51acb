"""Mamba-2 mixer (state-space duality form): a selective state-space recurrence with one
scalar decay per head and token.

With inner = heads * vdim, N = state, G = groups, the input projection's rows are
[z: inner | x: inner | B: G N | C: G N | dt: heads].  x, B and C pass a short causal
convolution per channel (bias, then SiLU).  Per head h (group g = h // (heads / G)), with
d = softplus(dt + dt_bias_h) and a = exp(-exp(A_log_h) d):

    S <- a S + d B_g x_h^T        (S is N x vdim, float32, zero at a sequence's start)
    y_h = S^T C_g + D_h x_h

The heads' y, times SiLU(z), are normalised in `norm_groups` equal parts (each by its own
root mean square), scaled by the norm weight and projected out.  Per request the part keeps
the recurrence's state and the convolution's last taps - 1 inputs, both in float32, in the
request's state slot; a step continues from what the step before left.
"""

from __future__ import annotations

import math

import torch

from tokensprint_amd.parts.base import MIXERS, Mixer, SlotStateNeed, TensorDecl, register


@register(MIXERS, "mamba2")
class Mamba2(Mixer):
    """params: prefix, heads, vdim, state, groups, conv (taps), norm_groups, eps."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.prefix = p["prefix"]
        self.heads, self.vdim, self.state = int(p["heads"]), int(p["vdim"]), int(p["state"])
        self.groups, self.taps = int(p["groups"]), int(p["conv"])
        self.norm_groups, self.eps = int(p["norm_groups"]), float(p["eps"])
        self.inner = self.heads * self.vdim
        self.bc = self.groups * self.state
        self.channels = self.inner + 2 * self.bc
        if self.heads % self.groups or self.inner % self.norm_groups:
            raise ValueError(f"{self.prefix}: heads={self.heads} must be a multiple of groups="
                             f"{self.groups}, heads*vdim of norm_groups={self.norm_groups}")
        self.w_in = self.w_o = self.conv_w = self.conv_b = None
        self.dt_bias = self.a_log = self.d_skip = self.norm_w = None

    def tensors(self):
        W, pre, H = self.ctx.width, self.prefix, self.heads
        return {
            pre + "in": TensorDecl((2 * self.inner + 2 * self.bc + H, W)),
            pre + "conv": TensorDecl((self.channels, self.taps), role="vector", init=(-0.6, 0.6)),
            pre + "conv.b": TensorDecl((self.channels,), role="vector", init=(-0.1, 0.1)),
            pre + "dt_bias": TensorDecl((H,), role="vector", init=(-3.0, -0.5)),
            pre + "A_log": TensorDecl((H,), role="vector", init=(-1.0, math.log(8.0))),
            pre + "D": TensorDecl((H,), role="vector"),
            pre + "norm": TensorDecl((self.inner,), role="vector"),
            pre + "o": TensorDecl((W, self.inner)),
        }

    def load(self, get):
        pre = self.prefix
        self.w_in, self.w_o = get(pre + "in"), get(pre + "o")
        self.conv_w, self.conv_b = get(pre + "conv"), get(pre + "conv.b")
        self.dt_bias, self.a_log = get(pre + "dt_bias"), get(pre + "A_log")
        self.d_skip, self.norm_w = get(pre + "D"), get(pre + "norm")

    def cache_need(self):
        return (SlotStateNeed((max(self.taps - 1, 0), self.channels), torch.float32, "conv"),
                SlotStateNeed((self.heads, self.state, self.vdim), torch.float32, "ssm"))

    def forward(self, h, batch, cache, write_cache):
        if cache is None or "ssm" not in cache.states:
            raise RuntimeError("mamba2 needs its per-request state")
        if not write_cache:
            raise RuntimeError(f"{self.prefix}: a recurrence cannot read another run's state")
        ops = self.ops
        proj = ops.linear(h, self.w_in, torch.float32)
        xbc = ops.conv_silu(proj, self.inner, self.channels, self.conv_w, self.conv_b, batch,
                            cache.states["conv"])
        y = ops.ssm_scan(xbc, proj, 2 * self.inner + 2 * self.bc, self.dt_bias, self.a_log,
                         self.d_skip, batch, cache.states["ssm"], heads=self.heads,
                         vdim=self.vdim, state_rows=self.state, groups=self.groups)
        gated = ops.gated_group_norm(y, proj, self.norm_w, self.norm_groups, self.eps,
                                     self.ctx.dtype)
        return ops.linear(gated, self.w_o, torch.float32)
