"""Softmax attention over a shared low-rank latent, kept in a paged cache.

Per token the part caches one vector [c | k_r]: c, the normalised key/value latent of
`kv_rank` elements, and k_r, `rot_dim` rotated key elements shared by all heads.  Head j's
key is [U_k,j c | k_r] and its value U_v,j c, so with q_j = [q_n | q_r] (the rotated part
rotated like k_r)

    score_j(i, t) = scale * ((U_k,j^T q_n) . c_t + q_r . k_r,t)
    out_j(i)      = U_v,j  sum_t softmax_t(score_j(i, t)) c_t

and neither keys nor values are ever expanded: queries are carried into the latent's space
before attention, and its output back out of it afterwards.  Both steps are folded into the
weights when they are loaded (products taken in float64, rounded once to the run's dtype):
the query up-projection becomes [U_k,j^T U_q,j ; U_q,j's rotated rows] per head, a plain
product from the query latent straight to q', and the output projection becomes
W_o,j U_v,j per head, a plain product from the attention's latent-space result to the
model width.  Queries come through a latent of their own (down, RMS norm, up).  A window W
lets position i see positions i-W+1..i.
"""

from __future__ import annotations

import torch

from tokensprint_amd.parts.base import MIXERS, Mixer, PagedLatentNeed, TensorDecl, register


@register(MIXERS, "latent_attention")
class LatentAttention(Mixer):
    """params: prefix, heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, eps, window (None
    = all earlier tokens), position (name of a shared interleaved rotation)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.prefix = p["prefix"]
        self.heads, self.dim, self.rot_dim = int(p["heads"]), int(p["dim"]), int(p["rot_dim"])
        self.vdim, self.q_rank, self.kv_rank = int(p["vdim"]), int(p["q_rank"]), int(p["kv_rank"])
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.window = p.get("window")
        self.position = ctx.positions[p["position"]]
        if self.position.dims > self.rot_dim:
            raise ValueError(f"{self.prefix}: the rotation covers {self.position.dims} "
                             f"dimensions, the rotated part has {self.rot_dim}")
        self.w_down = self.w_query = self.w_out = None
        self.q_norm = self.kv_norm = None

    def tensors(self):
        W, pre, H = self.ctx.width, self.prefix, self.heads
        return {
            pre + "dq": TensorDecl((self.q_rank, W)),
            pre + "dq.norm": TensorDecl((self.q_rank,), role="vector"),
            pre + "uq": TensorDecl((H * (self.dim + self.rot_dim), self.q_rank)),
            pre + "dkv": TensorDecl((self.kv_rank + self.rot_dim, W)),
            pre + "dkv.norm": TensorDecl((self.kv_rank,), role="vector"),
            pre + "uk": TensorDecl((H * self.dim, self.kv_rank)),
            pre + "uv": TensorDecl((H * self.vdim, self.kv_rank)),
            pre + "o": TensorDecl((W, H * self.vdim)),
        }

    def load(self, get):
        pre = self.prefix
        dq, dkv = get(pre + "dq"), get(pre + "dkv")
        if dq.dtype != dkv.dtype:
            raise ValueError(f"{pre}: the two down projections are stored in different dtypes")
        self.w_down = torch.cat([dq, dkv], dim=0).contiguous()
        self.q_norm, self.kv_norm = get(pre + "dq.norm"), get(pre + "dkv.norm")
        H, dn, dr, R, dv = self.heads, self.dim, self.rot_dim, self.kv_rank, self.vdim
        uq, uk, uv, wo = get(pre + "uq"), get(pre + "uk"), get(pre + "uv"), get(pre + "o")
        uq64 = uq.double().view(H, dn + dr, self.q_rank)
        carried = torch.einsum("hdr,hdq->hrq", uk.double().view(H, dn, R), uq64[:, :dn])
        self.w_query = torch.cat([carried, uq64[:, dn:]], dim=1) \
            .reshape(H * (R + dr), self.q_rank).to(uq.dtype).contiguous()
        self.w_out = torch.einsum("whv,hvr->whr", wo.double().view(-1, H, dv),
                                  uv.double().view(H, dv, R)) \
            .reshape(-1, H * R).to(wo.dtype).contiguous()

    def cache_need(self):
        return PagedLatentNeed(self.kv_rank + self.rot_dim, self.window)

    def forward(self, h, batch, cache, write_cache):
        if cache is None or cache.k_pages is None:
            raise RuntimeError("latent_attention needs a paged latent cache")
        if not write_cache:
            raise RuntimeError(f"{self.prefix}: reading another run's latent cache is not built")
        ops = self.ops
        table = batch.tables[cache.group]
        freqs, rot_dims = self.position.frequencies(), self.position.dims
        proj = ops.linear(h, self.w_down, torch.float32)
        cq = ops.latent_prepare(proj, batch, table, cache, q_rank=self.q_rank,
                                kv_rank=self.kv_rank, rot_dim=self.rot_dim, q_norm=self.q_norm,
                                kv_norm=self.kv_norm, eps=self.eps, freqs=freqs,
                                rot_dims=rot_dims, out_dtype=self.ctx.dtype)
        T = h.shape[0]
        qa = ops.linear(cq, self.w_query, torch.float32).view(T, self.heads,
                                                              self.kv_rank + self.rot_dim)
        ops.rotate_interleaved_inplace(qa, batch.positions, freqs, rot_dims, offset=self.kv_rank)
        ol = ops.latent_attention(qa, batch, table, cache, heads=self.heads,
                                  kv_rank=self.kv_rank, rot_dim=self.rot_dim, scale=self.scale,
                                  window=self.window, out_dtype=self.ctx.dtype)
        return ops.linear(ol.view(T, self.heads * self.kv_rank), self.w_out, torch.float32)
