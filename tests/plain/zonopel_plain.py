"""Plain Zonopel forward: one function per mechanism, whole sequences, no cache, CPU torch.

Everything runs over a whole sequence [T, ...] in one precision (float64 by default) with
explicit loops where the design is sequential, so that a mistake in the engine's state,
cache or batch handling cannot be mirrored here.  Nothing imports the engine package.

Notation: T tokens, D model width, eps the model's norm epsilon.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


def read_model_dir(model_dir, dtype=torch.float64):
    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    tensors = {}
    for file in sorted(model_dir.glob("*.safetensors")):
        with safe_open(str(file), framework="pt", device="cpu") as f:
            for key in f.keys():
                t = f.get_tensor(key)
                tensors[key] = t.to(dtype) if t.is_floating_point() else t
    return cfg, tensors


# --------------------------------------------------------------------------- small pieces


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


def silu(x):
    return x / (1.0 + torch.exp(-x))


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


# --------------------------------------------------------------------------- embedding


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table for every token: a hash of (previous, current); the first
    token of a sequence takes the table's last row (index `buckets`)."""
    rows = []
    for t, tok in enumerate(tokens):
        if t == 0:
            rows.append(buckets)
        else:
            rows.append((tokens[t - 1] * mul_prev + tok * mul_cur) % buckets)
    return rows


def embed(tokens, table, bigram, norm_weight, scale, buckets, mul_prev, mul_cur, eps):
    ids = torch.tensor(tokens, dtype=torch.long)
    x = table[ids] * scale
    x = x + bigram[torch.tensor(bigram_rows(tokens, buckets, mul_prev, mul_cur))]
    return rms_norm(x, norm_weight, eps)


# --------------------------------------------------------------------------- token shift


def token_shift(h, mix):
    """h_t + (h_(t-1) - h_t) * mix, with h_(-1) = 0; the h on the right is the unshifted one."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * mix


# --------------------------------------------------------------------------- mamba2


def causal_conv(u, weight, bias):
    """u [T, C]; weight [C, taps], the last tap is the current token's; zeros before the
    start.  y_t[c] = bias[c] + sum_k weight[c, k] * u_(t - (taps-1) + k)[c]."""
    T, C = u.shape
    taps = weight.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        acc = bias.clone()
        for k in range(taps):
            s = t - (taps - 1) + k
            if s >= 0:
                acc = acc + weight[:, k] * u[s]
        y[t] = acc
    return y


def ssm_scan(x, B, C, dt, A_log, D, heads, groups):
    """x [T, heads, P]; B, C [T, groups, N]; dt [T, heads] (already positive).
    Per head: S <- exp(-exp(A_log) dt) S + dt * outer(B, x)  (S is [N, P]);
    y = S^T C + D x.  Head h reads group h // (heads / groups)."""
    T, H, P = x.shape
    N = B.shape[-1]
    per = heads // groups
    y = torch.zeros_like(x)
    for h in range(H):
        g = h // per
        S = torch.zeros(N, P, dtype=x.dtype)
        a = -torch.exp(A_log[h])
        for t in range(T):
            S = torch.exp(a * dt[t, h]) * S + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D[h] * x[t, h]
    return y


def mamba2(h, w, pre, p, eps):
    """w: tensors; pre: '<layer>.mix.'; p: the mixer's sizes."""
    H, P, N, G = p["heads"], p["vdim"], p["state"], p["groups"]
    inner = H * P
    proj = h @ w[pre + "in"].T
    z, xbc, dt = torch.split(proj, [inner, inner + 2 * G * N, H], dim=-1)
    xbc = silu(causal_conv(xbc, w[pre + "conv"], w[pre + "conv.b"]))
    x, B, C = torch.split(xbc, [inner, G * N, G * N], dim=-1)
    T = h.shape[0]
    dt = softplus(dt + w[pre + "dt_bias"])
    y = ssm_scan(x.reshape(T, H, P), B.reshape(T, G, N), C.reshape(T, G, N), dt,
                 w[pre + "A_log"], w[pre + "D"], H, G)
    y = y.reshape(T, inner) * silu(z)
    ng = p["norm_groups"]
    y = unit_rms(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * w[pre + "norm"]
    return y @ w[pre + "o"].T


# --------------------------------------------------------------------------- latent attention


def rotate_interleaved(v, positions, base, dims):
    """v [T, ..., d]: dimension 2i pairs with 2i+1 for the first `dims` dimensions."""
    out = v.clone()
    half = dims // 2
    i = torch.arange(half, dtype=v.dtype)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(v.dtype)[:, None] * freq[None, :]            # [T, half]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    cos, sin = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def latent_attention(h, w, pre, p, eps):
    T = h.shape[0]
    H, dn, dr, dv, R = p["heads"], p["dim"], p["rot_dim"], p["vdim"], p["kv_rank"]
    pos = torch.arange(T)
    cq = rms_norm(h @ w[pre + "dq"].T, w[pre + "dq.norm"], eps)
    q = (cq @ w[pre + "uq"].T).reshape(T, H, dn + dr)
    kv = h @ w[pre + "dkv"].T
    c = rms_norm(kv[:, :R], w[pre + "dkv.norm"], eps)
    k_rot = kv[:, R:]                                                 # [T, dr], shared by heads
    k_n = (c @ w[pre + "uk"].T).reshape(T, H, dn)
    v = (c @ w[pre + "uv"].T).reshape(T, H, dv)
    rot = p["rot"]
    q_n, q_r = q[..., :dn], rotate_interleaved(q[..., dn:], pos, rot["base"], rot["dims"])
    k_r = rotate_interleaved(k_rot, pos, rot["base"], rot["dims"])
    window = p["mask"]["size"] if p.get("mask") else None
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for i in range(T):
        lo = 0 if window is None else max(0, i - window + 1)
        for hd in range(H):
            s = (k_n[lo:i + 1, hd] @ q_n[i, hd] + k_r[lo:i + 1] @ q_r[i, hd]) * p["scale"]
            pr = torch.softmax(s, dim=0)
            out[i, hd] = pr @ v[lo:i + 1, hd]
    return out.reshape(T, H * dv) @ w[pre + "o"].T


# --------------------------------------------------------------------------- feed-forward


def poly_norm(z, coef, eps):
    a, b, c, e = [coef[i] for i in range(4)]
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def dense_ff(h, w, pre, eps):
    return poly_norm(h @ w[pre + "up"].T, w[pre + "act"], eps) @ w[pre + "down"].T


# --------------------------------------------------------------------------- model

MIXERS = {"mamba2": mamba2, "latent_attention": latent_attention}


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] for one whole sequence (and the stream after every layer run)."""
    eps = cfg["norm"]["eps"]
    e = cfg["embedding"]
    bg = e["bigram"]
    x = embed(tokens, w["embed"], w["bigram"], w["embed.norm"], e["scale"], bg["buckets"],
              bg["mul_prev"], bg["mul_cur"], eps)
    after = []
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        L = f"l{src}."
        h = token_shift(rms_norm(x, w[L + "norm1"], eps), w[L + "shift"])
        m = MIXERS[layer["type"]](h, w, L + "mix.", layer["mixer"], eps)
        x = x + rms_norm(m, w[L + "norm1b"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']}")
            f = dense_ff(rms_norm(x, w[L + "norm2"], eps), w, L + "mlp.", eps)
            x = x + rms_norm(f, w[L + "norm2b"], eps)
        after.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(after)) if return_layers else logits
