"""Plain Palelix forward: one function per mechanism, whole sequences, no cache, CPU torch.

Everything runs over a whole sequence [T, ...] in one precision (float64 by default), a
token at a time wherever the design is a recurrence, so that a mistake in the engine's
state, cache or batch handling cannot be mirrored here.  Nothing imports the engine package.

Notation: T tokens, D model width, eps the model's norm epsilon; a linear weight W is
[out, in] and applied as x W^T.
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
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def unit_vector(x):
    """x / sqrt(sum(x^2) + 1e-6) over the last axis."""
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)


def short_conv(x, taps_w):
    """Causal convolution over time per channel: x [T, C], taps_w [C, taps]; the last column
    weighs the current token, zeros stand before the sequence."""
    T, C = x.shape
    taps = taps_w.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                out[t] += x[src] * taps_w[:, j]
    return out


# --------------------------------------------------------------------------- recurrences


def lightning_attention(q, k, v, decay):
    """q, k [T, H, dk], v [T, H, dv], decay [H]: S_t = decay S_(t-1) + k_t v_t^T (S is
    dk x dv), o_t = S_t^T q_t.  Returns [T, H, dv]."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for h in range(H):
        S = torch.zeros(dk, dv, dtype=q.dtype)
        for t in range(T):
            S = decay[h] * S + torch.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    return out


def gated_delta_rule(q, k, v, beta, g):
    """q, k [T, H, dk], v [T, H, dv], beta [T, H]; g [T, H] (a decay per head) or [T, H, dk]
    (a decay per key channel, i.e. per row of S).  Per head and token, in this order:
    S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for h in range(H):
        S = torch.zeros(dk, dv, dtype=q.dtype)
        for t in range(T):
            gt = g[t, h]
            S = S * (gt.unsqueeze(-1) if gt.dim() == 1 else gt)
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + torch.outer(k[t, h], u)
            out[t, h] = S.T @ q[t, h]
    return out


# --------------------------------------------------------------------------- mixers


def lightning_mixer(h, w, pre, m, eps):
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ w[pre + "q"].T).view(T, H, dk)
    k = silu(h @ w[pre + "k"].T).view(T, H, dk)
    v = silu(h @ w[pre + "v"].T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    o = lightning_attention(q, k, v, decay).reshape(T, H * dv)
    o = rms_norm(o, w[pre + "norm"], eps) * sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def delta_mixer(h, w, pre, m, eps, per_channel):
    """The gated delta rule mixer; `per_channel`: the decay comes from a two-step projection
    and differs per key channel, and the output gate is a sigmoid of a two-step projection;
    otherwise one decay per head and a SiLU gate of one projection."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).view(T, G, dk)
    k = silu(short_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).view(T, G, dk)
    v = silu(short_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).view(T, H, dv)
    q = unit_vector(q) * dk ** -0.5
    k = unit_vector(k)
    rep = H // G
    q = q.repeat_interleave(rep, dim=1)
    k = k.repeat_interleave(rep, dim=1)
    beta = sigmoid(h @ w[pre + "b"].T)                                  # [T, H]
    a = torch.exp(w[pre + "A_log"])                                     # [H]
    if per_channel:
        z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]  # [T, H*dk]
        g = torch.exp(-a.view(1, H, 1) * softplus(z).view(T, H, dk))
        gate = sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T)
    else:
        z = h @ w[pre + "a"].T + w[pre + "dt_bias"]                     # [T, H]
        g = torch.exp(-a * softplus(z))
        gate = silu(h @ w[pre + "g"].T)
    o = gated_delta_rule(q, k, v, beta, g)                              # [T, H, dv]
    o = unit_rms(o, eps) * w[pre + "norm"]
    return (o.reshape(T, H * dv) * gate) @ w[pre + "o"].T


def rotate_half(x, positions, dims, base):
    """x [T, heads, dim]: the first `dims` dimensions rotated, dimension i paired with
    i + dims/2, angle position * base^(-2i/dims)."""
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(x.dtype).unsqueeze(-1) * freq                   # [T, half]
    c, s = ang.cos().unsqueeze(1), ang.sin().unsqueeze(1)
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def softmax_attention(h, w, pre, m):
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    pos = torch.arange(T)
    q = rotate_half((h @ w[pre + "q"].T).view(T, H, dk), pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_half((h @ w[pre + "k"].T).view(T, G, dk), pos, m["rot"]["dims"], m["rot"]["base"])
    v = (h @ w[pre + "v"].T).view(T, G, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        for t in range(T):
            s = (k[: t + 1, g] @ q[t, hd]) * m["scale"]
            p = torch.softmax(s, dim=0)
            out[t, hd] = p @ v[: t + 1, g]
    return out.reshape(T, H * dv) @ w[pre + "o"].T


def parallel_mixer(h, w, pre, m, eps):
    left = softmax_attention(h, w, pre + "left.", m["left"])
    right = delta_mixer(h, w, pre + "right.", m["right"], eps, per_channel=True)
    return m["left_scale"] * left + m["right_scale"] * right


# --------------------------------------------------------------------------- feed-forwards


def dense_ff(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def expert_ff(h, w, pre, limit):
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def route(scores, top, group_count, group_keep):
    """scores [E] -> (chosen experts, weights): experts in `group_count` equal groups of
    neighbours; only experts of the `group_keep` groups whose best score is largest can be
    chosen; of those the `top` largest; weights are their scores over their sum."""
    E = scores.shape[0]
    per = E // group_count
    best = scores.view(group_count, per).max(dim=1).values
    kept = torch.topk(best, group_keep).indices
    allowed = torch.zeros(E, dtype=torch.bool)
    for gi in kept.tolist():
        allowed[gi * per:(gi + 1) * per] = True
    masked = torch.where(allowed, scores, torch.full_like(scores, -1.0))
    chosen = torch.topk(masked, top).indices
    wts = scores[chosen]
    return chosen, wts / (wts.sum() + 1e-20)


def moe_ff(h, w, pre, mlp):
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    scores = torch.softmax(h @ w[pre + "router"].T, dim=-1)
    out = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        chosen, wts = route(scores[t], top, r["groups"]["count"], r["groups"]["keep"])
        for e, wt in zip(chosen.tolist(), wts):
            out[t] += wt * expert_ff(h[t:t + 1], w, f"{pre}e{e}.", mlp["expert"]["limit"])[0]
    return out


# --------------------------------------------------------------------------- whole model


def run_order(cfg):
    """(layer index, pass number or None) in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t) for i in range(loop["start"], loop["stop"])]
    order += [(i, None) for i in range(loop["stop"], n)]
    return order


def layer(x, w, cfg, i):
    entry = cfg["layers"][i]
    eps = cfg["norm"]["eps"]
    pre = f"l{i}."
    h = rms_norm(x, w[pre + "norm1"], eps)
    kind, m = entry["type"], entry["mixer"]
    if kind == "lightning":
        y = lightning_mixer(h, w, pre + "mix.", m, eps)
    elif kind == "delta":
        y = delta_mixer(h, w, pre + "mix.", m, eps, per_channel=False)
    elif kind == "parallel":
        y = parallel_mixer(h, w, pre + "mix.", m, eps)
    else:
        raise ValueError(kind)
    mlp = entry.get("mlp")
    if mlp is not None:
        if mlp["kind"] == "dense":
            y = y + dense_ff(h, w, pre + "mlp.")
        else:
            y = y + moe_ff(h, w, pre + "mlp.", mlp)
    return x + y


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of a whole sequence (and the stream after every layer run)."""
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    loop = cfg.get("loop")
    streams = []
    for i, t in run_order(cfg):
        if t is not None and i == loop["start"]:
            x = x + w["loop.step"][t]
        x = layer(x, w, cfg, i)
        streams.append(x)
    x = rms_norm(x, w["final.norm"], cfg["norm"]["eps"])
    logits = x @ w["head"].T
    if return_layers:
        return logits, torch.stack(streams)
    return logits
