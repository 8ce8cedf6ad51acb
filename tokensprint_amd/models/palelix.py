"""Palelix as a `ModelSpec`: parallel layers (one norm; a mixer and a feed-forward that both
read it) with three kinds of mixer and two of feed-forward, and a stretch of layers that
runs several times with the same weights, every pass with a cache and state of its own and
a row of 'loop.step' added to the stream in front of it.

Tensor names: 'embed', 'loop.step', 'final.norm', 'head', and per layer i 'l<i>.norm1',
'l<i>.mix.*' (a parallel mixer's under '.left.' and '.right.'), 'l<i>.mlp.*'.
"""

from __future__ import annotations

from tokensprint_amd.config.palelix_config import (ARCHITECTURE, DenseFF, DeltaSizes,
                                                   LightningSizes, PalelixConfig)
from tokensprint_amd.config.registry import register_architecture
from tokensprint_amd.models.spec import LayerSpec, ModelSpec, PartSpec, Run
from tokensprint_amd.parts.attention import SoftmaxAttention

LOOP_TABLE = "loop.step"


def _delta_spec(m: DeltaSizes, pre: str, eps: float, state: str) -> PartSpec:
    return PartSpec("gated_delta", {
        "prefix": pre, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
        "conv": m.conv, "eps": eps, "per_channel": m.per_channel, "decay_rank": m.decay_rank,
        "gate_rank": m.gate_rank, "state": state})


def _mixer_spec(layer, pre: str, cfg: PalelixConfig, positions: dict) -> PartSpec:
    m = layer.mixer
    if isinstance(m, LightningSizes):
        return PartSpec("lightning_attention", {
            "prefix": pre, "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "decay": m.decay,
            "eps": cfg.eps, "state": "lightning"})
    if isinstance(m, DeltaSizes):
        return _delta_spec(m, pre, cfg.eps, "delta")
    left = m.left
    head = SoftmaxAttention.padded_head(left.dim, left.vdim)
    # one table per (base, rotated dimensions, head size), shared by the layers that use it
    name = f"rot_{left.rot_base!r}_{left.rot_dims}_{head}"
    positions.setdefault(name, PartSpec("rope_partial", {
        "dims": left.rot_dims, "base": left.rot_base, "head_dim": head,
        "max_position": cfg.max_position}))
    return PartSpec("side_by_side", {
        "left": PartSpec("softmax_attention", {
            "prefix": pre + "left.", "heads": left.heads, "kv_heads": left.kv_heads,
            "dim": left.dim, "vdim": left.vdim, "scale": left.scale, "position": name,
            "window": None}),
        "right": _delta_spec(m.right, pre + "right.", cfg.eps, "delta"),
        "left_scale": m.left_scale, "right_scale": m.right_scale})


def _ff_spec(mlp, pre: str) -> PartSpec | None:
    if mlp is None:
        return None
    if isinstance(mlp, DenseFF):
        return PartSpec("swiglu", {"prefix": pre, "inner_dim": mlp.ff,
                                   "names": ("gate", "up", "down")})
    return PartSpec("routed_experts", {
        "prefix": pre, "inner_dim": mlp.ff, "experts": mlp.experts, "top": mlp.top,
        "group_count": mlp.group_count, "group_keep": mlp.group_keep, "limit": mlp.limit})


def palelix_spec(cfg: PalelixConfig) -> ModelSpec:
    positions: dict[str, PartSpec] = {}
    layers = []
    for i, layer in enumerate(cfg.layers):
        pre = f"l{i}."
        layers.append(LayerSpec(
            "parallel_residual",
            mixer_norm=PartSpec("rmsnorm", {"dim": cfg.width, "eps": cfg.eps,
                                            "weight": pre + "norm1"}),
            mixer=_mixer_spec(layer, pre + "mix.", cfg, positions),
            feed_forward=_ff_spec(layer.mlp, pre + "mlp.")))
    start = cfg.loop.start if cfg.loop is not None else None
    order = tuple(Run(i, enter=(LOOP_TABLE, t) if t is not None and i == start else None)
                  for i, t in cfg.run_order())
    return ModelSpec(
        architecture=ARCHITECTURE, width=cfg.width, vocab_size=cfg.vocab_size,
        embedding=PartSpec("embedding", {"weight": "embed", "vocab_size": cfg.vocab_size}),
        positions=positions, layers=tuple(layers), order=order,
        final_norm=PartSpec("rmsnorm", {"dim": cfg.width, "eps": cfg.eps, "weight": "final.norm"}),
        head=PartSpec("head", {"weight": "head", "vocab_size": cfg.vocab_size}),
        max_position=cfg.max_position, eos_token_id=cfg.eos_token_id,
        enter_tables={LOOP_TABLE: cfg.loop.times} if cfg.loop is not None else {},
    )


register_architecture(ARCHITECTURE, parse_config=PalelixConfig.from_dict, build_spec=palelix_spec)
