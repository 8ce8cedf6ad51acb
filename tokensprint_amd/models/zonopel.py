"""Zonopel as a `ModelSpec`: a bigram-hashed embedding, layers that sandwich a mixer
(Mamba-2 or latent attention behind a token shift) and a PolyNorm feed-forward between
norms, shared weights between layers as repeated runs of one layer.

Tensor names: 'embed', 'bigram', 'embed.norm', 'final.norm', 'head', and per layer i
'l<i>.norm1|norm1b|norm2|norm2b|shift', 'l<i>.mix.*', 'l<i>.mlp.*'.
"""

from __future__ import annotations

from tokensprint_amd.config.registry import register_architecture
from tokensprint_amd.config.zonopel_config import (ARCHITECTURE, LatentAttentionSizes,
                                                   ZonopelConfig)
from tokensprint_amd.models.spec import LayerSpec, ModelSpec, PartSpec, Run


def _mixer_spec(layer, pre: str, eps: float, positions: dict) -> PartSpec:
    m = layer.mixer
    if isinstance(m, LatentAttentionSizes):
        # one rotation per (base, dims), shared by the layers that use it
        name = f"rot_{m.rot_base!r}_{m.rot_dims}"
        positions.setdefault(name, PartSpec("rope_interleaved",
                                            {"dims": m.rot_dims, "base": m.rot_base}))
        return PartSpec("latent_attention", {
            "prefix": pre + "mix.", "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
            "vdim": m.vdim, "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale,
            "eps": eps, "window": m.window, "position": name})
    return PartSpec("mamba2", {
        "prefix": pre + "mix.", "heads": m.heads, "vdim": m.vdim, "state": m.state,
        "groups": m.groups, "conv": m.conv, "norm_groups": m.norm_groups, "eps": eps})


def zonopel_spec(cfg: ZonopelConfig) -> ModelSpec:
    positions: dict[str, PartSpec] = {}
    layers, layer_of = [], {}

    def norm(name):
        return PartSpec("rmsnorm", {"dim": cfg.width, "eps": cfg.eps, "weight": name})

    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        pre = f"l{i}."
        parts = dict(
            mixer_norm=norm(pre + "norm1"),
            mixer_filter=PartSpec("token_shift", {"weight": pre + "shift", "dim": cfg.width}),
            mixer=_mixer_spec(layer, pre, cfg.eps, positions),
            mixer_post_norm=norm(pre + "norm1b"))
        if layer.ff is not None:
            parts.update(
                ffn_norm=norm(pre + "norm2"),
                feed_forward=PartSpec("polynorm_mlp", {"prefix": pre + "mlp.",
                                                       "inner_dim": layer.ff, "eps": cfg.eps}),
                ffn_post_norm=norm(pre + "norm2b"))
        layer_of[i] = len(layers)
        layers.append(LayerSpec("sandwich_norm", **parts))
    order = tuple(Run(layer_of[i if layer.weights_of is None else layer.weights_of])
                  for i, layer in enumerate(cfg.layers))
    return ModelSpec(
        architecture=ARCHITECTURE, width=cfg.width, vocab_size=cfg.vocab_size,
        embedding=PartSpec("bigram_embedding", {
            "weight": "embed", "bigram": "bigram", "norm": "embed.norm",
            "vocab_size": cfg.vocab_size, "scale": cfg.embed_scale, "eps": cfg.eps,
            "buckets": cfg.bigram_buckets, "mul_prev": cfg.bigram_mul_prev,
            "mul_cur": cfg.bigram_mul_cur}),
        positions=positions, layers=tuple(layers), order=order,
        final_norm=norm("final.norm"),
        head=PartSpec("head", {"weight": "head", "vocab_size": cfg.vocab_size}),
        max_position=cfg.max_position, eos_token_id=cfg.eos_token_id,
    )


register_architecture(ARCHITECTURE, parse_config=ZonopelConfig.from_dict, build_spec=zonopel_spec)
