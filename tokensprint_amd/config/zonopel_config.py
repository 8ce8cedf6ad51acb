"""Typed Zonopel configuration read from config.json.

A Zonopel model is a list of layers, each with a mixer (`mamba2` or `latent_attention`),
an optional dense feed-forward, norms before and after each sub-layer and a token shift
in front of the mixer; a layer may borrow another layer's weights (`weights_of`) while
keeping a cache or state of its own.  Every size and every constant that may differ
between two models is read here; nothing about them stands in code.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from tokensprint_amd.config.model_config import ConfigError

ARCHITECTURE = "Zonopel"
MIXER_TYPES = ("mamba2", "latent_attention")


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks '{key}'")
    return d[key]


def _pos_int(d: dict, key: str, where: str) -> int:
    v = _need(d, key, where)
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    return v


def _pos_float(d: dict, key: str, where: str) -> float:
    v = _need(d, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not v > 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class Mamba2Sizes:
    heads: int
    vdim: int            # channels per head
    state: int           # N: state rows per head
    groups: int          # B and C are shared by heads // groups heads
    conv: int            # taps of the short convolution
    norm_groups: int     # parts the gated output is normalised in

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def in_rows(self) -> int:
        return 2 * self.inner + 2 * self.groups * self.state + self.heads


@dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int             # unrotated query/key dimensions per head
    rot_dim: int         # rotated query/key dimensions per head (the key's are shared)
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int        # leading dimensions of the rotated part that are rotated
    window: int | None   # a query sees itself and the window - 1 tokens before it


@dataclass(frozen=True)
class ZonopelLayer:
    type: str
    mixer: Mamba2Sizes | LatentAttentionSizes
    ff: int | None                # feed-forward inner size, None: the layer has none
    weights_of: int | None        # the layer whose tensors this one uses, None: its own


@dataclass(frozen=True)
class ZonopelConfig:
    width: int
    vocab_size: int
    eps: float
    embed_scale: float
    bigram_buckets: int
    bigram_mul_prev: int
    bigram_mul_cur: int
    layers: tuple[ZonopelLayer, ...]
    eos_token_id: int | None = None
    max_position: int = 1 << 20
    architecture: str = ARCHITECTURE
    raw: dict = field(default_factory=dict, compare=False, repr=False)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "ZonopelConfig":
        width = _pos_int(raw, "width", "config")
        vocab = _pos_int(raw, "vocab", "config")
        eps = _pos_float(_need(raw, "norm", "config"), "eps", "norm")
        emb = _need(raw, "embedding", "config")
        bigram = _need(emb, "bigram", "embedding")
        entries = _need(raw, "layers", "config")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(entry, "type", where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type={kind!r}; Zonopel has "
                                  f"{', '.join(MIXER_TYPES)}")
            m = _need(entry, "mixer", where)
            if kind == "mamba2":
                mixer = cls._mamba2(m, where + ".mixer")
            else:
                mixer = cls._latent(m, where + ".mixer")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp.kind={mlp.get('kind')!r}; "
                                      "only 'dense' is built")
                ff = _pos_int(mlp, "ff", where + ".mlp")
            src = entry.get("weights_of")
            if src is not None and (not isinstance(src, int) or isinstance(src, bool)
                                    or not 0 <= src < len(entries) or src == i):
                raise ConfigError(f"config.json: {where}.weights_of={src!r} names no other layer")
            layers.append(ZonopelLayer(kind, mixer, ff, src))
        for i, layer in enumerate(layers):
            if layer.weights_of is not None:
                src = layers[layer.weights_of]
                if src.weights_of is not None:
                    raise ConfigError(f"config.json: layers[{i}] borrows from layers"
                                      f"[{layer.weights_of}], which has no tensors of its own")
                if (src.type, src.mixer, src.ff) != (layer.type, layer.mixer, layer.ff):
                    raise ConfigError(f"config.json: layers[{i}] borrows the weights of layers"
                                      f"[{layer.weights_of}] but differs from it")
        eos = raw.get("eos_token_id")
        # positions have no table to run out of; the bound keeps float32 angles exact in the
        # position and is what an engine is told when nobody gives it a length
        max_pos = raw.get("max_position", 1 << 20)
        return cls(width=width, vocab_size=vocab, eps=eps,
                   embed_scale=float(_need(emb, "scale", "embedding")),
                   bigram_buckets=_pos_int(bigram, "buckets", "embedding.bigram"),
                   bigram_mul_prev=int(_need(bigram, "mul_prev", "embedding.bigram")),
                   bigram_mul_cur=int(_need(bigram, "mul_cur", "embedding.bigram")),
                   layers=tuple(layers), eos_token_id=eos, max_position=int(max_pos),
                   raw=dict(raw))

    @staticmethod
    def _mamba2(m, where) -> Mamba2Sizes:
        s = Mamba2Sizes(heads=_pos_int(m, "heads", where), vdim=_pos_int(m, "vdim", where),
                        state=_pos_int(m, "state", where), groups=_pos_int(m, "groups", where),
                        conv=_pos_int(m, "conv", where),
                        norm_groups=_pos_int(m, "norm_groups", where))
        if s.heads % s.groups:
            raise ConfigError(f"config.json: {where}: heads={s.heads} is not a multiple of "
                              f"groups={s.groups}")
        if s.inner % s.norm_groups:
            raise ConfigError(f"config.json: {where}: heads*vdim={s.inner} is not a multiple "
                              f"of norm_groups={s.norm_groups}")
        return s

    @staticmethod
    def _latent(m, where) -> LatentAttentionSizes:
        rot = _need(m, "rot", where)
        mask = m.get("mask")
        window = None if not mask else _pos_int(mask, "size", where + ".mask")
        s = LatentAttentionSizes(
            heads=_pos_int(m, "heads", where), dim=_pos_int(m, "dim", where),
            rot_dim=_pos_int(m, "rot_dim", where), vdim=_pos_int(m, "vdim", where),
            q_rank=_pos_int(m, "q_rank", where), kv_rank=_pos_int(m, "kv_rank", where),
            scale=_pos_float(m, "scale", where), rot_base=_pos_float(rot, "base", where + ".rot"),
            rot_dims=_pos_int(rot, "dims", where + ".rot"), window=window)
        if s.rot_dims % 2 or s.rot_dims > s.rot_dim:
            raise ConfigError(f"config.json: {where}.rot.dims={s.rot_dims} must be even and at "
                              f"most rot_dim={s.rot_dim}")
        return s
