"""Typed Palelix configuration read from config.json.

A Palelix model is a list of parallel layers (one norm, a mixer and a feed-forward that both
read it), of which a stretch may run several times in a row with the same weights (`loop`),
each pass with a cache or state of its own.  Mixers: `lightning` (linear attention with a
fixed decay per head), `delta` (gated delta rule, one decay per head and token) and
`parallel` (softmax attention beside a gated delta rule with a decay per key channel).
Feed-forwards: dense SwiGLU, or routed experts chosen among the best groups.  Every size and
every constant that may differ between two models is read here.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from tokensprint_amd.config.model_config import ConfigError

ARCHITECTURE = "Palelix"
MIXER_TYPES = ("lightning", "delta", "parallel")


def _need(d, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks '{key}'")
    return d[key]


def _pos_int(d, key: str, where: str) -> int:
    v = _need(d, key, where)
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    return v


def _number(d, key: str, where: str, positive: bool = False) -> float:
    v = _need(d, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0):
        raise ConfigError(f"config.json: {where}.{key} must be a "
                          f"{'positive ' if positive else ''}number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class LightningSizes:
    heads: int
    dim: int                     # query/key size per head
    vdim: int
    decay: tuple[float, ...]     # one per head


@dataclass(frozen=True)
class DeltaSizes:
    heads: int                   # value heads
    kv_heads: int                # query/key heads
    dim: int
    vdim: int
    conv: int                    # taps of the short convolutions
    per_channel: bool            # a decay per key channel (low-rank projection) or per head
    decay_rank: int | None = None   # inner sizes of the two-step projections; None: what the
    gate_rank: int | None = None    # file's tensors have (random weights need them named)


@dataclass(frozen=True)
class SoftmaxSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int


@dataclass(frozen=True)
class ParallelSizes:
    left: SoftmaxSizes
    right: DeltaSizes
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class DenseFF:
    ff: int


@dataclass(frozen=True)
class RoutedFF:
    ff: int                      # inner size of one expert
    limit: float
    experts: int
    top: int
    group_count: int
    group_keep: int


@dataclass(frozen=True)
class PalelixLayer:
    type: str
    mixer: LightningSizes | DeltaSizes | ParallelSizes
    mlp: DenseFF | RoutedFF | None


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class PalelixConfig:
    width: int
    vocab_size: int
    eps: float
    layers: tuple[PalelixLayer, ...]
    loop: Loop | None = None
    eos_token_id: int | None = None
    max_position: int = 1 << 17
    architecture: str = ARCHITECTURE
    raw: dict = field(default_factory=dict, compare=False, repr=False)

    def run_order(self) -> list[tuple[int, int | None]]:
        """(layer, pass number or None) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        lp = self.loop
        order = [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, t) for i in range(lp.start, lp.stop)]
        return order + [(i, None) for i in range(lp.stop, n)]

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "PalelixConfig":
        width = _pos_int(raw, "width", "config")
        vocab = _pos_int(raw, "vocab", "config")
        eps = _number(_need(raw, "norm", "config"), "eps", "norm", positive=True)
        entries = _need(raw, "layers", "config")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(entry, "type", where)
            m = _need(entry, "mixer", where)
            if kind == "lightning":
                mixer = cls._lightning(m, where + ".mixer")
            elif kind == "delta":
                mixer = cls._delta(m, where + ".mixer", per_channel=False)
            elif kind == "parallel":
                mixer = ParallelSizes(
                    left=cls._softmax(_need(m, "left", where + ".mixer"), where + ".mixer.left"),
                    right=cls._delta(_need(m, "right", where + ".mixer"), where + ".mixer.right",
                                     per_channel=True),
                    left_scale=_number(m, "left_scale", where + ".mixer"),
                    right_scale=_number(m, "right_scale", where + ".mixer"))
            else:
                raise ConfigError(f"config.json: {where}.type={kind!r}; Palelix has "
                                  f"{', '.join(MIXER_TYPES)}")
            layers.append(PalelixLayer(kind, mixer, cls._mlp(entry.get("mlp"), where + ".mlp")))
        loop = None
        lp = raw.get("loop")
        if lp is not None:
            loop = Loop(start=int(_need(lp, "start", "loop")), stop=int(_need(lp, "stop", "loop")),
                        times=_pos_int(lp, "times", "loop"))
            if not 0 <= loop.start < loop.stop <= len(layers):
                raise ConfigError(f"config.json: loop [{loop.start}, {loop.stop}) does not lie "
                                  f"inside the {len(layers)} layers")
        return cls(width=width, vocab_size=vocab, eps=eps, layers=tuple(layers), loop=loop,
                   eos_token_id=raw.get("eos_token_id"),
                   max_position=int(raw.get("max_position", 1 << 17)), raw=dict(raw))

    @staticmethod
    def _lightning(m, where) -> LightningSizes:
        heads = _pos_int(m, "heads", where)
        decay = _need(m, "decay", where)
        if not isinstance(decay, list) or len(decay) != heads:
            raise ConfigError(f"config.json: {where}.decay must list one number per head")
        return LightningSizes(heads=heads, dim=_pos_int(m, "dim", where),
                              vdim=_pos_int(m, "vdim", where),
                              decay=tuple(float(d) for d in decay))

    @staticmethod
    def _delta(m, where, per_channel: bool) -> DeltaSizes:
        s = DeltaSizes(heads=_pos_int(m, "heads", where), kv_heads=_pos_int(m, "kv_heads", where),
                       dim=_pos_int(m, "dim", where), vdim=_pos_int(m, "vdim", where),
                       conv=_pos_int(m, "conv", where), per_channel=per_channel,
                       decay_rank=m.get("decay_rank"), gate_rank=m.get("gate_rank"))
        if s.heads % s.kv_heads:
            raise ConfigError(f"config.json: {where}: heads={s.heads} is not a multiple of "
                              f"kv_heads={s.kv_heads}")
        return s

    @staticmethod
    def _softmax(m, where) -> SoftmaxSizes:
        rot = _need(m, "rot", where)
        s = SoftmaxSizes(heads=_pos_int(m, "heads", where), kv_heads=_pos_int(m, "kv_heads", where),
                         dim=_pos_int(m, "dim", where), vdim=_pos_int(m, "vdim", where),
                         scale=_number(m, "scale", where, positive=True),
                         rot_base=_number(rot, "base", where + ".rot", positive=True),
                         rot_dims=_pos_int(rot, "dims", where + ".rot"))
        if s.heads % s.kv_heads:
            raise ConfigError(f"config.json: {where}: heads={s.heads} is not a multiple of "
                              f"kv_heads={s.kv_heads}")
        if s.rot_dims % 2 or s.rot_dims > s.dim:
            raise ConfigError(f"config.json: {where}.rot.dims={s.rot_dims} must be even and at "
                              f"most dim={s.dim}")
        return s

    @staticmethod
    def _mlp(mlp, where):
        if mlp is None:
            return None
        kind = _need(mlp, "kind", where)
        if kind == "dense":
            return DenseFF(ff=_pos_int(mlp, "ff", where))
        if kind != "moe":
            raise ConfigError(f"config.json: {where}.kind={kind!r}; Palelix has dense and moe")
        ex, r = _need(mlp, "expert", where), _need(mlp, "router", where)
        groups = r.get("groups") or {"count": 1, "keep": 1}
        f = RoutedFF(ff=_pos_int(ex, "ff", where + ".expert"),
                     limit=_number(ex, "limit", where + ".expert", positive=True),
                     experts=_pos_int(r, "experts", where + ".router"),
                     top=_pos_int(r, "top", where + ".router"),
                     group_count=_pos_int(groups, "count", where + ".router.groups"),
                     group_keep=_pos_int(groups, "keep", where + ".router.groups"))
        if f.experts % f.group_count or f.group_keep > f.group_count \
                or f.top > f.group_keep * (f.experts // f.group_count):
            raise ConfigError(f"config.json: {where}.router: {f.experts} experts in "
                              f"{f.group_count} groups, {f.group_keep} kept, cannot give {f.top}")
        return f
