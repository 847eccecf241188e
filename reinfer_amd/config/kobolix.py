"""Kobolix: typed configuration from its config.json.

A decoder of pre-norm layers whose addends enter the residual stream times a constant. A layer's mixer is a
matrix memory with exponential gates ("mlstm") or two mixers side by side on one input ("parallel":
grouped-query attention with rotated pairs and a value size of its own, and a gated delta rule with a short
causal filter); its feed-forward is a gated dense one, a mixture of gated experts with a sigmoid router that
is restricted to the best groups of experts and a shared expert, or absent. Norm weights are stored around
zero; the embedding is scaled on its way in and is the head as it is.

config.json nests its keys: ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``embedding.scale`` and
``layers[i]`` with ``type``, ``mixer`` and ``mlp``. Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.*`` (``.left.*`` / ``.right.*`` in a parallel layer), ``l<i>.mlp.*``, ``final.norm``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple, Union

from .puresun import _At, _section
from .schema import (BlockSpec, ConfigError, DeltaRuleSpec, FeedForwardSpec, MatrixMemorySpec, MixerSpec, ModelSpec,
                     MoESpec, NormSpec, PositionSpec, RunEntry, SideBySideSpec, read_float, read_int)

ARCHITECTURE = "Kobolix"

# config.json gives no context limit; the engine's own (block tables and captured steps are sized by it)
DEFAULT_MAX_POSITIONS = 1 << 16

# constants the design fixes
NORM_WEIGHT_OFFSET = 1.0        # a norm's factor is 1 + w
MEMORY_DENOM_EPS = 1e-6         # added to the matrix memory's denominator
UNIT_NORM_EPS = 1e-6            # inside the root of the delta rule's unit norms
GROUP_SCORE_TOP = 2             # a group of experts is scored by the sum of this many of its scores


@dataclass(frozen=True)
class KobolixMemoryMixer:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class KobolixAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int


@dataclass(frozen=True)
class KobolixDeltaRule:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class KobolixPair:
    left: KobolixAttention
    right: KobolixDeltaRule


@dataclass(frozen=True)
class KobolixDense:
    ff: int


@dataclass(frozen=True)
class KobolixMoE:
    experts: int
    top: int
    ff: int
    scale: float
    groups: int
    keep: int
    shared_ff: int          # 0: no shared expert


@dataclass(frozen=True)
class KobolixLayer:
    kind: str                                   # "mlstm" or "parallel"
    mixer: Union[KobolixMemoryMixer, KobolixPair]
    mlp: Union[KobolixDense, KobolixMoE, None]


@dataclass(frozen=True)
class KobolixConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    embedding_scale: float
    layers: Tuple[KobolixLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS
    architecture: str = ARCHITECTURE

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any]) -> "KobolixConfig":
        vocab = read_int(cfg, "vocab", minimum=1)
        width = read_int(cfg, "width", minimum=1)
        eps = _At(_section(cfg, "norm"), "norm.").float("eps")
        if eps < 0.0:
            raise ConfigError("norm.eps", "must be >= 0")
        mult = read_float(cfg, "residual_mult", 1.0)
        emb = _section(cfg, "embedding", required=False)
        emb_scale = _At(emb, "embedding.").float("scale", 1.0) if emb is not None else 1.0
        raw_layers = cfg.get("layers", None)
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("layers", "expected a non-empty list of layers")
        layers = tuple(cls._read_layer(L, f"layers[{i}].") for i, L in enumerate(raw_layers))
        max_pos = read_int(cfg, "max_positions", DEFAULT_MAX_POSITIONS, minimum=1)
        return cls(vocab=vocab, width=width, norm_eps=eps, residual_mult=mult, embedding_scale=emb_scale,
                   layers=layers, max_positions=max_pos)

    @staticmethod
    def _read_memory(m: Mapping[str, Any], where: str) -> KobolixMemoryMixer:
        at = _At(m, where)
        cap = at.float("gate_cap", 0.0)                  # absent: the gates are not capped
        if cap < 0.0:
            raise ConfigError(where + "gate_cap", "must be > 0 (absent: no cap)")
        return KobolixMemoryMixer(heads=at.int("heads", minimum=1), dim=at.int("dim", minimum=1),
                                  vdim=at.int("vdim", minimum=1), gate_cap=cap)

    @staticmethod
    def _read_attention(m: Mapping[str, Any], where: str) -> KobolixAttention:
        at = _At(m, where)
        heads, kv = at.int("heads", minimum=1), at.int("kv_heads", minimum=1)
        if heads % kv:
            raise ConfigError(where + "kv_heads", f"{heads} query heads do not divide into {kv} groups")
        dim = at.int("dim", minimum=1)
        rot = _section(m, "rot", where, required=False)
        base, dims = 10000.0, 0
        if rot is not None:
            rat = _At(rot, where + "rot.")
            base, dims = rat.float("base"), rat.int("dims", minimum=0)
            if base <= 0.0:
                raise ConfigError(where + "rot.base", "must be > 0")
            if dims % 2 or dims > dim:
                raise ConfigError(where + "rot.dims", f"{dims} entries in pairs out of {dim}")
        return KobolixAttention(heads=heads, kv_heads=kv, dim=dim, vdim=at.int("vdim", minimum=1),
                                scale=at.float("scale", float(dim) ** -0.5), rot_base=base, rot_dims=dims)

    @staticmethod
    def _read_delta(m: Mapping[str, Any], where: str) -> KobolixDeltaRule:
        at = _At(m, where)
        heads, kv = at.int("heads", minimum=1), at.int("kv_heads", minimum=1)
        if heads % kv:
            raise ConfigError(where + "kv_heads", f"{heads} heads do not divide into {kv} key heads")
        return KobolixDeltaRule(heads=heads, kv_heads=kv, dim=at.int("dim", minimum=1),
                                vdim=at.int("vdim", minimum=1), conv=at.int("conv", minimum=1))

    @classmethod
    def _read_layer(cls, L: Any, where: str) -> KobolixLayer:
        if not isinstance(L, dict):
            raise ConfigError(where.rstrip("."), f"expected an object, got {L!r}")
        kind = L.get("type", None)
        m = _section(L, "mixer", where)
        if kind == "mlstm":
            mixer: Any = cls._read_memory(m, where + "mixer.")
        elif kind == "parallel":
            mixer = KobolixPair(left=cls._read_attention(_section(m, "left", where + "mixer."), where + "mixer.left."),
                                right=cls._read_delta(_section(m, "right", where + "mixer."), where + "mixer.right."))
        else:
            raise ConfigError(where + "type", f"unknown mixer {kind!r}; this design has 'mlstm' and 'parallel'")
        mlp: Any = None
        f = L.get("mlp", None)
        if f is not None:
            if not isinstance(f, dict):
                raise ConfigError(where + "mlp", f"expected an object or null, got {f!r}")
            fk = f.get("kind", None)
            if fk == "dense":
                mlp = KobolixDense(ff=_At(f, where + "mlp.").int("ff", minimum=1))
            elif fk == "moe":
                rsec = _section(f, "router", where + "mlp.")
                router = _At(rsec, where + "mlp.router.")
                experts, top = router.int("experts", minimum=1), router.int("top", minimum=1)
                groups, keep = 1, 1
                gsec = _section(rsec, "groups", where + "mlp.router.", required=False)
                if gsec is not None:
                    gat = _At(gsec, where + "mlp.router.groups.")
                    groups, keep = gat.int("count", minimum=1), gat.int("keep", minimum=1)
                if experts % groups:
                    raise ConfigError(where + "mlp.router.groups.count", f"{experts} experts in {groups} equal groups")
                if keep > groups:
                    raise ConfigError(where + "mlp.router.groups.keep", f"{keep} of {groups} groups")
                if top > keep * (experts // groups):
                    raise ConfigError(where + "mlp.router.top", f"{top} of the {keep * (experts // groups)} experts "
                                                                "that can be chosen")
                ff = _At(_section(f, "expert", where + "mlp."), where + "mlp.expert.").int("ff", minimum=1)
                ssec = _section(f, "shared", where + "mlp.", required=False)
                shared = _At(ssec, where + "mlp.shared.").int("ff", minimum=1) if ssec is not None else 0
                mlp = KobolixMoE(experts=experts, top=top, ff=ff, scale=router.float("scale", 1.0), groups=groups,
                                 keep=keep, shared_ff=shared)
            else:
                raise ConfigError(where + "mlp.kind", f"unknown feed-forward {fk!r}; this design has 'dense' and 'moe'")
        return KobolixLayer(kind=kind, mixer=mixer, mlp=mlp)

    # ---------------------------------------------------------------- writing
    def to_dict(self) -> Dict[str, Any]:
        layers: List[Dict[str, Any]] = []
        for L in self.layers:
            if L.kind == "mlstm":
                m = L.mixer
                mixer: Dict[str, Any] = {"dim": m.dim, "heads": m.heads, "vdim": m.vdim}
                if m.gate_cap:
                    mixer["gate_cap"] = m.gate_cap
            else:
                a, d = L.mixer.left, L.mixer.right
                left: Dict[str, Any] = {"dim": a.dim, "heads": a.heads, "kv_heads": a.kv_heads, "scale": a.scale,
                                        "vdim": a.vdim}
                if a.rot_dims:
                    left["rot"] = {"base": a.rot_base, "dims": a.rot_dims}
                mixer = {"left": left,
                         "right": {"conv": d.conv, "dim": d.dim, "heads": d.heads, "kv_heads": d.kv_heads,
                                   "vdim": d.vdim}}
            mlp: Any = None
            if isinstance(L.mlp, KobolixDense):
                mlp = {"ff": L.mlp.ff, "kind": "dense"}
            elif isinstance(L.mlp, KobolixMoE):
                f = L.mlp
                mlp = {"expert": {"ff": f.ff}, "kind": "moe",
                       "router": {"experts": f.experts, "groups": {"count": f.groups, "keep": f.keep},
                                  "scale": f.scale, "top": f.top}}
                if f.shared_ff:
                    mlp["shared"] = {"ff": f.shared_ff}
            layers.append({"mixer": mixer, "mlp": mlp, "type": L.kind})
        d: Dict[str, Any] = {"architecture": ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
                             "layers": layers, "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
                             "vocab": self.vocab, "width": self.width}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        return d

    # ---------------------------------------------------------------- the model
    def _mixer_spec(self, L: KobolixLayer) -> MixerSpec:
        if L.kind == "mlstm":
            m = L.mixer
            return MixerSpec(kind="matrix_memory", hidden=self.width,
                             params=MatrixMemorySpec(heads=m.heads, key_dim=m.dim, value_dim=m.vdim,
                                                     gate_cap=m.gate_cap, norm_eps=self.norm_eps,
                                                     denom_eps=MEMORY_DENOM_EPS))
        a, d = L.mixer.left, L.mixer.right
        left = MixerSpec(kind="gqa_attention", hidden=self.width, num_heads=a.heads, num_kv_heads=a.kv_heads,
                         head_dim=a.dim, value_dim=a.vdim, scale=a.scale,
                         position=PositionSpec("rope_interleaved", rotary_dim=a.rot_dims, theta=a.rot_base)
                         if a.rot_dims else PositionSpec("none"),
                         extra=(("names", ("q", "k", "v", "o")),))
        right = MixerSpec(kind="gated_delta_rule", hidden=self.width,
                          params=DeltaRuleSpec(heads=d.heads, key_heads=d.kv_heads, key_dim=d.dim, value_dim=d.vdim,
                                               conv_taps=d.conv, norm_eps=self.norm_eps, unit_eps=UNIT_NORM_EPS))
        return MixerSpec(kind="side_by_side", hidden=self.width,
                         params=SideBySideSpec(members=(("left.", left), ("right.", right)), norm_eps=self.norm_eps,
                                               out_name="out"))

    def _ffn_spec(self, f) -> Optional[FeedForwardSpec]:
        if f is None:
            return None
        if isinstance(f, KobolixDense):
            return FeedForwardSpec(kind="swiglu", hidden=self.width, intermediate=f.ff,
                                   extra=(("names", ("gate", "up", "down")),))
        return FeedForwardSpec(kind="moe", hidden=self.width, intermediate=f.ff,
                               params=MoESpec(experts=f.experts, top=f.top, activation="silu_gated", weights="sigmoid",
                                              weight_scale=f.scale, groups=f.groups, groups_kept=f.keep,
                                              group_top=GROUP_SCORE_TOP, shared=f.shared_ff))

    def to_spec(self) -> ModelSpec:
        norm = NormSpec("rmsnorm", self.width, self.norm_eps, offset=NORM_WEIGHT_OFFSET)
        blocks: List[BlockSpec] = []
        for i, L in enumerate(self.layers):
            ffn = self._ffn_spec(L.mlp)
            blocks.append(BlockSpec(kind="prenorm", mixer=self._mixer_spec(L), ffn=ffn, mixer_norm=norm,
                                    ffn_norm=norm if ffn is not None else None, prefix=f"l{i}.",
                                    mixer_prefix="mix.", ffn_prefix="mlp.", mixer_norm_name="norm1",
                                    ffn_norm_name="norm2", residual_scale=self.residual_mult))
        return ModelSpec(
            architecture=ARCHITECTURE, vocab_size=self.vocab, hidden=self.width, max_positions=self.max_positions,
            blocks=tuple(blocks), run_order=tuple(RunEntry(i) for i in range(len(blocks))), final_norm=norm,
            tie_embeddings=True, embed_name="embed", final_norm_name="final.norm", head_name="head",
            embed_scale=self.embedding_scale)
