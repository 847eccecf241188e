"""Puresun: typed configuration from its config.json.

A decoder of parallel layers (one norm, mixer and feed-forward side by side) whose mixers attend over a
cached low-rank latent inside a sliding window, with mixture-of-experts feed-forwards, a hashed token-pair
table added to the embedding, a run of layers that is repeated with the embedding fed in again, and capped
logits. config.json nests its keys: ``vocab``, ``width``, ``norm.eps``, ``logit_softcap``,
``embedding.bigram.{buckets, mul_prev, mul_cur}``, ``loop.{start, stop, times}`` and ``layers[i]`` with
``type``, ``mixer`` and ``mlp``. Tensor names: ``embed``, ``bigram``, ``loop.step``, ``l<i>.norm1``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .schema import (BlockSpec, ConfigError, FeedForwardSpec, InputSpec, LatentAttentionSpec, MixerSpec,
                     ModelSpec, MoESpec, NormSpec, PairHashSpec, PositionSpec, RunEntry, StreamAdd, read_float,
                     read_int)

ARCHITECTURE = "Puresun"

# config.json gives no context limit; the engine's own (block tables and captured steps are sized by it)
DEFAULT_MAX_POSITIONS = 1 << 16


def _section(cfg: Mapping[str, Any], key: str, where: str = "", required: bool = True) -> Optional[Mapping[str, Any]]:
    v = cfg.get(key, None)
    if v is None:
        if required:
            raise ConfigError(where + key, "required key is missing")
        return None
    if not isinstance(v, dict):
        raise ConfigError(where + key, f"expected an object, got {v!r}")
    return v


class _At:
    """A mapping whose key readers name the full path in their errors."""

    def __init__(self, cfg: Mapping[str, Any], where: str):
        self.cfg, self.where = cfg, where

    def _rename(self, fn, key, *a, **kw):
        try:
            return fn(self.cfg, key, *a, **kw)
        except ConfigError as e:
            raise ConfigError(self.where + e.key, e.why) from None

    def int(self, key, *a, **kw):
        return self._rename(read_int, key, *a, **kw)

    def float(self, key, *a, **kw):
        return self._rename(read_float, key, *a, **kw)


@dataclass(frozen=True)
class PuresunLatentMixer:
    heads: int
    dim: int            # unrotated query/key entries a head
    rot_dim: int        # rotated query/key entries a head (one key part shared by all heads)
    vdim: int
    kv_rank: int
    scale: float
    window: int         # 0: every earlier key
    rot_base: float
    rot_dims: int       # entries of the rotated part that are turned


@dataclass(frozen=True)
class PuresunMoE:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class PuresunLayer:
    mixer: PuresunLatentMixer
    mlp: Optional[PuresunMoE]


@dataclass(frozen=True)
class PuresunConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[PuresunLayer, ...]
    logit_softcap: float = 0.0
    bigram: Optional[Tuple[int, int, int]] = None          # buckets, mul_prev, mul_cur
    loop: Optional[Tuple[int, int, int]] = None            # start, stop, times
    max_positions: int = DEFAULT_MAX_POSITIONS
    architecture: str = ARCHITECTURE

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any]) -> "PuresunConfig":
        vocab = read_int(cfg, "vocab", minimum=1)
        width = read_int(cfg, "width", minimum=1)
        eps = _At(_section(cfg, "norm"), "norm.").float("eps")
        if eps < 0.0:
            raise ConfigError("norm.eps", "must be >= 0")
        cap = read_float(cfg, "logit_softcap", 0.0)
        if cap < 0.0:
            raise ConfigError("logit_softcap", "must be >= 0 (0: no cap)")
        bigram = None
        emb = _section(cfg, "embedding", required=False)
        big = _section(emb, "bigram", "embedding.", required=False) if emb is not None else None
        if big is not None:
            at = _At(big, "embedding.bigram.")
            bigram = (at.int("buckets", minimum=1), at.int("mul_prev", minimum=0), at.int("mul_cur", minimum=0))
        raw_layers = cfg.get("layers", None)
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("layers", "expected a non-empty list of layers")
        layers = tuple(cls._read_layer(L, f"layers[{i}].") for i, L in enumerate(raw_layers))
        loop = None
        lp = _section(cfg, "loop", required=False)
        if lp is not None:
            at = _At(lp, "loop.")
            start, stop, times = at.int("start", minimum=0), at.int("stop", minimum=0), at.int("times", minimum=1)
            if not start < stop <= len(layers):
                raise ConfigError("loop", f"layers {start}..{stop - 1} of {len(layers)}")
            loop = (start, stop, times)
        max_pos = read_int(cfg, "max_positions", DEFAULT_MAX_POSITIONS, minimum=1)
        return cls(vocab=vocab, width=width, norm_eps=eps, layers=layers, logit_softcap=cap, bigram=bigram,
                   loop=loop, max_positions=max_pos)

    @staticmethod
    def _read_layer(L: Any, where: str) -> PuresunLayer:
        if not isinstance(L, dict):
            raise ConfigError(where.rstrip("."), f"expected an object, got {L!r}")
        kind = L.get("type", None)
        if kind != "latent_attention":
            raise ConfigError(where + "type", f"unknown mixer {kind!r}; this design has 'latent_attention'")
        m = _section(L, "mixer", where)
        at = _At(m, where + "mixer.")
        heads, dim = at.int("heads", minimum=1), at.int("dim", minimum=0)
        rot_dim, vdim = at.int("rot_dim", minimum=0), at.int("vdim", minimum=1)
        rank = at.int("kv_rank", minimum=1)
        if dim + rot_dim == 0:
            raise ConfigError(where + "mixer.dim", "a head needs at least one query/key entry")
        scale = at.float("scale")
        mask = _section(m, "mask", where + "mixer.", required=False)
        window = _At(mask, where + "mixer.mask.").int("size", minimum=1) if mask is not None else 0
        rot = _section(m, "rot", where + "mixer.", required=rot_dim > 0)
        base, dims = 10000.0, 0
        if rot is not None:
            rat = _At(rot, where + "mixer.rot.")
            base, dims = rat.float("base"), rat.int("dims", rot_dim, minimum=0)
            if base <= 0.0:
                raise ConfigError(where + "mixer.rot.base", "must be > 0")
            if dims % 2 or dims > rot_dim:
                raise ConfigError(where + "mixer.rot.dims", f"{dims} entries in pairs out of {rot_dim}")
        mixer = PuresunLatentMixer(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank, scale=scale,
                                   window=window, rot_base=base, rot_dims=dims)
        mlp = None
        f = L.get("mlp", None)
        if f is not None:
            if not isinstance(f, dict):
                raise ConfigError(where + "mlp", f"expected an object or null, got {f!r}")
            if f.get("kind", "moe") != "moe":
                raise ConfigError(where + "mlp.kind", f"unknown feed-forward {f.get('kind')!r}; this design has 'moe'")
            router = _At(_section(f, "router", where + "mlp."), where + "mlp.router.")
            experts = router.int("experts", minimum=1)
            top = router.int("top", minimum=1)
            if top > experts:
                raise ConfigError(where + "mlp.router.top", f"{top} of {experts} experts")
            ff = _At(_section(f, "expert", where + "mlp."), where + "mlp.expert.").int("ff", minimum=1)
            mlp = PuresunMoE(experts=experts, top=top, ff=ff)
        return PuresunLayer(mixer=mixer, mlp=mlp)

    # ---------------------------------------------------------------- writing
    def to_dict(self) -> Dict[str, Any]:
        layers: List[Dict[str, Any]] = []
        for L in self.layers:
            m = L.mixer
            mixer: Dict[str, Any] = {"dim": m.dim, "heads": m.heads, "kv_rank": m.kv_rank, "rot_dim": m.rot_dim,
                                     "scale": m.scale, "vdim": m.vdim,
                                     "rot": {"base": m.rot_base, "dims": m.rot_dims}}
            if m.window:
                mixer["mask"] = {"size": m.window}
            mlp = None
            if L.mlp is not None:
                mlp = {"kind": "moe", "expert": {"ff": L.mlp.ff},
                       "router": {"experts": L.mlp.experts, "top": L.mlp.top}}
            layers.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
        d: Dict[str, Any] = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width,
                             "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        if self.bigram is not None:
            d["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))}
        if self.loop is not None:
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        return d

    # ---------------------------------------------------------------- the model
    def to_spec(self) -> ModelSpec:
        norm = NormSpec("rmsnorm", self.width, self.norm_eps)
        blocks: List[BlockSpec] = []
        for i, L in enumerate(self.layers):
            m = L.mixer
            mixer = MixerSpec(
                kind="latent_attention", hidden=self.width, num_heads=m.heads, num_kv_heads=1, head_dim=m.dim,
                scale=m.scale, window=m.window,
                position=PositionSpec("rope_neox", rotary_dim=m.rot_dims, theta=m.rot_base) if m.rot_dims
                else PositionSpec("none"),
                params=LatentAttentionSpec(rank=m.kv_rank, rot_width=m.rot_dim, value_dim=m.vdim,
                                           norm_eps=self.norm_eps, gated=True))
            ffn = None
            if L.mlp is not None:
                ffn = FeedForwardSpec(kind="moe", hidden=self.width, intermediate=L.mlp.ff,
                                      params=MoESpec(experts=L.mlp.experts, top=L.mlp.top, activation="relu2",
                                                     weights="softmax_chosen"))
            blocks.append(BlockSpec(kind="parallel", mixer=mixer, ffn=ffn, mixer_norm=norm, prefix=f"l{i}.",
                                    mixer_prefix="mix.", ffn_prefix="mlp.", mixer_norm_name="norm1"))
        n = len(self.layers)
        order: List[RunEntry] = []
        vectors: Tuple[Tuple[str, int], ...] = ()
        if self.loop is None:
            order = [RunEntry(i) for i in range(n)]
        else:
            start, stop, times = self.loop
            vectors = (("loop.step", times),)
            order += [RunEntry(i) for i in range(start)]
            for p in range(times):
                for i in range(start, stop):
                    before = StreamAdd(embedding=p > 0, vector="loop.step", row=p) if i == start else None
                    order.append(RunEntry(i, before=before))
            order += [RunEntry(i) for i in range(stop, n)]
        inputs: Tuple[InputSpec, ...] = ()
        if self.bigram is not None:
            inputs = (InputSpec("pair_hash", PairHashSpec(*self.bigram, table_name="bigram")),)
        return ModelSpec(
            architecture=ARCHITECTURE, vocab_size=self.vocab, hidden=self.width, max_positions=self.max_positions,
            blocks=tuple(blocks), run_order=tuple(order), final_norm=norm, tie_embeddings=False,
            embed_name="embed", final_norm_name="final.norm", head_name="head", inputs=inputs,
            stream_vectors=vectors, logit_softcap=self.logit_softcap)
