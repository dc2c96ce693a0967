"""Vuzazen as data: its config.json typed, and turned into a `ModelSpec`.

A decoder-only model whose layers are listed one by one in config.json (`layers`: each entry a `type`, the mixer's
sizes under `mixer`, and `mlp` or null).  What the design fixes is written here; what config.json gives is read from
there:

  embedding   x = embed[token] * embedding.scale + bigram[row], row = (previous token * mul_prev + token * mul_cur) mod
              buckets, and row `buckets` (the table's last) for a sequence's first token
  layer       pre-norm: x <- x + mixer(norm1(x)), then x <- x + ff(norm2(x)); `mlp: null` leaves the second out;
              every norm (the model's last one too) is x * rsqrt(mean(x^2) + eps) * (1 + w): the tensor holds the
              factor's distance from one
  type "mlstm"             a matrix memory per head (`parts/mlstm.py`): exponential input gate, sigmoid forget gate,
              both logits capped by gate_cap * tanh(. / gate_cap), a running maximum that keeps the exponentials in
              range; q scaled by dim^-1/2; the heads' results divided by their root mean square, times a weight, times
              sigmoid(g h)
  type "latent_attention"  what a token keeps is a latent c (kv_rank dims, RMS-normed with a weight) and one rotated key
              part of rot_dim dims shared by the heads; a head's plain key dims and its values are products of c; the
              queries come through a latent of their own (q_rank dims, RMS-normed with a weight); rotary positions
              on the rot_dim part in pairs (i, i + rot_dim / 2), f_i = rot.base^(-2i / rot.dims); every earlier token is
              seen; each head times one number sigmoid(g h) before the output projection
  type "attention"         grouped-query softmax attention over every earlier token without positions: q, k and v
              through a causal convolution per channel over the last `conv` tokens; RMS norm with a weight over the
              whole q and the whole k projection; every value head divided by its root mean square; head h's
              score is sum_g talk[h, g] * (q_g . k) * scale; each head times one number sigmoid(g h)
  mlp         dense: down(silu(gate h) * (up h)); moe: `router.experts` such feed-forwards of `expert.ff`, a token
              takes the `router.top` with the largest sigmoid(router h) and expert e sees score_e * h
  output      the norm `final.norm`, then the embedding table itself as the head

Tensor names: `embed`, `bigram`, `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*`, `l<i>.mlp.{gate,up,down}` or
`l<i>.mlp.{router,e<j>.gate,e<j>.up,e<j>.down}`, `final.norm`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.model_config import ConfigError, _require, _typed
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import ModelFamily, register_architecture

DEFAULT_POSITIONS = 1 << 15       # config.json names no longest sequence: what the engine plans its tables for


def _obj(raw: Any, what: str, where: str) -> Dict[str, Any]:
    if not isinstance(raw, dict):
        raise ConfigError(f"{where}: {what!r} must be an object")
    return raw


def _opt(raw: Optional[Dict[str, Any]], key: str, typ, where: str):
    return None if not raw or raw.get(key) is None else _typed(raw[key], key, typ, where)


@dataclass(frozen=True)
class Rotary:
    dims: int
    base: float

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "Rotary":
        raw = _obj(raw, "rot", where)
        r = cls(_require(raw, "dims", int, where), _require(raw, "base", float, where))
        if r.dims <= 0 or r.dims % 2 or not r.base > 1:
            raise ConfigError(f"{where}: rot.dims must be even and positive, rot.base above 1")
        return r

    def to_dict(self) -> Dict[str, Any]:
        return {"dims": self.dims, "base": self.base}


@dataclass(frozen=True)
class MatrixMemoryMixer:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "MatrixMemoryMixer":
        raw = _obj(raw, "mixer", where)
        dim = _require(raw, "dim", int, where)
        m = cls(_require(raw, "heads", int, where), dim, _opt(raw, "vdim", int, where) or dim,
                _require(raw, "gate_cap", float, where))
        if min(m.heads, m.dim, m.vdim) <= 0 or not m.gate_cap > 0:
            raise ConfigError(f"{where}: {m.heads} heads of {m.dim} by {m.vdim} with a gate cap of {m.gate_cap} cannot be run")
        return m

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class LatentMixer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: Rotary

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "LatentMixer":
        raw = _obj(raw, "mixer", where)
        dim = _require(raw, "dim", int, where)
        m = cls(_require(raw, "heads", int, where), dim, _require(raw, "rot_dim", int, where), _opt(raw, "vdim", int, where) or dim,
                _require(raw, "kv_rank", int, where), _require(raw, "q_rank", int, where), _require(raw, "scale", float, where),
                Rotary.from_dict(raw.get("rot"), where))
        if min(m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.q_rank) <= 0 or m.rot.dims != m.rot_dim:
            raise ConfigError(f"{where}: {m.heads} heads of {m.dim} + {m.rot_dim} dims (rot.dims {m.rot.dims}) over latents of "
                              f"{m.kv_rank} and {m.q_rank} cannot be run")
        return m

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "q_rank": self.q_rank, "scale": self.scale, "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class ConvAttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int                          # taps of the convolution over time; 0: none (one tap: a factor a channel)

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "ConvAttentionMixer":
        raw = _obj(raw, "mixer", where)
        dim = _require(raw, "dim", int, where)
        m = cls(_require(raw, "heads", int, where), _require(raw, "kv_heads", int, where), dim, _opt(raw, "vdim", int, where) or dim,
                _require(raw, "scale", float, where), _opt(raw, "conv", int, where) or 0)
        if min(m.heads, m.kv_heads, m.dim, m.vdim) <= 0 or m.heads % m.kv_heads or m.conv < 0:
            raise ConfigError(f"{where}: {m.heads} heads of {m.dim}/{m.vdim} on {m.kv_heads} kv heads with {m.conv} taps cannot be run")
        return m

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale}
        if self.conv:
            out["conv"] = self.conv
        return out


MIXERS = {"mlstm": MatrixMemoryMixer, "latent_attention": LatentMixer, "attention": ConvAttentionMixer}


@dataclass(frozen=True)
class FeedForward:
    kind: str                          # "dense" or "moe"
    ff: int                            # the inner size (of one expert)
    experts: int = 0
    top: int = 0

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "FeedForward":
        raw = _obj(raw, "mlp", where)
        kind = str(raw.get("kind", "dense"))
        if kind == "dense":
            f = cls("dense", _require(raw, "ff", int, where))
        elif kind == "moe":
            router = _obj(raw.get("router"), "mlp.router", where)
            f = cls("moe", _require(_obj(raw.get("expert"), "mlp.expert", where), "ff", int, where),
                    _require(router, "experts", int, where), _require(router, "top", int, where))
            if not (0 < f.top <= f.experts):
                raise ConfigError(f"{where}: {f.top} of {f.experts} experts cannot be chosen")
        else:
            raise ConfigError(f"{where}: unknown mlp kind {kind!r} (dense, moe)")
        if f.ff <= 0:
            raise ConfigError(f"{where}: the feed-forward's inner size must be positive")
        return f

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class VuzazenLayer:
    type: str
    mixer: Any
    mlp: Optional[FeedForward]         # None: no feed-forward


@dataclass(frozen=True)
class VuzazenConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    buckets: int
    mul_prev: int
    mul_cur: int
    layers: Tuple[VuzazenLayer, ...]
    max_positions: int = DEFAULT_POSITIONS
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Vuzazen"

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "VuzazenConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where}: 'layers' must be a list of layers")
        out = []
        for i, l in enumerate(layers):
            at = f"{where}: layers[{i}]"
            l = _obj(l, f"layers[{i}]", where)
            kind = _require(l, "type", str, at)
            if kind not in MIXERS:
                raise ConfigError(f"{at}: unknown layer type {kind!r} ({', '.join(MIXERS)})")
            out.append(VuzazenLayer(kind, MIXERS[kind].from_dict(l.get("mixer"), at),
                                    None if l.get("mlp") is None else FeedForward.from_dict(l["mlp"], at)))
        emb = _obj(raw.get("embedding"), "embedding", where)
        big = _obj(emb.get("bigram"), "embedding.bigram", where)
        eos = raw.get("eos_token_id")
        cfg = cls(vocab=_require(raw, "vocab", int, where), width=_require(raw, "width", int, where),
                  norm_eps=_require(_obj(raw.get("norm"), "norm", where), "eps", float, where),
                  embedding_scale=_require(emb, "scale", float, where), buckets=_require(big, "buckets", int, where),
                  mul_prev=_require(big, "mul_prev", int, where), mul_cur=_require(big, "mul_cur", int, where),
                  layers=tuple(out), max_positions=_opt(raw, "max_positions", int, where) or DEFAULT_POSITIONS,
                  eos_token_id=None if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos])),
                  architecture=str(raw.get("architecture") or (raw.get("architectures") or ["Vuzazen"])[0]))
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.max_positions <= 0 or cfg.buckets <= 0 or min(cfg.mul_prev, cfg.mul_cur) < 0:
            raise ConfigError(f"{where}: vocab, width, max_positions and buckets must be positive, the multipliers not negative")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        layers = [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                  for l in self.layers]
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps},
                               "embedding": {"scale": self.embedding_scale,
                                             "bigram": {"buckets": self.buckets, "mul_prev": self.mul_prev, "mul_cur": self.mul_cur}},
                               "layers": layers}
        if self.max_positions != DEFAULT_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            out["eos_token_id"] = list(self.eos_token_id)
        return out


def _mixer_spec(cfg: VuzazenConfig, l: VuzazenLayer) -> PartSpec:
    m = l.mixer
    if l.type == "mlstm":
        return PartSpec("mlstm", dict(hidden_size=cfg.width, num_heads=m.heads, key_dim=m.dim, value_dim=m.vdim,
                                      gate_cap=m.gate_cap, norm_eps=cfg.norm_eps))
    if l.type == "latent_attention":
        rope = PartSpec("rope", dict(head_dim=m.rot_dim, rotary_dim=m.rot.dims, theta=m.rot.base,
                                     max_positions=cfg.max_positions, interleaved=False))
        return PartSpec("latent_attention", dict(
            hidden_size=cfg.width, num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim, kv_rank=m.kv_rank,
            q_rank=m.q_rank, scale=m.scale, window=None, norm_eps=cfg.norm_eps, sinks=False, gate="head", position=rope))
    return PartSpec("attention", dict(
        hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim, bias=False,
        qk_norm="row", qk_norm_eps=cfg.norm_eps, window=None, scale=m.scale, position=None, conv=m.conv,
        value_norm="head_unit", talking_heads=True, head_gate=True,
        names={"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "q_conv": "q.conv",
               "k_conv": "k.conv", "v_conv": "v.conv", "talk": "talk", "head_gate": "g"}))


def _feed_forward_spec(cfg: VuzazenConfig, f: FeedForward) -> PartSpec:
    if f.kind == "dense":
        return PartSpec("gated_mlp", dict(hidden_size=cfg.width, intermediate_size=f.ff, activation="silu",
                                          names={"gate": "gate", "up": "up", "down": "down"}))
    return PartSpec("routed_experts", dict(
        hidden_size=cfg.width, intermediate_size=f.ff, num_experts=f.experts, top=f.top, activation="silu",
        scores="sigmoid", weigh="input",
        names={"router": "router", "gate": "e{i}.gate", "up": "e{i}.up", "down": "e{i}.down"}))


def vuzazen_spec(cfg: VuzazenConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name=name, weight_offset=1.0))

    layers = []
    for i, l in enumerate(cfg.layers):
        norms = {"norm1": norm(f"l{i}.norm1")}
        if l.mlp is not None:
            norms["norm2"] = norm(f"l{i}.norm2")
        layers.append(LayerSpec(prefix=f"l{i}", block="prenorm", mixer=_mixer_spec(cfg, l),
                                feed_forward=None if l.mlp is None else _feed_forward_spec(cfg, l.mlp), norms=norms,
                                mixer_name="mix", feed_forward_name="mlp"))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.max_positions,
        embedding=PartSpec("embedding", dict(name="embed", vocab_size=cfg.vocab, dim=cfg.width, scale=cfg.embedding_scale,
                                             pairs=dict(name="bigram", buckets=cfg.buckets, mul_prev=cfg.mul_prev,
                                                        mul_cur=cfg.mul_cur))),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
        final_norm=norm("final.norm"),
        head=PartSpec("lm_head", dict(name="embed", tied=True, vocab_size=cfg.vocab, dim=cfg.width)),
        eos_token_ids=tuple(cfg.eos_token_id or ()))


VUZAZEN = ModelFamily("vuzazen", VuzazenConfig, vuzazen_spec)
register_architecture("Vuzazen", VUZAZEN)
