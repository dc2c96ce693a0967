"""Debusun as data: its config.json typed, and turned into a `ModelSpec`.

A decoder-only model whose layers are listed one by one in config.json (`layers`: each entry a `type`, the mixer's
sizes under `mixer`, and `mlp` or null); a span of the layers may run several times in a row (`loop`).  What the design
fixes is written here; what config.json gives is read from there:

  embedding   x = embed[token] * embedding.scale + bigram[row], row = (previous token * mul_prev + token * mul_cur) mod
              buckets, and row `buckets` (the table's last) for a sequence's first token
  loop        layers start .. stop - 1 run `times` times with the same tensors, each pass on a cache and state of its
              own; before a pass's first layer x gets the embedding's output once more (not before the first pass) and
              then row t of `loop.step`, t the number of the pass
  layer       pre-norm: x <- x + mixer(norm1(x)), then x <- x + ff(norm2(x)); `mlp: null` leaves the second out
  type "attention"         grouped-query softmax attention over the last mask.size tokens; rotary positions on the first
              rot.dims dims of q and k in pairs (2i, 2i + 1), f_i = rot.base^(-2i / rot.dims); after the rotation every q
              and k head is divided by its root mean square (eps of the model, no weight); score = (q . k) * scale;
              value heads of a size of their own
  type "latent_attention"  what a token keeps is a latent c (kv_rank dims, RMS-normed with a weight) and one rotated key
              part of rot_dim dims shared by the heads; a head's plain key dims and its values are products of c; the
              rotary frequencies are blended along a ramp (rot.scaling: factor, original, fast, slow) and cos and sin
              grow by 0.1 ln(factor) + 1; a window; a sink in the softmax's denominator for every head; the heads times
              sigmoid(g h) before the output projection
  type "mamba2"            a selective state space per head with a short causal convolution in front, a gate and a
              grouped RMS norm behind (`parts/ssm.py`)
  mlp         dense: down(relu(up h)^2)
  output      RMSNorm `final.norm`, `head`

Tensor names: `embed`, `bigram`, `loop.step`, `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*`, `l<i>.mlp.{up,down}`,
`final.norm`, `head`.
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
    scaling: Optional[Tuple[float, float, float, float]] = None      # factor, original, fast, slow

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "Rotary":
        raw = _obj(raw, "rot", where)
        scaling = None
        if raw.get("scaling") is not None:
            sc = _obj(raw["scaling"], "rot.scaling", where)
            scaling = tuple(_require(sc, k, float, where) for k in ("factor", "original", "fast", "slow"))
            if min(scaling) <= 0:
                raise ConfigError(f"{where}: rot.scaling needs positive numbers")
        r = cls(_require(raw, "dims", int, where), _require(raw, "base", float, where), scaling)
        if r.dims <= 0 or r.dims % 2 or not r.base > 1:
            raise ConfigError(f"{where}: rot.dims must be even and positive, rot.base above 1")
        return r

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return out

    def spec(self, head_dim: int, max_positions: int) -> PartSpec:
        params: Dict[str, Any] = dict(head_dim=head_dim, rotary_dim=self.dims, theta=self.base, max_positions=max_positions,
                                      interleaved=True)
        if self.scaling is not None:
            factor, original, fast, slow = self.scaling
            params["scaling"] = dict(kind="ramp", factor=factor, original=original, fast=fast, slow=slow)
        return PartSpec("rope", params)


def _window(raw: Dict[str, Any], where: str) -> int:
    if raw.get("mask") is None:
        return 0
    w = _require(_obj(raw["mask"], "mask", where), "size", int, where)
    if w <= 0:
        raise ConfigError(f"{where}: mask.size must be positive")
    return w


@dataclass(frozen=True)
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    rot: Optional[Rotary]

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "AttentionMixer":
        raw = _obj(raw, "mixer", where)
        dim = _require(raw, "dim", int, where)
        m = cls(_require(raw, "heads", int, where), _require(raw, "kv_heads", int, where), dim, _opt(raw, "vdim", int, where) or dim,
                _require(raw, "scale", float, where), _window(raw, where),
                Rotary.from_dict(raw["rot"], where) if raw.get("rot") is not None else None)
        if min(m.heads, m.kv_heads, m.dim, m.vdim) <= 0 or m.heads % m.kv_heads:
            raise ConfigError(f"{where}: {m.heads} heads of {m.dim}/{m.vdim} on {m.kv_heads} kv heads cannot be run")
        if m.rot is not None and m.rot.dims > m.dim:
            raise ConfigError(f"{where}: {m.rot.dims} rotated dims of a head of {m.dim}")
        return m

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale}
        if self.window:
            out["mask"] = {"size": self.window}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class LatentMixer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int
    rot: Rotary

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "LatentMixer":
        raw = _obj(raw, "mixer", where)
        dim = _require(raw, "dim", int, where)
        m = cls(_require(raw, "heads", int, where), dim, _require(raw, "rot_dim", int, where), _opt(raw, "vdim", int, where) or dim,
                _require(raw, "kv_rank", int, where), _require(raw, "scale", float, where), _window(raw, where),
                Rotary.from_dict(raw.get("rot"), where))
        if min(m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank) <= 0 or m.rot.dims != m.rot_dim:
            raise ConfigError(f"{where}: {m.heads} heads of {m.dim} + {m.rot_dim} dims (rot.dims {m.rot.dims}) over a latent of "
                              f"{m.kv_rank} cannot be run")
        return m

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                               "kv_rank": self.kv_rank, "scale": self.scale, "rot": self.rot.to_dict()}
        if self.window:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class StateSpaceMixer:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "StateSpaceMixer":
        raw = _obj(raw, "mixer", where)
        m = cls(*(_require(raw, k, int, where) for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")))
        if (min(m.heads, m.vdim, m.state, m.groups, m.conv, m.norm_groups) <= 0 or m.heads % m.groups
                or (m.heads * m.vdim) % m.norm_groups):
            raise ConfigError(f"{where}: {m.heads} heads of {m.vdim} in {m.groups} groups, {m.norm_groups} norm groups cannot be run")
        return m

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


MIXERS = {"attention": AttentionMixer, "latent_attention": LatentMixer, "mamba2": StateSpaceMixer}


@dataclass(frozen=True)
class DebusunLayer:
    type: str
    mixer: Any
    ff: Optional[int]                # the dense feed-forward's inner size; None: no feed-forward


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class DebusunConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    buckets: int
    mul_prev: int
    mul_cur: int
    layers: Tuple[DebusunLayer, ...]
    loop: Optional[Loop] = None
    max_positions: int = DEFAULT_POSITIONS
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Debusun"

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "DebusunConfig":
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
            ff = None
            if l.get("mlp") is not None:
                mlp = _obj(l["mlp"], "mlp", at)
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{at}: unknown mlp kind {mlp.get('kind')!r} (dense)")
                ff = _require(mlp, "ff", int, at)
                if ff <= 0:
                    raise ConfigError(f"{at}: mlp.ff must be positive")
            out.append(DebusunLayer(kind, MIXERS[kind].from_dict(l.get("mixer"), at), ff))
        loop = None
        if raw.get("loop") is not None:
            lp = _obj(raw["loop"], "loop", where)
            loop = Loop(*(_require(lp, k, int, where) for k in ("start", "stop", "times")))
            if not (0 <= loop.start < loop.stop <= len(out)) or loop.times < 1:
                raise ConfigError(f"{where}: loop {loop.start}..{loop.stop} x {loop.times} does not fit {len(out)} layers")
        emb = _obj(raw.get("embedding"), "embedding", where)
        big = _obj(emb.get("bigram"), "embedding.bigram", where)
        eos = raw.get("eos_token_id")
        cfg = cls(vocab=_require(raw, "vocab", int, where), width=_require(raw, "width", int, where),
                  norm_eps=_require(_obj(raw.get("norm"), "norm", where), "eps", float, where),
                  embedding_scale=_require(emb, "scale", float, where), buckets=_require(big, "buckets", int, where),
                  mul_prev=_require(big, "mul_prev", int, where), mul_cur=_require(big, "mul_cur", int, where),
                  layers=tuple(out), loop=loop, max_positions=_opt(raw, "max_positions", int, where) or DEFAULT_POSITIONS,
                  eos_token_id=None if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos])),
                  architecture=str(raw.get("architecture") or (raw.get("architectures") or ["Debusun"])[0]))
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.max_positions <= 0 or cfg.buckets <= 0 or min(cfg.mul_prev, cfg.mul_cur) < 0:
            raise ConfigError(f"{where}: vocab, width, max_positions and buckets must be positive, the multipliers not negative")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        layers = [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}}
                  for l in self.layers]
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps},
                               "embedding": {"scale": self.embedding_scale,
                                             "bigram": {"buckets": self.buckets, "mul_prev": self.mul_prev, "mul_cur": self.mul_cur}},
                               "layers": layers}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        if self.max_positions != DEFAULT_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            out["eos_token_id"] = list(self.eos_token_id)
        return out


def _mixer_spec(cfg: DebusunConfig, l: DebusunLayer) -> PartSpec:
    m = l.mixer
    if l.type == "attention":
        return PartSpec("attention", dict(
            hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim, bias=False,
            qk_norm="head_unit", qk_norm_eps=cfg.norm_eps, window=m.window or None, scale=m.scale,
            position=None if m.rot is None else m.rot.spec(m.dim, cfg.max_positions),
            names={"q": "q", "k": "k", "v": "v", "o": "o"}))
    if l.type == "latent_attention":
        return PartSpec("latent_attention", dict(
            hidden_size=cfg.width, num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim, kv_rank=m.kv_rank,
            scale=m.scale, window=m.window or None, norm_eps=cfg.norm_eps, sinks=True, gate=True,
            position=m.rot.spec(m.rot_dim, cfg.max_positions)))
    return PartSpec("mamba2", dict(hidden_size=cfg.width, num_heads=m.heads, value_dim=m.vdim, state_dim=m.state, groups=m.groups,
                                   conv=m.conv, norm_groups=m.norm_groups, norm_eps=cfg.norm_eps))


def debusun_spec(cfg: DebusunConfig) -> ModelSpec:
    layers = []
    for i, l in enumerate(cfg.layers):
        norms = {"norm1": PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name=f"l{i}.norm1"))}
        if l.ff is not None:
            norms["norm2"] = PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name=f"l{i}.norm2"))
        ff = None if l.ff is None else PartSpec("mlp", dict(hidden_size=cfg.width, intermediate_size=l.ff, activation="relu2",
                                                            names={"up": "up", "down": "down"}))
        layers.append(LayerSpec(prefix=f"l{i}", block="prenorm", mixer=_mixer_spec(cfg, l), feed_forward=ff, norms=norms,
                                mixer_name="mix", feed_forward_name="mlp"))
    n = len(cfg.layers)
    schedule = []
    if cfg.loop is None:
        schedule = [ScheduleEntry(i) for i in range(n)]
    else:
        a, b, times = cfg.loop.start, cfg.loop.stop, cfg.loop.times
        schedule = [ScheduleEntry(i) for i in range(a)]
        next_id = n                                             # caches of the passes after the first
        for t in range(times):
            start = PartSpec("pass_start", dict(name="loop.step", dim=cfg.width, rows=times, row=t, add_first=t > 0))
            for i in range(a, b):
                cache_id = None
                if t > 0:
                    cache_id, next_id = next_id, next_id + 1
                schedule.append(ScheduleEntry(i, cache_id=cache_id, before=start if i == a else None))
        schedule += [ScheduleEntry(i) for i in range(b, n)]
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.max_positions,
        embedding=PartSpec("embedding", dict(name="embed", vocab_size=cfg.vocab, dim=cfg.width, scale=cfg.embedding_scale,
                                             pairs=dict(name="bigram", buckets=cfg.buckets, mul_prev=cfg.mul_prev,
                                                        mul_cur=cfg.mul_cur))),
        layers=tuple(layers), schedule=tuple(schedule),
        final_norm=PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name="final.norm")),
        head=PartSpec("lm_head", dict(name="head", tied=False, vocab_size=cfg.vocab, dim=cfg.width)),
        eos_token_ids=tuple(cfg.eos_token_id or ()))


DEBUSUN = ModelFamily("debusun", DebusunConfig, debusun_spec)
register_architecture("Debusun", DEBUSUN)
