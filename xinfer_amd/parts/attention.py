"""Paged grouped-query attention as a mixer.

h -> packed q/k/v projection (+ bias) -> per-head RMSNorm of q and k -> rotation by position ->
keys/values into the paged cache -> causal attention over the cache (all keys, or the
last `window`) -> output projection.  Reference: Attention::forward_with_kv,
/root/reference/src/models/layers/attention.rs:796-977 (projection 805-828, q/k norm
709-748, RoPE 872-879, paged attention 947-958, o_proj 976); q, k, v weights are
concatenated at load as in attention.rs:376-407.

Beside that form the mixer takes, each as a parameter of its spec: values of another head size
than the keys (`value_dim`); the q/k RMSNorm over the whole projection instead of head by head
(`qk_norm="row"`, weights as long as the projection); a soft cap c on the scores, c tanh(s / c)
(`score_softcap`); a bias that takes `distance_slopes[h] * (i - j)` off head h's score of query i
and key j; values blended with those another layer made for the same token, (1 - m) v + m v_other
(`value_mix`: the layers of one `key` share the values of the one that is their `source`, m is a
scalar tensor of the layer); other tensor names (`names`).  Any of these takes the step through
`_forward_general`: one kernel norms the projection, blends the values and writes the cache, and
the attention kernels that know the score's options follow.  That kernel also rotates q and k by
position (pairs (i, i + rotary_dim / 2), float32 tables) where the spec names a position encoding and
no q/k norm.

`qk_norm="head_unit"`: every q and k head is divided by its root mean square over head_dim (`qk_norm_eps` inside the
root), without a weight, AFTER the rotation.  A rotation turns pairs of dims and leaves a head's sum of squares as it
is, so the plain form computes this with its own kernels (norm with a weight of ones, then rotation: the same but for
rounding); with the options of the paragraph above, or with `general=True`, a kernel that takes a head at a time does
it in the order given (`kernels.head_rows`: rotation of either pairing, then the unit norm, then the cache write).

A third group of options, each a parameter of the spec, goes through `_forward_rows` (no rotation, `qk_norm` "row" or
none): `conv` n: q, k and v pass a causal convolution per channel over the last n tokens right after the
projection (tensors `q_conv`, `k_conv`, `v_conv` [channels, n], no bias; the last n - 1 projected rows of a request are
state of the layer, "conv_tail"; one tap is a factor a channel and keeps nothing); `value_norm="head_unit"`: every value head is divided by its root mean square and
cached so; `talking_heads`: head h's score of a key is sum_g talk[h, g] * (head g's score) before the softmax (tensor
`talk` [heads, heads]); `head_gate`: head h's result times sigmoid(w_h . x), one number a head (tensor `head_gate`
[heads, hidden], packed with q, k and v).  The heads' sum moves to the query's side, q'_h = [sum_{g on kv head c}
talk[h, g] q_g for every kv head c], scored against a token's whole k row: the K pool of such a layer holds one head
of kv_heads * head_dim dims and the attention kernels read the keys of that one head and the values of the query head's
own kv head.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import (Folded, KVNeed, LayerCache, Mixer, PAGE, PoolNeed, StateNeed, StepContext, position_encoding_class,
                   register_mixer)
from .linear import Linear


@register_mixer("attention")
class PagedAttention(Mixer):
    VECTOR_MIN_DECODE = 512      # decoded tokens lie in a page each: the form with one wave per head stays ahead up to here
    DECODE_PACKED = True         # steps of single tokens: norm, rotation and cache write inside the attention kernel

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.nq = int(spec["num_heads"])
        self.nkv = int(spec["num_kv_heads"])
        self.d = int(spec["head_dim"])
        self.bias = bool(spec.get("bias", False))
        self.qk_norm = bool(spec.get("qk_norm", False))
        self.qk_norm_eps = float(spec.get("qk_norm_eps", 1e-6))
        self.window = int(spec.get("window") or 0)
        self.scale = float(spec.get("scale", self.d ** -0.5))
        self.dv = int(spec.get("value_dim") or self.d)
        self.row_norm = spec.get("qk_norm") == "row"
        self.unit_norm = spec.get("qk_norm") == "head_unit"
        self.softcap = float(spec.get("score_softcap") or 0.0)
        slopes = spec.get("distance_slopes")
        self.slope_values = None if slopes is None else tuple(float(a) for a in slopes)
        if self.slope_values is not None and len(self.slope_values) != self.nq:
            raise ValueError(f"{len(self.slope_values)} distance slopes for {self.nq} query heads")
        vm = spec.get("value_mix")
        self.value_mix_key = None if not vm else str(vm.get("key", "values"))
        self.value_mix_source = bool(vm and vm.get("source", False))
        self.mix = 0.0               # the blend's scalar, read at load
        self.slopes = None           # float32 [nq] on the device
        # the options that the fused q/k kernel and the attention kernels of the plain form do not know
        self.general = bool(self.dv != self.d or self.row_norm or self.softcap > 0 or self.slope_values is not None
                            or self.value_mix_key is not None or spec.get("general", False))
        interleaved = spec.get("position") is not None and bool(spec["position"].get("interleaved", False))
        # the general form's heads are made ready a head at a time where they are normed one by one or turned in pairs
        # (2i, 2i + 1); else a row at a time
        self.by_head = self.general and (self.unit_norm or interleaved)
        if self.by_head and (self.row_norm or self.value_mix_key is not None):
            raise NotImplementedError("attention whose heads are normed one by one or turned in pairs (2i, 2i + 1) takes no "
                                      "norm over the whole projection and no blended values")
        self.taps = int(spec.get("conv") or 0)
        self.value_unit = spec.get("value_norm") == "head_unit"
        if spec.get("value_norm") not in (None, "head_unit"):
            raise ValueError(f"value_norm {spec.get('value_norm')!r}: 'head_unit' or none")
        self.talking = bool(spec.get("talking_heads", False))
        self.head_gate = bool(spec.get("head_gate", False))
        # a convolution, normed values, mixed heads or a gate a head: one kernel makes a token's row ready
        self.rows_form = self.taps >= 1 or self.value_unit or self.talking or self.head_gate
        if self.rows_form:
            self.general = True
            if (self.by_head or spec.get("position") is not None or self.softcap > 0 or self.slope_values is not None
                    or self.value_mix_key is not None or self.bias or (self.qk_norm and not self.row_norm)):
                raise NotImplementedError("attention with a convolution, normed values, mixed heads or a gate a head takes the "
                                          "q/k norm over the whole projection or none, and no rotation, cap, bias or blend")
        self.conv_w = self.talk = None
        if self.general and not self.by_head and spec.get("position") is not None and self.qk_norm:
            raise NotImplementedError("attention with a soft cap, a distance bias, blended values or another value size takes a "
                                      "rotation of the pairs (i, i + rotary_dim / 2) and then no q/k norm")
        if self.general and (self.qk_norm and not (self.row_norm or self.unit_norm) or self.bias):
            raise NotImplementedError("attention with a soft cap, a distance bias, blended values or another value size "
                                      "takes the q/k norm over the whole projection, the heads' unit norm or none, and no biases")
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} kv heads")
        # A step of single tokens reads nothing on the host where the split-K decode kernel or the
        # generic kernel serves it; sizes that only the prefill kernel takes (more than 16 query heads
        # per kv head) need the step's lengths on the host to lay out its tiles.
        self.graph_safe = (dtype != torch.bfloat16 or kernels.decode_attention_takes(self.nq, self.nkv, self.d)
                           or self.general)
        self.decode_packed = (self.DECODE_PACKED and dtype == torch.bfloat16 and not self.general
                              and kernels.decode_attention_takes(self.nq, self.nkv, self.d))
        pos = spec.get("position")
        self.position = position_encoding_class(pos.kind)(pos, dtype) if pos is not None else None
        self.qkv: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.q_norm_w = self.k_norm_w = None
        self.qkv_bias = None         # float32 [(nq + 2 nkv) d], added by the kernel after the projection

    # ---- weights -----------------------------------------------------------
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
             "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias",
             "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "value_mix": "value_mix",
             "q_conv": "q_conv.weight", "k_conv": "k_conv.weight", "v_conv": "v_conv.weight", "talk": "talk",
             "head_gate": "head_gate.weight"}

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str):
        """The tensors' names: the spec's `names` (what follows the prefix) over the defaults."""
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, nq, nkv, d = (int(spec[k]) for k in ("hidden_size", "num_heads", "num_kv_heads", "head_dim"))
        dv = int(spec.get("value_dim") or d)
        n = cls._names(spec, prefix)
        out = [TensorDecl(n["q"], (nq * d, h)), TensorDecl(n["k"], (nkv * d, h)),
               TensorDecl(n["v"], (nkv * dv, h)), TensorDecl(n["o"], (h, nq * dv))]
        if spec.get("bias", False):    # q, k and v only: the reference's o_proj has none (attention.rs:596-608)
            out += [TensorDecl(n["q_bias"], (nq * d,)), TensorDecl(n["k_bias"], (nkv * d,)),
                    TensorDecl(n["v_bias"], (nkv * dv,))]
        if spec.get("qk_norm") == "row":
            out += [TensorDecl(n["q_norm"], (nq * d,), "norm"), TensorDecl(n["k_norm"], (nkv * d,), "norm")]
        elif spec.get("qk_norm", False) and spec.get("qk_norm") != "head_unit":
            out += [TensorDecl(n["q_norm"], (d,), "norm"), TensorDecl(n["k_norm"], (d,), "norm")]
        vm = spec.get("value_mix")
        if vm and not vm.get("source", False):
            out.append(TensorDecl(n["value_mix"], (), "mix"))
        taps = int(spec.get("conv") or 0)
        if taps >= 1:
            out += [TensorDecl(n["q_conv"], (nq * d, taps), "normal(0,0.5)"), TensorDecl(n["k_conv"], (nkv * d, taps), "normal(0,0.5)"),
                    TensorDecl(n["v_conv"], (nkv * dv, taps), "normal(0,0.5)")]
        if spec.get("talking_heads", False):
            out.append(TensorDecl(n["talk"], (nq, nq), "normal(0,0.5)"))
        if spec.get("head_gate", False):
            out.append(TensorDecl(n["head_gate"], (nq, h)))
        return out

    def load(self, store: WeightStore, prefix: str, device) -> None:
        def lin(name):
            t = store.get(name, None, device)
            return t.to(self.dtype) if (self.dtype == torch.float32 or t.dtype != torch.float32) else t
        names = self._names(self.spec, prefix)
        parts = [lin(names[n]) for n in (("q", "k", "v", "head_gate") if self.head_gate else ("q", "k", "v"))]
        if self.taps >= 1:
            self.conv_w = torch.cat([store.get(names[n], torch.float32, device) for n in ("q_conv", "k_conv", "v_conv")]).contiguous()
        if self.talking:
            self.talk = store.get(names["talk"], torch.float32, device).contiguous()
        common = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
        self.qkv = Linear(torch.cat([p.to(common) for p in parts], dim=0))
        self.o = Linear(lin(names["o"]))
        if self.bias:
            self.qkv_bias = torch.cat([store.get(names[f"{n}_bias"], torch.float32, device)
                                       for n in ("q", "k", "v")]).contiguous()
        if self.unit_norm:         # the plain form's kernels norm with a weight: ones
            self.q_norm_w = self.k_norm_w = None if self.general else torch.ones(self.d, dtype=torch.float32, device=device)
        elif self.qk_norm:
            self.q_norm_w = store.get(names["q_norm"], torch.float32, device).contiguous()
            self.k_norm_w = store.get(names["k_norm"], torch.float32, device).contiguous()
        if self.value_mix_key is not None and not self.value_mix_source:
            self.mix = float(store.get(names["value_mix"], torch.float32, "cpu").reshape(-1)[0])
        if self.slope_values is not None:
            self.slopes = torch.tensor(self.slope_values, dtype=torch.float32, device=device)
        if self.position is not None:
            self.position.load(store, prefix, device)

    # ---- cache ---------------------------------------------------------------
    def cache_need(self) -> KVNeed:
        # the matrix-core kernels of the bfloat16 path read V in groups of eight keys
        need = KVNeed.keys_values(self.nkv, self.d, self.window, v_grouped=self.dtype == torch.bfloat16,
                                  value_dim=self.dv)
        if self.talking:           # mixed heads score against a token's whole k row: one key head of all kv heads' dims
            need = KVNeed(need.window, (PoolNeed("k", (1, PAGE, self.nkv * self.d)), need.pools[1]))
        return need

    def state_need(self):
        if self.taps > 1:
            return StateNeed((self.taps - 1, self.nq * self.d + self.nkv * (self.d + self.dv)), torch.float32, "conv_tail")
        return None

    # ---- step ----------------------------------------------------------------
    takes_sink = True
    takes_folded = True

    def forward(self, x, ctx: StepContext, cache: LayerCache, sink=None):
        """`x`: rows or a `Folded`; `sink`: see `Part.takes_sink`."""
        if self.general:
            return self._forward_general(x, ctx, cache, sink)
        # a decode step of 17 to 256 rows: the tiled split-K product is ahead of the library, and the
        # kernel below adds its partial sums (which the form for prompt portions does not take)
        rows = None if isinstance(x, Folded) else x.shape[0]
        parts = (rows is not None and self.dtype == torch.bfloat16 and ctx.max_q_len == 1
                 and kernels.MID_FROM <= rows <= min(kernels.MID_ROWS, self.VECTOR_MIN_DECODE - 1))
        qkv = self.qkv(x, out_dtype=self.dtype, allow_split=parts)
        pos = self.position
        slots = ctx.slots[cache.group] if cache.write else ctx.no_slots
        vt = self.dtype == torch.bfloat16
        if (vt and ctx.max_q_len == 1 and self.decode_packed
                and kernels.mfma_attention_supported(self.nq, self.nkv, self.d, cache.k.shape[2])):
            # a step of single tokens: the attention kernel norms and rotates its own heads and
            # stores the new keys and values, one launch less in every layer
            a = kernels.attention_decode_packed_bf16(
                qkv, self.q_norm_w, self.k_norm_w, self.qk_norm_eps,
                pos.cos if pos is not None else ctx.empty_f32,
                pos.sin if pos is not None else ctx.empty_f32,
                pos.rotary_dim if pos is not None else 0,
                pos.interleaved if pos is not None else False,
                ctx.positions, slots, cache.k, cache.v, ctx.block_tables[cache.group], ctx.ctx_lens, ctx.max_ctx_len,
                self.nq, self.scale, self.window, bias=self.qkv_bias,
                similar=getattr(ctx, "similar_lengths", False))
            return self.o(a, out_dtype=self.dtype, allow_split=True, sink=sink)
        q = kernels.qk_norm_rope_kv(
            qkv, self.q_norm_w, self.k_norm_w, self.qk_norm_eps,
            pos.cos if pos is not None else ctx.empty_f32,
            pos.sin if pos is not None else ctx.empty_f32,
            pos.rotary_dim if pos is not None else 0,
            pos.interleaved if pos is not None else False,
            ctx.positions, slots, cache.k, cache.v, self.nq, self.nkv, self.d, v_grouped=vt,
            vector_min_tokens=128 if ctx.max_q_len > 1 else self.VECTOR_MIN_DECODE, bias=self.qkv_bias)
        a = kernels.attention(q, cache.k, cache.v, ctx, cache.group, self.scale, self.window, v_grouped=vt)
        return self.o(a, out_dtype=self.dtype, allow_split=True, sink=sink)     # the next norm adds the parts

    def _forward_general(self, x, ctx: StepContext, cache: LayerCache, sink=None):
        """The step with the options of the module's second paragraph (no rotation)."""
        if self.rows_form:
            return self._forward_rows(x, ctx, cache)
        qkv = self.qkv(x, out_dtype=self.dtype)
        slots = ctx.slots[cache.group] if cache.write else ctx.no_slots
        vt = self.dtype == torch.bfloat16
        v_other = None
        if self.value_mix_key is not None:
            key = ("value_mix", self.value_mix_key)
            if self.value_mix_source:          # this step's values, as projected, for the layers that blend them in
                ctx.scratch[key] = qkv[:, (self.nq + self.nkv) * self.d:]
            else:
                v_other = ctx.scratch.get(key)
                if v_other is None:
                    raise RuntimeError(f"values {self.value_mix_key!r} are blended in before the layer that makes them has run")
        pos = self.position
        if self.by_head:
            q = kernels.head_rows(qkv, slots, cache.k, cache.v, self.nq, self.nkv, self.d, self.dv, v_grouped=vt,
                                  cos=pos.cos if pos is not None else None, sin=pos.sin if pos is not None else None,
                                  rotary_dim=pos.rotary_dim if pos is not None else 0,
                                  interleaved=pos.interleaved if pos is not None else False, positions=ctx.positions,
                                  unit_norm=self.unit_norm, eps=self.qk_norm_eps)
            a = kernels.attention(q, cache.k, cache.v, ctx, cache.group, self.scale, self.window, v_grouped=vt,
                                  softcap=self.softcap, slopes=self.slopes)
            return self.o(a, out_dtype=self.dtype, allow_split=True, sink=sink)
        q = kernels.qkv_rows(qkv, self.q_norm_w, self.k_norm_w, self.qk_norm_eps, slots, cache.k, cache.v,
                             self.nq, self.nkv, self.d, self.dv, v_grouped=vt, v_other=v_other, mix=self.mix,
                             cos=pos.cos if pos is not None else None, sin=pos.sin if pos is not None else None,
                             rotary_dim=pos.rotary_dim if pos is not None else 0, positions=ctx.positions)
        a = kernels.attention(q, cache.k, cache.v, ctx, cache.group, self.scale, self.window, v_grouped=vt,
                              softcap=self.softcap, slopes=self.slopes)
        return self.o(a, out_dtype=self.dtype, allow_split=True, sink=sink)

    def _forward_rows(self, x, ctx: StepContext, cache: LayerCache):
        """The step with the options of the module's last paragraph."""
        p = self.qkv(x, out_dtype=self.dtype)                      # [q | k | v | a gate a head]
        C = self.nq * self.d + self.nkv * (self.d + self.dv)
        slots = ctx.slots[cache.group] if cache.write else ctx.no_slots
        vt = self.dtype == torch.bfloat16
        tails = None
        if self.taps > 1:
            tails = cache.states.get("conv_tail")
            if tails is None:
                raise RuntimeError("an attention with a convolution was given no state slots")
        q = kernels.conv_qkv_rows(p, self.conv_w, tails, ctx.state_slots, ctx.tok_seq, ctx.cu_q, self.q_norm_w, self.k_norm_w,
                                  self.qk_norm_eps, slots, cache.k, cache.v, self.nq, self.nkv, self.d, self.dv, v_grouped=vt,
                                  value_unit_norm=self.value_unit, talk=self.talk)
        if self.taps > 1 and cache.write:
            kernels.conv_tail(p[:, :C], tails, ctx.state_slots, ctx.cu_q)
        a = kernels.attention(q, cache.k, cache.v, ctx, cache.group, self.scale, self.window, v_grouped=vt)
        if self.head_gate:
            kernels.head_gate_(a, p[:, C:], self.nq)
        return self.o(a, out_dtype=self.dtype, allow_split=True)
