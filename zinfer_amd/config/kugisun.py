"""Typed configuration of the Kugisun decoder, read from its config.json.

A Kugisun model keeps its residual stream in several copies.  A sublayer reads a weighted sum
of the copies through an RMS norm whose gain is stored around zero, and its output joins every
copy with a weight of its own after the copies have been mixed among themselves; the logits
come from the copies added up.  A layer's mixer is two mixers side by side on the same input,
causal grouped-query attention (biases, a norm a head on q and k, neighbouring pairs of some
leading elements rotated by the position) and a gated delta rule (short convolutions, a matrix
a head that every token corrects towards its value), added with a weight each.  The
feed-forward is a gated one, or a mixture of such experts whose router takes a soft-max over
all its outputs, lets a correction and groups of experts into the choice only, and has outputs
without an expert behind them that hand their input on; a shared expert with a gate a token
runs beside it.  A learned position row is added to the embedding; the head is the embedding.
A layer may run with another layer's tensors and a cache and state of its own.  Every size and
every constant that can differ between models comes from config.json; the layers may all
differ.

    {"architecture": "Kugisun", "vocab": V, "width": W, "max_positions": P, "streams": S,
     "norm": {"eps": e},
     "layers": [
       {"type": "parallel",
        "mixer": {"left": {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": s,
                           "rot": {"dims": r, "base": b}},
                  "right": {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": taps},
                  "left_scale": cl, "right_scale": cr},
        "mlp": ...},
       {"type": "parallel", "mixer": ..., "mlp": ..., "weights_of": j}]}
    mlp: null | {"kind": "dense", "ff": f}
              | {"kind": "moe", "expert": {"ff": f}, "shared": null | {"ff": f},
                 "router": {"experts": E, "identity": I, "top": k, "scale": c,
                            "groups": null | {"count": G, "keep": g}}}

Without "streams" the stream is one and a layer is x += mixer(norm1(x)); x += ff(norm2(x)).

Tensor names: ``embed``, ``pos``, ``final.norm``, and per layer i under ``l<i>.``: ``norm1``,
``norm2``, ``hc1.in hc1.mix hc1.out`` (``hc2.*`` for the feed-forward); the mixer's under
``mix.left.``: ``q q.b k k.b v v.b q.norm k.norm o`` and ``mix.right.``: ``q q.conv k k.conv v
v.conv b a A_log dt_bias g norm o``; the feed-forward's under ``mlp.``: ``gate up down`` or
``router correction e<j>.gate e<j>.up e<j>.down shared.gate shared.up shared.down shared.sg``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError
from .nupovik import _int, _num, _obj
from .specs import (GatedDeltaRuleSpec, GatedExpertSpec, LayerNormSpec, LeadingRotarySpec,
                    MaskedGqaAttentionSpec, ModelSpec, MoeSpec, ParallelMixerSpec, ScheduleEntry,
                    StreamBlockSpec, SwiGluSpec)
from .registry import register_architecture

# constants the design fixes
UNIT_EPS = 1e-6               # inside the root of the delta rule's unit vectors
NORM_GAIN_OFFSET = 1.0        # the layers' norms store their gain around zero
MIXERS = ("parallel",)


def pair_frequencies(dims: int, base: float) -> Tuple[float, ...]:
    """f_i = base^(-2i / dims) for the pairs i < dims / 2, formed in 64-bit."""
    return tuple(float(base) ** (-2.0 * i / dims) for i in range(dims // 2))


@dataclass(frozen=True)
class KugisunConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    streams: Optional[int]
    layers: Tuple[object, ...]            # one StreamBlockSpec for every layer with tensors
    layer_numbers: Tuple[int, ...]        # the number each of them goes by in the file
    order: Tuple[int, ...]                # for every run, the index into ``layers``
    raw: dict

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, raw: dict) -> "KugisunConfig":
        vocab = _int(raw, "vocab", "")
        width = _int(raw, "width", "")
        max_positions = _int(raw, "max_positions", "")
        eps = _num(_obj(raw, "norm", ""), "eps", "norm.")
        if not eps >= 0.0:
            raise ConfigError(f"config.json: norm.eps={eps} must not be negative")
        streams = None if raw.get("streams") is None else _int(raw, "streams", "")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        # whose tensors every layer runs with
        owner = []
        for i, L in enumerate(layers):
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
            j = i
            seen = set()
            while layers[j].get("weights_of") is not None:
                seen.add(j)
                j = _int(layers[j], "weights_of", f"layers[{j}].", 0)
                if j >= len(layers) or j in seen or not isinstance(layers[j], dict):
                    raise ConfigError(f"config.json: layers[{i}].weights_of does not lead to a "
                                      "layer with tensors of its own")
            owner.append(j)
        numbers = tuple(sorted(set(owner)))
        norm = cls._norm(width, eps)
        blocks = tuple(cls._block(j, layers[j], width, eps, norm, streams) for j in numbers)
        order = tuple(numbers.index(j) for j in owner)
        return cls(vocab, width, max_positions, eps, streams, blocks, numbers, order,
                   copy.deepcopy(raw))

    @staticmethod
    def _norm(width: int, eps: float) -> LayerNormSpec:
        # x / sqrt(mean x^2 + eps) * (1 + w): not centred, no bias; the tensor is the prefix itself
        return LayerNormSpec(width, eps, centred=False, weight_name="", bias_name=None,
                             gain_offset=NORM_GAIN_OFFSET)

    @staticmethod
    def _attention(m, mw: str, width: int, eps: float) -> MaskedGqaAttentionSpec:
        heads, kv = _int(m, "heads", mw), _int(m, "kv_heads", mw)
        dim = _int(m, "dim", mw)
        if heads % kv != 0:
            raise ConfigError(f"config.json: {mw}heads={heads} is no multiple of kv_heads={kv}")
        rotary = None
        if m.get("rot") is not None:
            r = _obj(m, "rot", mw)
            dims = _int(r, "dims", mw + "rot.", 0)
            base = _num(r, "base", mw + "rot.")
            if dims % 2 != 0 or dims > dim or not base > 0.0:
                raise ConfigError(f"config.json: {mw}rot: {dims} elements of heads of {dim} "
                                  f"with base {base} cannot be rotated in pairs")
            if dims > 0:
                rotary = LeadingRotarySpec(dims, pair_frequencies(dims, base), interleaved=True)
        return MaskedGqaAttentionSpec(
            hidden_size=width, n_heads=heads, n_kv_heads=kv, head_dim=dim,
            value_dim=_int(m, "vdim", mw), scale=_num(m, "scale", mw), qk_norm_eps=eps,
            qk_norm_per_head=True, bias=True, rotary=rotary, q_name="q", k_name="k", v_name="v",
            o_name="o", q_norm_name="q.norm", k_norm_name="k.norm")

    @staticmethod
    def _delta(m, mw: str, width: int, eps: float) -> GatedDeltaRuleSpec:
        heads, kv = _int(m, "heads", mw), _int(m, "kv_heads", mw)
        if heads % kv != 0:
            raise ConfigError(f"config.json: {mw}heads={heads} is no multiple of kv_heads={kv}")
        return GatedDeltaRuleSpec(
            hidden_size=width, n_heads=heads, n_kv_heads=kv, head_dim=_int(m, "dim", mw),
            value_dim=_int(m, "vdim", mw), conv_taps=_int(m, "conv", mw), norm_eps=eps,
            unit_eps=UNIT_EPS)

    @staticmethod
    def _block(i: int, L, width: int, eps: float, norm: LayerNormSpec,
               streams: Optional[int]) -> StreamBlockSpec:
        where = f"layers[{i}]."
        kind = L.get("type")
        if kind not in MIXERS:
            raise ConfigError(f"config.json: {where}type={kind!r}: the mixers of this design "
                              f"are {', '.join(repr(m) for m in MIXERS)}")
        m = _obj(L, "mixer", where)
        mw = where + "mixer."
        mixer = ParallelMixerSpec(
            left=KugisunConfig._attention(_obj(m, "left", mw), mw + "left.", width, eps),
            right=KugisunConfig._delta(_obj(m, "right", mw), mw + "right.", width, eps),
            left_scale=_num(m, "left_scale", mw), right_scale=_num(m, "right_scale", mw))
        ff = KugisunConfig._feed_forward(L.get("mlp"), where + "mlp.", width)
        return StreamBlockSpec(streams=streams or 1, mixer=mixer, feed_forward=ff,
                               mixer_norm=norm, ff_norm=norm if ff is not None else None,
                               learned=streams is not None)

    @staticmethod
    def _feed_forward(f, fw: str, width: int):
        if f is None:
            return None
        kind = f.get("kind") if isinstance(f, dict) else f
        if kind == "dense":
            return SwiGluSpec(width, _int(f, "ff", fw), gate_name="gate", up_name="up",
                              down_name="down")
        if kind != "moe":
            raise ConfigError(f"config.json: {fw}kind={kind!r}: the feed-forwards of this design "
                              "are 'dense' and 'moe'")
        r = _obj(f, "router", fw)
        rw = fw + "router."
        experts, top = _int(r, "experts", rw), _int(r, "top", rw)
        identity = 0 if r.get("identity") is None else _int(r, "identity", rw, 0)
        outputs = experts + identity
        if top > outputs:
            raise ConfigError(f"config.json: {rw}top={top} of {outputs} router outputs")
        groups = None
        if r.get("groups") is not None:
            g = _obj(r, "groups", rw)
            count, keep = _int(g, "count", rw + "groups."), _int(g, "keep", rw + "groups.")
            if outputs % count != 0 or keep > count or top > keep * (outputs // count):
                raise ConfigError(f"config.json: {rw}groups: {outputs} router outputs in {count} "
                                  f"equal groups, {keep} kept, {top} chosen do not fit together")
            groups = (count, keep)
        shared = None
        if f.get("shared") is not None:
            shared = GatedExpertSpec(_int(_obj(f, "shared", fw), "ff", fw + "shared."))
        return MoeSpec(hidden_size=width, n_experts=experts, top_k=top,
                       expert=GatedExpertSpec(_int(_obj(f, "expert", fw), "ff", fw + "expert.")),
                       shared=shared, scoring="softmax_all", correction_name="correction",
                       groups=groups, group_mark=1, normalize=False,
                       weight_scale=1.0 if r.get("scale") is None else _num(r, "scale", rw),
                       n_identity=identity,
                       shared_gate_name="sg" if shared is not None else None,
                       router_name="router", expert_prefix="e{}.", shared_prefix="shared.",
                       gate_name="gate", up_name="up", down_name="down")

    def to_dict(self) -> dict:
        return copy.deepcopy(self.raw)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def model_type(self) -> str:
        return "kugisun"

    # ------------------------------------------------------------------ the model's parts
    def model_spec(self) -> ModelSpec:
        """Every run of a layer, also one with another layer's tensors, has a cache and a state
        of its own."""
        return ModelSpec(
            vocab_size=self.vocab, hidden_size=self.width, max_positions=self.max_positions,
            layers=self.layers, schedule=tuple(ScheduleEntry(i) for i in self.order),
            final_norm=self._norm(self.width, self.norm_eps), tie_word_embeddings=True,
            embed_name="embed", final_norm_prefix="final.norm", head_name="head",
            layer_prefix="l{}.", position_table_name="pos",
            streams=self.streams if self.streams is not None else None,
            layer_numbers=self.layer_numbers)


register_architecture("Kugisun", KugisunConfig)
