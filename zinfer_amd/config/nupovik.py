"""Typed configuration of the Nupovik decoder, read from its config.json.

A Nupovik model is a list of layers, each with one of three mixers and an optional
feed-forward (dense, or a mixture of experts); both sublayers of a layer read the same residual
stream, each through an RMS norm of its own, and their outputs are added to it together.  A
position vector of sines and cosines is added to the embedding.  A ``loop`` runs a range of
layers several times in a row with the same weights, every pass with caches and states of its
own; a pass begins by mixing the stream with the embedding's output through one matrix.
Every size and every constant that can differ between models comes from config.json (or, for
the narrow middles of the decays, from the tensors' shapes); the layers may all differ.

    {"architecture": "Nupovik", "vocab": V, "width": W, "norm": {"eps": e}, "logit_scale": s,
     "loop": null | {"start": a, "stop": b, "times": n},
     "layers": [
       {"type": "gla", "mixer": {"heads": H, "dim": d, "vdim": dv, "tau": t}, "mlp": ...},
       {"type": "latent_attention",
        "mixer": {"heads": H, "dim": d, "vdim": dv, "kv_rank": r, "scale": s}, "mlp": ...},
       {"type": "wkv", "mixer": {"heads": H, "dim": d}, "mlp": ...}]}
    mlp: null | {"kind": "dense", "ff": f}
              | {"kind": "moe", "expert": {"ff": f},
                 "router": {"experts": E, "top": k, "groups": null | {"count": G, "keep": g}}}

A mixer of "gla" or "wkv" may also say "decay_rank": the width of its decay's narrow middle; a
file's tensors decide it otherwise (16 when weights are drawn at random).

Tensor names: ``embed``, ``head``, ``final.norm``, ``loop.in``, and per layer i under ``l<i>.``:
``norm1``, ``norm2``; the mixer's under ``mix.``: ``q k v g o norm a1 a2 a2.b`` (gla),
``q dkv dkv.norm uk uv g o`` (latent_attention), ``mu.r mu.k mu.v mu.g mu.w r k v g w1 w2 w0 u
norm o`` (wkv); the feed-forward's under ``mlp.``: ``up down`` or ``router correction
e<j>.up e<j>.down``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError
from .registry import register_architecture
from .specs import (DenseMlpSpec, GatedLinearAttentionSpec, LatentAttentionSpec, LayerNormSpec,
                    ModelSpec, MoeSpec, ParallelBlockSpec, PlainExpertSpec, ScheduleEntry,
                    SinusoidalPositionSpec, TokenShiftRecurrenceSpec)

# positions are 32-bit numbers in the kernels, and exact as such up to here
MAX_POSITIONS = 1 << 24
# constants the design fixes
FF_ACTIVATION = "relu2"                 # dense layers and experts: the square of max(z, 0)
POSITION_BASE = 10000.0                 # the position vector's frequencies are base^(-2i / width)
MIXERS = ("gla", "latent_attention", "wkv")


def _int(d, key: str, where: str, minimum: int = 1) -> int:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json: {where}{key!r} must be an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json: {where}{key!r} must be at least {minimum}, got {v}")
    return v


def _num(d, key: str, where: str) -> float:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}{key!r} must be a number, got {v!r}")
    return float(v)


def _obj(d, key: str, where: str) -> dict:
    v = d.get(key) if isinstance(d, dict) else None
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: {where}{key!r} must be an object, got {v!r}")
    return v


def _opt_int(d, key: str, where: str) -> Optional[int]:
    return None if d.get(key) is None else _int(d, key, where)


@dataclass(frozen=True)
class NupovikConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float
    layers: Tuple[object, ...]                 # one ParallelBlockSpec a layer
    loop: Optional[Tuple[int, int, int]]       # (start, stop, times)
    raw: dict

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, raw: dict) -> "NupovikConfig":
        vocab = _int(raw, "vocab", "")
        width = _int(raw, "width", "")
        eps = _num(_obj(raw, "norm", ""), "eps", "norm.")
        if not eps >= 0.0:
            raise ConfigError(f"config.json: norm.eps={eps} must not be negative")
        scale = 1.0 if raw.get("logit_scale") is None else _num(raw, "logit_scale", "")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        norm = cls._norm(width, eps)
        blocks = tuple(cls._block(i, L, width, eps, norm) for i, L in enumerate(layers))
        loop = None
        if raw.get("loop") is not None:
            lp = _obj(raw, "loop", "")
            a, b = _int(lp, "start", "loop.", 0), _int(lp, "stop", "loop.", 0)
            times = _int(lp, "times", "loop.", 1)
            if not (a <= b <= len(blocks)):
                raise ConfigError(f"config.json: loop {a}..{b} does not lie within the "
                                  f"{len(blocks)} layers")
            loop = (a, b, times)
        return cls(vocab, width, eps, scale, blocks, loop, copy.deepcopy(raw))

    @staticmethod
    def _norm(width: int, eps: float) -> LayerNormSpec:
        # x / sqrt(mean x^2 + eps) * w: not centred, no bias; the gain's tensor is the prefix itself
        return LayerNormSpec(width, eps, centred=False, weight_name="", bias_name=None)

    @staticmethod
    def _block(i: int, L, width: int, eps: float, norm: LayerNormSpec) -> ParallelBlockSpec:
        where = f"layers[{i}]."
        if not isinstance(L, dict):
            raise ConfigError(f"config.json: layers[{i}] must be an object")
        kind = L.get("type")
        if kind not in MIXERS:
            raise ConfigError(f"config.json: {where}type={kind!r}: the mixers of this design "
                              f"are {', '.join(repr(m) for m in MIXERS)}")
        m = _obj(L, "mixer", where)
        mw = where + "mixer."
        if kind == "gla":
            tau = _num(m, "tau", mw)
            if not tau > 0.0:
                raise ConfigError(f"config.json: {mw}tau={tau} must be positive")
            mixer = GatedLinearAttentionSpec(
                hidden_size=width, n_heads=_int(m, "heads", mw), head_dim=_int(m, "dim", mw),
                value_dim=_int(m, "vdim", mw), decay_rank=_opt_int(m, "decay_rank", mw),
                tau=tau, norm_eps=eps)
        elif kind == "wkv":
            mixer = TokenShiftRecurrenceSpec(
                hidden_size=width, n_heads=_int(m, "heads", mw), head_dim=_int(m, "dim", mw),
                decay_rank=_opt_int(m, "decay_rank", mw), norm_eps=eps)
        else:
            mixer = LatentAttentionSpec(
                hidden_size=width, n_heads=_int(m, "heads", mw), head_dim=_int(m, "dim", mw),
                rot_dim=0, value_dim=_int(m, "vdim", mw), q_rank=None,
                kv_rank=_int(m, "kv_rank", mw), scale=_num(m, "scale", mw), norm_eps=eps,
                head_gate=True, uq_name="q", dkv_name="dkv", dkv_norm_name="dkv.norm",
                uk_name="uk", uv_name="uv", gate_name="g", o_name="o")
        ff = NupovikConfig._feed_forward(L.get("mlp"), where + "mlp.", width)
        return ParallelBlockSpec(mixer=mixer, feed_forward=ff, mixer_norm=norm,
                                 ff_norm=norm if ff is not None else None, mixer_prefix="mix.",
                                 ff_prefix="mlp.", mixer_norm_prefix="norm1",
                                 ff_norm_prefix="norm2")

    @staticmethod
    def _feed_forward(f, fw: str, width: int):
        if f is None:
            return None
        kind = f.get("kind") if isinstance(f, dict) else f
        if kind == "dense":
            return DenseMlpSpec(width, _int(f, "ff", fw), FF_ACTIVATION, up_name="up",
                                down_name="down")
        if kind != "moe":
            raise ConfigError(f"config.json: {fw}kind={kind!r}: the feed-forwards of this design "
                              "are 'dense' and 'moe'")
        r = _obj(f, "router", fw)
        rw = fw + "router."
        experts, top = _int(r, "experts", rw), _int(r, "top", rw)
        if top > experts:
            raise ConfigError(f"config.json: {rw}top={top} of {experts} experts")
        groups = None
        if r.get("groups") is not None:
            g = _obj(r, "groups", rw)
            count, keep = _int(g, "count", rw + "groups."), _int(g, "keep", rw + "groups.")
            if experts % count != 0 or keep > count or top > keep * (experts // count):
                raise ConfigError(f"config.json: {rw}groups: {experts} experts in {count} equal "
                                  f"groups, {keep} kept, {top} chosen do not fit together")
            groups = (count, keep)
        return MoeSpec(hidden_size=width, n_experts=experts, top_k=top,
                       expert=PlainExpertSpec(_int(_obj(f, "expert", fw), "ff", fw + "expert."),
                                              FF_ACTIVATION),
                       scoring="sigmoid", correction_name="correction", groups=groups,
                       router_name="router", expert_prefix="e{}.", up_name="up", down_name="down")

    def to_dict(self) -> dict:
        return copy.deepcopy(self.raw)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def model_type(self) -> str:
        return "nupovik"

    # ------------------------------------------------------------------ the model's parts
    def layer_order(self) -> Tuple[Tuple[int, bool], ...]:
        """(layer, whether a pass begins before it) for every run, in order."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, False) for i in range(n))
        a, b, times = self.loop
        runs = [(i, False) for i in range(a)]
        for _ in range(times):
            runs += [(i, i == a) for i in range(a, b)]
        return tuple(runs + [(i, False) for i in range(b, n)])

    def model_spec(self) -> ModelSpec:
        """Every run of a layer, a repeated one too, has a cache or state of its own."""
        order = self.layer_order()
        return ModelSpec(
            vocab_size=self.vocab, hidden_size=self.width, max_positions=MAX_POSITIONS,
            layers=self.layers,
            schedule=tuple(ScheduleEntry(i, reentry=begins) for i, begins in order),
            final_norm=self._norm(self.width, self.norm_eps), tie_word_embeddings=False,
            embed_name="embed", final_norm_prefix="final.norm", head_name="head",
            layer_prefix="l{}.", logit_scale=self.logit_scale,
            sinusoidal_positions=SinusoidalPositionSpec(POSITION_BASE),
            reentry_name="loop.in" if self.loop is not None else None)


register_architecture("Nupovik", NupovikConfig)
