from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.specs import GatedDeltaRuleSpec, ParallelMixerSpec
from ..errors import ConfigError
from .base import KVNeed, Mixer, StateNeed, TensorDecl, build_part, register_part
from .linear import Linear, place_gain, place_matrix


class GatedDeltaRule(Mixer):
    """The mixer of ``GatedDeltaRuleSpec``.  q, k, v and the output gate come from one product
    over the stacked matrices; the decays' and step sizes' numbers from a second one that leaves
    its accumulators as 32-bit numbers.  One kernel runs the short convolutions with their silu
    from the product's rows and the request's last rows, makes q and k unit vectors and scales
    q, all in 32-bit; the recurrence kernel forms decay and step size a head and token and walks
    the step's tokens; one more kernel norms each head and applies gain and gate.  A request's
    state slot holds the matrices and, behind them, the convolutions' last rows (32-bit)."""
    graph_safe = True
    stores_output = True
    kernel_modules = ("gemm", "delta", "recurrent")

    def __init__(self, spec: GatedDeltaRuleSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        s = spec
        if min(s.n_heads, s.n_kv_heads, s.head_dim, s.value_dim, s.conv_taps) < 1:
            raise ConfigError("InvalidDimensions: heads, head sizes and taps must be at least 1")
        if s.n_heads % s.n_kv_heads != 0:
            raise ConfigError(f"InvalidGrouping: {s.n_heads} value heads, {s.n_kv_heads} q/k heads")
        if s.head_dim > ops.DELTA_MAX_KEY_DIM:
            raise ConfigError(f"InvalidHeadDim: dim={s.head_dim}: the delta rule's kernel takes "
                              f"key sizes up to {ops.DELTA_MAX_KEY_DIM}")
        if s.conv_taps > ops.SHORT_CONV_MAX_TAPS:
            raise ConfigError(f"conv={s.conv_taps}: the convolution kernel takes up to "
                              f"{ops.SHORT_CONV_MAX_TAPS} taps")
        self.qk_width = s.n_kv_heads * s.head_dim
        self.v_width = s.n_heads * s.value_dim
        self.conv_width = 2 * self.qk_width + self.v_width
        self.q_scale = float(s.q_scale) if s.q_scale is not None else s.head_dim ** -0.5
        # the matrices (rounded up to whole 16 bytes), then the convolutions' last rows
        self.matrix_size = (ops.delta_state_size(s.n_heads, s.head_dim, s.value_dim) + 3) // 4 * 4
        self.state_size = (self.matrix_size + (s.conv_taps - 1) * self.conv_width + 3) // 4 * 4
        self.output_scale = 1.0

    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        d = {}
        for name, width in ((s.q_name, self.qk_width), (s.k_name, self.qk_width),
                            (s.v_name, self.v_width)):
            d[p + name] = TensorDecl((width, s.hidden_size))
            d[p + name + s.conv_suffix] = TensorDecl((width, s.conv_taps))
        d[p + s.gate_name] = TensorDecl((self.v_width, s.hidden_size))
        d[p + s.beta_name] = TensorDecl((s.n_heads, s.hidden_size))
        d[p + s.decay_name] = TensorDecl((s.n_heads, s.hidden_size))
        d[p + s.decay_log_name] = TensorDecl((s.n_heads,))
        d[p + s.decay_bias_name] = TensorDecl((s.n_heads,))
        d[p + s.norm_name] = TensorDecl((s.value_dim,), init="gain")
        d[p + s.o_name] = TensorDecl((s.hidden_size, self.v_width))
        return d

    def bind(self, tensors) -> None:
        s, p = self.spec, self.prefix
        rows = [tensors[p + n] for n in (s.q_name, s.k_name, s.v_name, s.gate_name)]
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        self.proj = Linear(place_matrix(torch.cat(rows, dim=0), self.ctx))
        small = [tensors[p + s.decay_name], tensors[p + s.beta_name]]
        if len({t.dtype for t in small}) > 1:
            small = [t.float() for t in small]
        self.decay_beta = Linear(place_matrix(torch.cat(small, dim=0), self.ctx))
        self.taps = place_gain(torch.cat([tensors[p + n + s.conv_suffix].to(torch.float32)
                                          for n in (s.q_name, s.k_name, s.v_name)], dim=0),
                               self.ctx)
        self.decay_log = place_gain(tensors[p + s.decay_log_name], self.ctx)
        self.decay_bias = place_gain(tensors[p + s.decay_bias_name], self.ctx)
        self.gain = place_gain(tensors[p + s.norm_name], self.ctx)
        self._gain = self.gain
        self.o = Linear(place_matrix(tensors[p + s.o_name], self.ctx))
        self.set_output_scale(self.output_scale)

    def set_output_scale(self, scale: float) -> bool:
        """The mixer's output times ``scale``: the head norm's gain carries it (in 32-bit, ahead
        of the one rounding of the normed heads)."""
        self.output_scale = float(scale)
        if hasattr(self, "_gain"):
            self.gain = self._gain if scale == 1.0 else (self._gain * float(scale)).contiguous()
        return True

    def cache_need(self):
        return StateNeed((self.state_size,), torch.float32)

    def forward(self, h, residual, step, cache, accumulate: bool = True) -> None:
        s = self.spec
        T = h.shape[0]
        act = self.ctx.act_dtype
        if hasattr(h, "materialize"):
            h = h.materialize()
        QK, V = self.qk_width, self.v_width
        proj = step.scratch("delta_proj", (T, self.proj.out_features), act)
        self.proj.forward(h, proj)
        ab = step.scratch("delta_decay_beta", (T, 2 * s.n_heads), torch.float32)
        self.decay_beta.forward(h, ab)
        qkv = step.scratch("delta_qkv", (T, self.conv_width), torch.float32)
        ops.short_conv(proj, self.taps, cache.state, self.matrix_size, step.state_slots,
                       step.seq_index, step.q_start, qkv, unit_heads=2 * s.n_kv_heads,
                       head_dim=s.head_dim, scaled_heads=s.n_kv_heads, scale=self.q_scale,
                       unit_eps=float(s.unit_eps), single_tokens=step.max_q_len == 1)
        o = step.scratch("delta_out", (T, V), torch.float32)
        ops.delta_recurrence(qkv, 0, QK, 2 * QK, ab, self.decay_log, self.decay_bias, cache.state,
                             step.state_slots, step.q_start, o, s.n_heads, s.n_kv_heads,
                             s.head_dim, s.value_dim)
        mixed = step.scratch("delta_mixed", (T, V), act)
        ops.head_norm_gate(o, self.gain, proj[:, 2 * QK + V:], mixed, s.n_heads,
                           float(s.norm_eps))
        self.o.forward(mixed, residual, accumulate=accumulate, step=step if accumulate else None)


class ParallelMixer(Mixer):
    """Two mixers side by side on the same input (``ParallelMixerSpec``): each has its tensors,
    its cache or state (the run's cache view holds both) and its kernels.  A mixer that can
    carry a factor on its output itself (``set_output_scale``) does; the sum then is the first
    one's output stored and the second one's added in 32-bit.  Otherwise both store into
    branches of their own (``forward_branches``) that whoever adds them weighs."""
    stores_output = True

    def __init__(self, spec: ParallelMixerSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        self.left = build_part("mixer", spec.left, ctx, prefix + spec.left_prefix)
        self.right = build_part("mixer", spec.right, ctx, prefix + spec.right_prefix)
        self.parts = (self.left, self.right)
        for part in self.parts:
            if not getattr(part, "stores_output", False):
                raise ConfigError(f"{type(part).__name__} cannot stand beside another mixer: it "
                                  "only adds into the residual stream")
        self.graph_safe = all(p.graph_safe for p in self.parts)
        self.kernel_modules = tuple(sorted({m for p in self.parts for m in p.kernel_modules}))
        needs = [n for n in (p.cache_need() for p in self.parts) if n is not None]
        if sum(isinstance(n, KVNeed) for n in needs) > 1 \
                or sum(isinstance(n, StateNeed) for n in needs) > 1:
            raise ConfigError("two mixers side by side may bring one cache of keys and values "
                              "and one state of fixed size between them")
        self._needs = tuple(needs)
        # factors the mixers carry themselves; what is left is applied where the branches meet
        self.factors = []
        for part, scale in ((self.left, spec.left_scale), (self.right, spec.right_scale)):
            carried = scale == 1.0 or (hasattr(part, "set_output_scale")
                                       and part.set_output_scale(float(scale)))
            self.factors.append(1.0 if carried else float(scale))

    def declare(self) -> Dict[str, TensorDecl]:
        d: Dict[str, TensorDecl] = {}
        for part in self.parts:
            d.update(part.declare())
        return d

    def bind(self, tensors) -> None:
        for part in self.parts:
            part.bind(tensors)

    def cache_need(self):
        if not self._needs:
            return None
        return self._needs[0] if len(self._needs) == 1 else self._needs

    def accept_cache(self, cache) -> None:
        for part in self.parts:
            part.accept_cache(cache)

    def hint_providers(self):
        return [q for p in self.parts for q in p.hint_providers()]

    def forward_branches(self, h, step, cache):
        """[(float32 [T, W] branch, factor)] whose weighted sum is the mixer's output."""
        if hasattr(h, "materialize"):
            h = h.materialize()
        if self.factors == [1.0, 1.0]:
            y = step.scratch("branch", (h.shape[0], self.spec.left.hidden_size), torch.float32)
            self.left.forward(h, y, step, cache, accumulate=False)
            self.right.forward(h, y, step, cache, accumulate=True)
            return [(y, 1.0)]
        out = []
        for name, part, factor in (("branch", self.left, self.factors[0]),
                                   ("branch_right", self.right, self.factors[1])):
            y = step.scratch(name, (h.shape[0], self.spec.left.hidden_size), torch.float32)
            part.forward(h, y, step, cache, accumulate=False)
            out.append((y, factor))
        return out

    def forward(self, h, residual, step, cache, accumulate: bool = True) -> None:
        if self.factors != [1.0, 1.0]:
            raise ConfigError("mixers side by side with factors of their own run inside a block "
                              "that adds their branches (forward_branches)")
        if hasattr(h, "materialize"):
            h = h.materialize()
        self.left.forward(h, residual, step, cache, accumulate=accumulate)
        self.right.forward(h, residual, step, cache, accumulate=True)


register_part("mixer", GatedDeltaRuleSpec, GatedDeltaRule)
register_part("mixer", ParallelMixerSpec, ParallelMixer)
