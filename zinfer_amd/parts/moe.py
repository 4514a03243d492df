from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.specs import MoeSpec, PlainExpertSpec
from ..errors import ConfigError
from .base import FeedForward, TensorDecl, register_part
from .linear import Linear, place_gain, place_matrix


class MoeFeedForward(FeedForward):
    """A mixture of gated experts: the router's logits z = W_r h (+ b_r) are formed in 32-bit,
    the ``top_k`` largest choose a token's experts, the soft-max over the chosen logits alone
    weighs them; an expert is W_down act(W_gate h, W_up h) with the clamped, gated activation
    of ``GatedExpertSpec``; an optional shared expert runs for every token and is added with
    weight 1; with ``scoring`` "sigmoid" the router is the one ``MoeSpec`` describes (sigmoid
    scores, a correction that enters the choice only, groups of experts), and a
    ``PlainExpertSpec`` is an expert without a gate, W_down act(W_up h).  The experts' matrices
    are stacked at load (gate rows above up rows, expert by expert) so that the kernels find an
    expert by its number.  Every token's sum runs over its
    chosen experts in the order the router ranked them, then the shared one.  The other options
    of ``MoeSpec`` (a soft-max over all outputs, a group's mark, weights that are not normalized,
    router outputs without an expert, a gate a token on the shared expert) are parameters of the
    same kernels."""
    graph_safe = True
    stores_output = True
    kernel_modules = ("gemm", "moe")

    def __init__(self, spec: MoeSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        self.outputs = spec.n_experts + spec.n_identity      # what the router chooses among
        if not (1 <= spec.top_k <= self.outputs <= ops.MOE_MAX_EXPERTS - 1
                and spec.n_experts >= 1 and spec.n_identity >= 0):
            raise ConfigError(f"a mixture of {spec.n_experts} experts (and {spec.n_identity} "
                              f"outputs without one) with {spec.top_k} a token: 1 <= top <= "
                              f"outputs < {ops.MOE_MAX_EXPERTS}")
        self.plain = isinstance(spec.expert, PlainExpertSpec)
        if self.plain and spec.expert.activation not in ops.ACTIVATIONS:
            raise ConfigError(f"activation {spec.expert.activation!r}: known are "
                              f"{sorted(ops.ACTIVATIONS)}")
        if spec.scoring not in ops.ROUTER_SCORINGS:
            raise ConfigError(f"router scoring {spec.scoring!r}: known are "
                              f"{sorted(ops.ROUTER_SCORINGS)}")
        if spec.scoring == "softmax" and (spec.correction_name is not None
                                          or spec.groups is not None or not spec.normalize
                                          or spec.shared_gate_name is not None):
            raise ConfigError("a correction of the choice, groups of experts, weights that are "
                              "not normalized and a gate on the shared expert belong to the "
                              "routers that score every expert")
        if spec.groups is not None:
            count, keep = spec.groups
            if not (0 < keep <= count <= self.outputs and self.outputs % count == 0
                    and spec.top_k <= keep * (self.outputs // count)):
                raise ConfigError(f"{self.outputs} router outputs in {count} equal groups, {keep} "
                                  f"kept, {spec.top_k} chosen do not fit together")
        if spec.group_mark not in (1, 2):
            raise ConfigError(f"a group is marked by its largest or its two largest choice "
                              f"scores, not by {spec.group_mark}")
        if self.plain and spec.shared is not None:
            raise ConfigError("a shared expert is a gated one")
        if spec.shared_gate_name is not None and spec.shared is None:
            raise ConfigError("a gate on the shared expert without a shared expert")

    def _expert_names(self, prefix: str):
        s = self.spec
        return prefix + s.gate_name, prefix + s.up_name, prefix + s.down_name

    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        d = {p + s.router_name: TensorDecl((self.outputs, s.hidden_size))}
        if s.router_bias:
            d[p + s.router_bias_name] = TensorDecl((self.outputs,))
        if s.correction_name is not None:
            d[p + s.correction_name] = TensorDecl((self.outputs,))
        if s.shared_gate_name is not None:
            d[p + s.shared_prefix + s.shared_gate_name] = TensorDecl((1, s.hidden_size))
        if self.plain:
            for e in range(s.n_experts):
                prefix = p + s.expert_prefix.format(e)
                d[prefix + s.up_name] = TensorDecl((s.expert.intermediate_size, s.hidden_size))
                d[prefix + s.down_name] = TensorDecl((s.hidden_size, s.expert.intermediate_size))
            return d
        groups = [(p + s.expert_prefix.format(e), s.expert) for e in range(s.n_experts)]
        if s.shared is not None:
            groups.append((p + s.shared_prefix, s.shared))
        for prefix, ex in groups:
            g, u, dn = self._expert_names(prefix)
            d[g] = TensorDecl((ex.intermediate_size, s.hidden_size))
            d[u] = TensorDecl((ex.intermediate_size, s.hidden_size))
            d[dn] = TensorDecl((s.hidden_size, ex.intermediate_size))
        return d

    def _stack(self, tensors, prefixes):
        """(gate_up [E, 2 ff, W], down [E, W, ff]) of the experts under ``prefixes``, on the
        device in the compute dtype, built expert by expert."""
        gate_up, down = [], []
        for prefix in prefixes:
            gn, un, dnn = self._expert_names(prefix)
            u, dn = tensors[un], tensors[dnn]
            if self.plain:                  # no gate: the up rows alone
                gate_up.append(place_matrix(u, self.ctx))
            else:
                g = tensors[gn]
                if g.dtype != u.dtype:
                    g, u = g.float(), u.float()
                gate_up.append(place_matrix(torch.cat([g, u], dim=0), self.ctx))
            down.append(place_matrix(dn, self.ctx))
        dtypes = {t.dtype for t in gate_up + down}
        if len(dtypes) > 1:
            gate_up, down = [t.float() for t in gate_up], [t.float() for t in down]
        return torch.stack(gate_up).contiguous(), torch.stack(down).contiguous()

    def bind(self, tensors) -> None:
        s, p = self.spec, self.prefix
        # the router's logits are 32-bit numbers: its matrix is widened once
        router = tensors[p + s.router_name].to(torch.float32)
        if s.shared_gate_name is not None:
            # the shared expert's gate is one more row of the router's matrix: its number a
            # token is formed in 32-bit by the same kernel
            router = torch.cat([router, tensors[p + s.shared_prefix + s.shared_gate_name]
                                .to(torch.float32).reshape(1, -1)], dim=0)
        self.router = place_gain(router, self.ctx)
        self.router_bias = place_gain(tensors[p + s.router_bias_name], self.ctx) \
            if s.router_bias else None
        self.correction = place_gain(tensors[p + s.correction_name], self.ctx) \
            if s.correction_name is not None else None
        self.gate_up, self.down = self._stack(
            tensors, [p + s.expert_prefix.format(e) for e in range(s.n_experts)])
        if s.shared is not None:
            # the expert every token uses is two plain products around the activation
            gu, dn = self._stack(tensors, [p + s.shared_prefix])
            self.shared_gate_up, self.shared_down = Linear(gu[0]), Linear(dn[0])

    def forward(self, h, residual, step, accumulate: bool = True) -> None:
        s = self.spec
        if hasattr(h, "materialize"):
            h = h.materialize()
        T = h.shape[0]
        dtype = self.gate_up.dtype
        if h.dtype != dtype:
            raise ConfigError(f"the experts are held in {dtype}, the activations in {h.dtype}")
        ids = step.scratch("moe_ids", (T, s.top_k), torch.int32)
        share = step.scratch("moe_share", (T, s.top_k), torch.float32)
        shared_gate = step.scratch("moe_shared_gate", (T, 1), torch.float32) \
            if s.shared_gate_name is not None else None
        ops.moe_route(h, self.router, self.router_bias, ids, share, scoring=s.scoring,
                      correction=self.correction, groups=s.groups, group_mark=s.group_mark,
                      normalize=s.normalize, weight_scale=float(s.weight_scale),
                      extra=shared_gate)
        ex = s.expert
        y = step.scratch("moe_act", (T, s.top_k, ex.intermediate_size), dtype)
        if self.plain:
            ops.moe_experts(h, self.gate_up, self.down, ids, share, y, residual, 0.0, 1.0, 0.0,
                            add=accumulate, act=ex.activation, n_identity=s.n_identity)
        else:
            ops.moe_experts(h, self.gate_up, self.down, ids, share, y, residual,
                            float(ex.limit or 0.0), float(ex.alpha), float(ex.shift),
                            add=accumulate, n_identity=s.n_identity)
        if s.shared is not None:
            sh = s.shared
            gu = step.scratch("moe_shared_gate_up", (T, 2 * sh.intermediate_size), dtype)
            self.shared_gate_up.forward(h, gu)
            ys = step.scratch("moe_shared_act", (T, sh.intermediate_size), dtype)
            ops.gated_act(gu, ys, float(sh.limit or 0.0), float(sh.alpha), float(sh.shift),
                          row_factor=shared_gate[:, 0] if shared_gate is not None else None)
            self.shared_down.forward(ys, residual, accumulate=True)


register_part("feed_forward", MoeSpec, MoeFeedForward)
