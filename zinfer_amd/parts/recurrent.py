from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.specs import GatedLinearAttentionSpec, TokenShiftRecurrenceSpec
from ..errors import ConfigError
from .base import Mixer, StateNeed, TensorDecl, register_part
from .linear import Linear, place_gain, place_matrix


def _check_heads(n_heads: int, head_dim: int, value_dim: int) -> None:
    if min(n_heads, head_dim, value_dim) < 1:
        raise ConfigError("InvalidDimensions: heads and head sizes must be at least 1")
    if head_dim > ops.RECURRENCE_MAX_KEY_DIM:
        raise ConfigError(f"InvalidHeadDim: dim={head_dim}: the recurrence kernel takes key sizes "
                          f"up to {ops.RECURRENCE_MAX_KEY_DIM}")


def _middle(tensors, down_name: str, up_name: str, rank) -> int:
    """The width of a decay's narrow middle, from the two matrices around it."""
    have = tensors[down_name].shape[0]
    if tensors[up_name].shape[1] != have or (rank is not None and rank != have):
        raise ConfigError(f"{down_name} {tuple(tensors[down_name].shape)} and {up_name} "
                          f"{tuple(tensors[up_name].shape)} do not share a middle"
                          + (f" of {rank}" if rank is not None else ""))
    return have


class GatedLinearAttention(Mixer):
    """The mixer of ``GatedLinearAttentionSpec``: q, k, v and the output gate come from one
    product over the stacked matrices (each output keeps its own dot product); the decay's
    numbers z = W_a2 (W_a1 h) leave their product as 32-bit numbers, and the recurrence kernel
    turns them into decays, walks the step's tokens (long portions in spans side by side) and
    keeps every request's matrices in its state slot (32-bit); one more kernel norms each head,
    applies the gain and the gate."""
    graph_safe = True
    kernel_modules = ("gemm", "recurrent")

    def __init__(self, spec: GatedLinearAttentionSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        s = spec
        _check_heads(s.n_heads, s.head_dim, s.value_dim)
        if not s.tau > 0.0:
            raise ConfigError(f"tau={s.tau} must be positive")
        self.qk_width = s.n_heads * s.head_dim
        self.v_width = s.n_heads * s.value_dim
        self.q_scale = float(s.q_scale) if s.q_scale is not None else s.head_dim ** -0.5
        self.state_size = ops.recurrence_state_size(s.n_heads, s.head_dim, s.value_dim)

    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        return {p + s.q_name: TensorDecl((self.qk_width, s.hidden_size)),
                p + s.k_name: TensorDecl((self.qk_width, s.hidden_size)),
                p + s.v_name: TensorDecl((self.v_width, s.hidden_size)),
                p + s.gate_name: TensorDecl((self.v_width, s.hidden_size)),
                p + s.o_name: TensorDecl((s.hidden_size, self.v_width)),
                p + s.norm_name: TensorDecl((s.value_dim,), init="gain"),
                p + s.decay_down_name: TensorDecl((s.decay_rank, s.hidden_size)),
                p + s.decay_up_name: TensorDecl((self.qk_width, s.decay_rank)),
                p + s.decay_bias_name: TensorDecl((self.qk_width,))}

    def bind(self, tensors) -> None:
        s, p = self.spec, self.prefix
        rows = [tensors[p + n] for n in (s.q_name, s.k_name, s.v_name, s.gate_name)]
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        self.proj = Linear(place_matrix(torch.cat(rows, dim=0), self.ctx))
        self.o = Linear(place_matrix(tensors[p + s.o_name], self.ctx))
        self.rank = _middle(tensors, p + s.decay_down_name, p + s.decay_up_name, s.decay_rank)
        self.decay_down = Linear(place_matrix(tensors[p + s.decay_down_name], self.ctx))
        self.decay_up = Linear(place_matrix(tensors[p + s.decay_up_name], self.ctx))
        self.decay_bias = place_gain(tensors[p + s.decay_bias_name], self.ctx)
        self.gain = place_gain(tensors[p + s.norm_name], self.ctx)

    def cache_need(self):
        return StateNeed((self.state_size,), torch.float32)

    def forward(self, h, residual, step, cache) -> None:
        s = self.spec
        T = h.shape[0]
        act = self.ctx.act_dtype
        if hasattr(h, "materialize"):
            h = h.materialize()
        QK, V = self.qk_width, self.v_width
        proj = step.scratch("rec_proj", (T, self.proj.out_features), act)
        self.proj.forward(h, proj)
        low = step.scratch("rec_decay_low", (T, self.rank), act)
        self.decay_down.forward(h, low)
        z = step.scratch("rec_decay_z", (T, QK), torch.float32)
        self.decay_up.forward(low, z)
        o = step.scratch("rec_out", (T, V), torch.float32)
        ops.decay_recurrence(proj[:, :QK], proj[:, QK:2 * QK], proj[:, 2 * QK:2 * QK + V], z,
                             self.decay_bias, None, cache.state, step.state_slots, step.q_start,
                             o, s.n_heads, s.head_dim, s.value_dim, "sigmoid_root",
                             tau=float(s.tau), q_scale=self.q_scale, max_q_len=step.max_q_len)
        mixed = step.scratch("rec_mixed", (T, V), act)
        ops.head_norm_gate(o, self.gain, proj[:, 2 * QK + V:], mixed, s.n_heads,
                           float(s.norm_eps))
        self.o.forward(mixed, residual, accumulate=True, step=step)


class TokenShiftRecurrence(Mixer):
    """The mixer of ``TokenShiftRecurrenceSpec``.  One kernel blends every row with the row
    before it, five ways (the row before a portion's first comes from the request's state,
    which takes the portion's last); five products read their own blend; the decay's numbers
    pass a tanh between their two products and leave the second as 32-bit numbers; the
    recurrence kernel reads the state before the token's own outer product joins it and adds
    that product weighted by u.  The state slot holds the matrices and, behind them, the last
    row (32-bit)."""
    graph_safe = True
    kernel_modules = ("elementwise", "gemm", "recurrent")
    MIXES = "rkvgw"

    def __init__(self, spec: TokenShiftRecurrenceSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        s = spec
        _check_heads(s.n_heads, s.head_dim, s.head_dim)
        self.width = s.n_heads * s.head_dim
        self.matrix_size = ops.recurrence_state_size(s.n_heads, s.head_dim, s.head_dim)

    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        d = {p + s.mix_name.format(m): TensorDecl((s.hidden_size,)) for m in self.MIXES}
        for n in (s.r_name, s.k_name, s.v_name, s.gate_name):
            d[p + n] = TensorDecl((self.width, s.hidden_size))
        d[p + s.decay_down_name] = TensorDecl((s.decay_rank, s.hidden_size))
        d[p + s.decay_up_name] = TensorDecl((self.width, s.decay_rank))
        d[p + s.decay_bias_name] = TensorDecl((self.width,))
        d[p + s.bonus_name] = TensorDecl((s.n_heads, s.head_dim))
        d[p + s.norm_name] = TensorDecl((self.width,), init="gain")
        d[p + s.o_name] = TensorDecl((s.hidden_size, self.width))
        return d

    def bind(self, tensors) -> None:
        s, p = self.spec, self.prefix
        self.mu = torch.stack([tensors[p + s.mix_name.format(m)].to(torch.float32)
                               for m in self.MIXES]).to(self.ctx.device).contiguous()
        self.products = [Linear(place_matrix(tensors[p + n], self.ctx))
                         for n in (s.r_name, s.k_name, s.v_name, s.gate_name)]
        self.rank = _middle(tensors, p + s.decay_down_name, p + s.decay_up_name, s.decay_rank)
        self.decay_down = Linear(place_matrix(tensors[p + s.decay_down_name], self.ctx))
        self.decay_up = Linear(place_matrix(tensors[p + s.decay_up_name], self.ctx))
        self.decay_bias = place_gain(tensors[p + s.decay_bias_name], self.ctx)
        self.bonus = place_gain(tensors[p + s.bonus_name].reshape(-1), self.ctx)
        self.gain = place_gain(tensors[p + s.norm_name], self.ctx)
        self.o = Linear(place_matrix(tensors[p + s.o_name], self.ctx))

    def cache_need(self):
        # the matrices, then the last row the mixer read
        return StateNeed((self.matrix_size + self.spec.hidden_size,), torch.float32)

    def forward(self, h, residual, step, cache) -> None:
        s = self.spec
        T = h.shape[0]
        act = self.ctx.act_dtype
        if hasattr(h, "materialize"):
            h = h.materialize()
        mixes = step.scratch("shift_mixes", (len(self.MIXES), T, s.hidden_size), act)
        ops.token_shift_mix(h, self.mu, cache.state, self.matrix_size, step.state_slots,
                            step.seq_index, step.q_start, mixes)
        rkvg = step.scratch("shift_rkvg", (4, T, self.width), act)
        for i, product in enumerate(self.products):
            product.forward(mixes[i], rkvg[i])
        low = step.scratch("rec_decay_low", (T, self.rank), act)
        self.decay_down.forward(mixes[4], low)
        ops.activation(low, low, "tanh")
        z = step.scratch("rec_decay_z", (T, self.width), torch.float32)
        self.decay_up.forward(low, z)
        o = step.scratch("rec_out", (T, self.width), torch.float32)
        ops.decay_recurrence(rkvg[0], rkvg[1], rkvg[2], z, self.decay_bias, self.bonus,
                             cache.state, step.state_slots, step.q_start, o, s.n_heads,
                             s.head_dim, s.head_dim, "double_exp", max_q_len=step.max_q_len)
        mixed = step.scratch("rec_mixed", (T, self.width), act)
        ops.head_norm_gate(o, self.gain, rkvg[3], mixed, s.n_heads, float(s.norm_eps))
        self.o.forward(mixed, residual, accumulate=True, step=step)


register_part("mixer", GatedLinearAttentionSpec, GatedLinearAttention)
register_part("mixer", TokenShiftRecurrenceSpec, TokenShiftRecurrence)
