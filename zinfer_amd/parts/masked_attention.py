from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.specs import LatentAttentionSpec, MaskedGqaAttentionSpec
from ..errors import ConfigError
from .base import KVNeed, Mixer, TensorDecl, register_part
from .linear import Linear, place_gain, place_matrix


def _frequencies(rotary, ctx):
    """A rotation's frequencies as the kernels take them: 32-bit numbers on the device."""
    if rotary is None:
        return None
    return torch.tensor(rotary.frequencies, dtype=torch.float64).to(torch.float32).to(ctx.device)


def _check_mask(spec) -> None:
    for name in ("window", "chunk"):
        v = getattr(spec, name)
        if v is not None and v < 1:
            raise ConfigError(f"{name}={v} must be at least 1")


class MaskedGqaAttention(Mixer):
    """Causal grouped-query attention with the options of ``MaskedGqaAttentionSpec``: q, k, v
    and the per-head gate come from one product over the stacked matrices (each output keeps
    its own dot product); one kernel norms q and k over their whole projections, rotates the
    leading elements of every head by the token's position, and stores the token's key and
    value rows in the cache; the attention kernel caps the scores, keeps to the query's chunk
    or window, counts the head's sink in the denominator and multiplies by the head's gate.
    Norms, angles, scores, weights and their sums are 32-bit in both dtypes."""
    graph_safe = True
    stores_output = True
    kernel_modules = ("gemm", "masked_attention")

    def __init__(self, spec: MaskedGqaAttentionSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        s = spec
        if s.n_heads < 1 or s.n_kv_heads < 1 or s.head_dim < 1 or s.value_dim < 1:
            raise ConfigError("InvalidDimensions: heads and head sizes must be at least 1")
        if s.n_heads % s.n_kv_heads != 0:
            raise ConfigError(f"InvalidGrouping: {s.n_heads} query heads, {s.n_kv_heads} kv heads")
        if s.value_dim > ops.MAX_HEAD_DIM:
            raise ConfigError(f"InvalidHeadDim: value_dim={s.value_dim}: the attention kernels "
                              f"take value sizes up to {ops.MAX_HEAD_DIM}")
        if s.rotary is not None and not (0 < s.rotary.dims <= s.head_dim and s.rotary.dims % 2 == 0
                                         and len(s.rotary.frequencies) == s.rotary.dims // 2):
            raise ConfigError(f"a rotation of {s.rotary.dims} elements does not fit heads of "
                              f"{s.head_dim}")
        _check_mask(s)
        self.q_width = s.n_heads * s.head_dim
        self.k_width = s.n_kv_heads * s.head_dim
        self.v_width = s.n_kv_heads * s.value_dim
        self.freq = _frequencies(s.rotary, ctx)

    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        d = {p + s.q_name: TensorDecl((self.q_width, s.hidden_size)),
             p + s.k_name: TensorDecl((self.k_width, s.hidden_size)),
             p + s.v_name: TensorDecl((self.v_width, s.hidden_size)),
             p + s.o_name: TensorDecl((s.hidden_size, s.n_heads * s.value_dim))}
        if s.qk_norm_eps is not None:
            per = s.qk_norm_per_head
            d[p + s.q_norm_name] = TensorDecl((s.head_dim if per else self.q_width,), init="gain")
            d[p + s.k_norm_name] = TensorDecl((s.head_dim if per else self.k_width,), init="gain")
        if s.bias:
            for name, width in ((s.q_name, self.q_width), (s.k_name, self.k_width),
                                (s.v_name, self.v_width)):
                d[p + name + s.bias_suffix] = TensorDecl((width,))
        if s.sink:
            d[p + s.sink_name] = TensorDecl((s.n_heads,))
        if s.head_gate:
            d[p + s.gate_name] = TensorDecl((s.n_heads, s.hidden_size))
        return d

    def bind(self, tensors) -> None:
        s, p = self.spec, self.prefix
        rows = [tensors[p + s.q_name], tensors[p + s.k_name], tensors[p + s.v_name]]
        if s.head_gate:
            rows.append(tensors[p + s.gate_name])
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        self.proj = Linear(place_matrix(torch.cat(rows, dim=0), self.ctx))
        self.o = Linear(place_matrix(tensors[p + s.o_name], self.ctx))
        self.q_gain = self.k_gain = self.sink = None
        self.q_bias = self.k_bias = self.v_bias = None
        if s.bias:
            self.q_bias, self.k_bias, self.v_bias = (
                place_gain(tensors[p + n + s.bias_suffix], self.ctx)
                for n in (s.q_name, s.k_name, s.v_name))
        if s.qk_norm_eps is not None:
            self.q_gain = place_gain(tensors[p + s.q_norm_name], self.ctx)
            self.k_gain = place_gain(tensors[p + s.k_norm_name], self.ctx)
        if s.sink:
            self.sink = place_gain(tensors[p + s.sink_name], self.ctx)

    def cache_need(self):
        s = self.spec
        return KVNeed(s.n_kv_heads, s.head_dim, s.window, value_dim=s.value_dim, chunk=s.chunk)

    def accept_cache(self, cache) -> None:
        for pool in (cache.k_pool, cache.v_pool):
            if pool is not None and pool.dtype != self.ctx.act_dtype:
                raise ConfigError(f"the cache is kept in the compute dtype ({self.ctx.act_dtype}): "
                                  f"a cache of {pool.dtype} needs a model built with that dtype")

    def forward(self, h, residual, step, cache, accumulate: bool = True) -> None:
        s = self.spec
        T = h.shape[0]
        act = self.ctx.act_dtype
        if hasattr(h, "materialize"):
            h = h.materialize()
        kv = step.kv_tables(cache.group)
        proj = step.scratch("qkvg", (T, self.proj.out_features), act)
        self.proj.forward(h, proj)
        q = step.scratch("q", (T, self.q_width), act)
        eps = float(s.qk_norm_eps) if s.qk_norm_eps is not None else 0.0
        rot = dict(rot_dims=s.rotary.dims, freq=self.freq, mag=s.rotary.magnitude,
                   interleaved=s.rotary.interleaved) if s.rotary is not None else {}
        per = dict(per_head=s.qk_norm_per_head)
        segments = [ops.RowSegment(0, self.q_width, q, gain=self.q_gain, eps=eps, hd=s.head_dim,
                                   bias=self.q_bias, **per, **rot)]
        if cache.writes:
            segments.append(ops.RowSegment(self.q_width, self.k_width, cache.k_pool,
                                           gain=self.k_gain, eps=eps, hd=s.head_dim,
                                           pool_heads=s.n_kv_heads, bias=self.k_bias, **per,
                                           **rot))
            segments.append(ops.RowSegment(self.q_width + self.k_width, self.v_width, cache.v_pool,
                                           hd=s.value_dim, pool_heads=s.n_kv_heads,
                                           bias=self.v_bias))
        ops.project_rows(proj, step.positions, kv.slot_mapping if cache.writes else None,
                         cache.page_size, segments)
        gate = proj[:, self.q_width + self.k_width + self.v_width:] if s.head_gate else None
        attn = step.scratch("attn", (T, s.n_heads * s.value_dim), act)
        ops.attend_masked(q, gate, "head" if s.head_gate else None, cache.k_pool, cache.v_pool,
                          self.sink, kv.block_table, step.q_start, step.ctx_len, step.seq_index,
                          attn, float(s.scale), float(s.softcap or 0.0), int(s.window or 0),
                          int(s.chunk or 0), s.n_heads, s.n_kv_heads, s.head_dim, s.value_dim,
                          cache.page_size, step.max_q_len, step.max_ctx_len)
        self.o.forward(attn, residual, accumulate=accumulate, step=step if accumulate else None)


class LatentAttention(Mixer):
    """Attention over one cached latent row a token (``LatentAttentionSpec``).  The per-head key
    and value matrices never touch the cache's rows: with k_h = U_h c the plain part of a score
    is q_h . (U_h c) = (U_h^T q_h) . c, so the query is taken to the latent's side once a
    token, the attention runs with one kv head whose key row is [latent | rotated part] and
    whose value is the latent itself (the leading columns of the key row), and the head's
    value matrix is applied to the attention's output, with the gate in that product's
    epilogue (a gate an element) or in the attention's own (a gate a head: the value matrix
    is linear, so the gate may stand on either side of it).  The cache holds kv_rank + rot_dim
    numbers a token whatever the number of heads.  Without a query latent (``q_rank`` None) the
    queries come out of the same product as the key latent; without a rotated part
    (``rot_dim`` 0) the key row is the latent alone."""
    graph_safe = True
    stores_output = True
    kernel_modules = ("gemm", "masked_attention")

    def __init__(self, spec: LatentAttentionSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        s = spec
        if min(s.n_heads, s.head_dim, s.value_dim, s.kv_rank) < 1 or s.rot_dim < 0 \
                or (s.q_rank is not None and s.q_rank < 1):
            raise ConfigError("InvalidDimensions: heads, head sizes and ranks must be at least 1")
        if s.kv_rank > ops.MAX_HEAD_DIM:
            raise ConfigError(f"InvalidHeadDim: kv_rank={s.kv_rank}: the attention kernels take "
                              f"latents up to {ops.MAX_HEAD_DIM} wide")
        if s.rotary is not None and not (s.rotary.dims == s.rot_dim and s.rot_dim % 2 == 0
                                         and len(s.rotary.frequencies) == s.rot_dim // 2):
            raise ConfigError(f"the rotated part of a head ({s.rot_dim}) is rotated whole, not "
                              f"{s.rotary.dims} of it")
        if s.element_gate and s.head_gate:
            raise ConfigError("a gate an element or a gate a head, not both")
        _check_mask(s)
        self.q_head = s.head_dim + s.rot_dim
        self.key_width = s.kv_rank + s.rot_dim
        self.gate_width = s.n_heads * s.value_dim if s.element_gate else \
            (s.n_heads if s.head_gate else 0)
        self.freq = _frequencies(s.rotary, ctx)

    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        d = {p + s.dkv_name: TensorDecl((self.key_width, s.hidden_size)),
             p + s.dkv_norm_name: TensorDecl((s.kv_rank,), init="gain"),
             p + s.uk_name: TensorDecl((s.n_heads * s.head_dim, s.kv_rank)),
             p + s.uv_name: TensorDecl((s.n_heads * s.value_dim, s.kv_rank)),
             p + s.o_name: TensorDecl((s.hidden_size, s.n_heads * s.value_dim))}
        if s.q_rank is not None:
            d[p + s.dq_name] = TensorDecl((s.q_rank, s.hidden_size))
            d[p + s.dq_norm_name] = TensorDecl((s.q_rank,), init="gain")
            d[p + s.uq_name] = TensorDecl((s.n_heads * self.q_head, s.q_rank))
        else:
            d[p + s.uq_name] = TensorDecl((s.n_heads * self.q_head, s.hidden_size))
        if self.gate_width:
            d[p + s.gate_name] = TensorDecl((self.gate_width, s.hidden_size))
        return d

    def bind(self, tensors) -> None:
        s, p = self.spec, self.prefix
        # one product over the stacked matrices: [query latent or queries | key latent | gate]
        first = tensors[p + s.dq_name] if s.q_rank is not None else tensors[p + s.uq_name]
        rows = [first, tensors[p + s.dkv_name]]
        if self.gate_width:
            rows.append(tensors[p + s.gate_name])
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        self.first_width = first.shape[0]
        self.down = Linear(place_matrix(torch.cat(rows, dim=0), self.ctx))
        self.uq = self.dq_gain = None
        if s.q_rank is not None:
            self.uq = Linear(place_matrix(tensors[p + s.uq_name], self.ctx))
            self.dq_gain = place_gain(tensors[p + s.dq_norm_name], self.ctx)
        self.o = Linear(place_matrix(tensors[p + s.o_name], self.ctx))
        # [H, kv_rank, head_dim]: the key matrix of a head, transposed, takes a query to the latent
        uk = tensors[p + s.uk_name].view(s.n_heads, s.head_dim, s.kv_rank).transpose(1, 2)
        self.uk_t = place_matrix(uk.contiguous(), self.ctx)
        self.uv = place_matrix(tensors[p + s.uv_name].view(s.n_heads, s.value_dim, s.kv_rank)
                               .contiguous(), self.ctx)
        self.dkv_gain = place_gain(tensors[p + s.dkv_norm_name], self.ctx)

    def cache_need(self):
        s = self.spec
        # one row a token: [latent | rotated part]; the values are its leading columns
        return KVNeed(1, self.key_width, s.window, value_dim=0, chunk=s.chunk)

    def accept_cache(self, cache) -> None:
        if cache.k_pool is not None and cache.k_pool.dtype != self.ctx.act_dtype:
            raise ConfigError(f"the cache is kept in the compute dtype ({self.ctx.act_dtype}): "
                              f"a cache of {cache.k_pool.dtype} needs a model built with that "
                              "dtype")

    def forward(self, h, residual, step, cache, accumulate: bool = True) -> None:
        s = self.spec
        T = h.shape[0]
        act = self.ctx.act_dtype
        if hasattr(h, "materialize"):
            h = h.materialize()
        kv = step.kv_tables(cache.group)
        KW, H, F = self.key_width, s.n_heads, self.first_width
        rot = dict(rot_dims=s.rot_dim, freq=self.freq, mag=s.rotary.magnitude) \
            if s.rotary is not None else {}
        down = step.scratch("latent_down", (T, self.down.out_features), act)
        self.down.forward(h, down)
        segments = []
        if s.q_rank is not None:
            cq = step.scratch("latent_cq", (T, s.q_rank), act)
            segments.append(ops.RowSegment(0, s.q_rank, cq, gain=self.dq_gain,
                                           eps=float(s.norm_eps)))
        if cache.writes:
            segments.append(ops.RowSegment(F, s.kv_rank, cache.k_pool, gain=self.dkv_gain,
                                           eps=float(s.norm_eps), dst_hd=KW, pool_heads=1))
            if s.rot_dim:
                segments.append(ops.RowSegment(F + s.kv_rank, s.rot_dim, cache.k_pool,
                                               dst_off=s.kv_rank, dst_hd=KW, pool_heads=1, **rot))
        if segments:
            ops.project_rows(down, step.positions, kv.slot_mapping if cache.writes else None,
                             cache.page_size, segments)
        if s.q_rank is not None:
            q = step.scratch("latent_q", (T, H * self.q_head), act)
            self.uq.forward(cq, q)
        else:
            q = down[:, :F]
        # the query on the latent's side: [U_h^T q_plain | rotated q_rot] a head
        qa = step.scratch("latent_qa", (T, H * KW), act)
        ops.head_products(q, 0, self.q_head, self.uk_t, None, qa, 0, KW)
        if s.rot_dim:
            ops.project_rows(q, step.positions, None, cache.page_size,
                             [ops.RowSegment(0, H * self.q_head, qa, hd=self.q_head,
                                             rot_off=s.head_dim, skip=s.head_dim,
                                             dst_off=s.kv_rank, dst_hd=KW, **rot)])
        gate = down[:, F + KW:] if self.gate_width else None
        mixed = step.scratch("latent_mixed", (T, H * s.kv_rank), act)
        ops.attend_masked(qa, gate if s.head_gate else None, "head" if s.head_gate else None,
                          cache.k_pool, None, None, kv.block_table,
                          step.q_start, step.ctx_len, step.seq_index, mixed, float(s.scale), 0.0,
                          int(s.window or 0), int(s.chunk or 0), H, 1, KW, s.kv_rank,
                          cache.page_size, step.max_q_len, step.max_ctx_len)
        attn = step.scratch("attn", (T, H * s.value_dim), act)
        ops.head_products(mixed, 0, s.kv_rank, self.uv, gate if s.element_gate else None, attn, 0,
                          s.value_dim)
        self.o.forward(attn, residual, accumulate=accumulate, step=step if accumulate else None)


register_part("mixer", MaskedGqaAttentionSpec, MaskedGqaAttention)
register_part("mixer", LatentAttentionSpec, LatentAttention)
