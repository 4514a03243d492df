"""One flat table of the engine's kernels: name -> (the function that launches it, the csrc
module it lives in, where the reference implementation states the formula it computes).  The
reference's counterpart is its table of ops that the per-op benchmark walks
(`src/app/cli/tools/bench/ops.zig:12-49`).  Kernels without a counterpart there (paging,
batching, fusions of two of the reference's operations) name the operations they are made of,
or say "own"."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict

from . import (gated_act, moe_grouped, norm_add_norm, tied_attention_mfma)
from . import delta_recurrence, short_conv, streams_step
from . import (concat_rows, decay_recurrence, embed_sinusoid, head_norm_gate, token_shift_mix)
from . import (activation, head_products, masked_attention, masked_attention_mfma,
               norm_add_store, project_rows)
from . import (embed_position, kv_rows_write, moe_down, moe_gate_up, moe_route, norm_rows,
               shared_kv_attention)
from . import (advance_decode, apply_penalties, argmax, argmax_no_alloc, cast, check_tables,
               decode_attention_fused, embed, gather_rows, gemm, gemm_emit, gemm_given,
               gemm_partials, gemm_sum_norm, gemm_swiglu, mfma_loop, norm_gemm, paged_attention,
               poison_pages,
               qk_norm_rope_kv_write, randinit, rmsnorm, sample_topk, scale_cap, stream_read,
               swiglu)


@dataclass(frozen=True)
class KernelEntry:
    launch: Callable
    module: str          # csrc/<module>.hip
    formula: str         # file:lines of the reference implementation, or "own: ..."


_LINEAR = "src/kernel/core/cpu.zig:21-36"
_RMSNORM = "src/kernel/core/cpu.zig:38-48,73-110"
_ATTENTION = "src/kernel/attention/basic.zig:5-76"
_QK = "src/kernel/core/cpu.zig:50-71; src/kernel/attention/rope.zig:25-34,67-90"

KERNELS: Dict[str, KernelEntry] = {
    "embed": KernelEntry(embed, "elementwise", "src/model/layers/decoder_only_stack.zig:48-93"),
    "rmsnorm": KernelEntry(rmsnorm, "elementwise", _RMSNORM),
    "qk_norm_rope_kv_write": KernelEntry(
        qk_norm_rope_kv_write, "elementwise",
        _QK + "; src/model/runtime/optimized_kv_cache/cache.zig:21-107"),
    "swiglu": KernelEntry(swiglu, "elementwise", "src/kernel/core/cpu.zig:130-147"),
    "gather_rows": KernelEntry(gather_rows, "elementwise", "own: rows whose logits are wanted"),
    "argmax": KernelEntry(argmax, "elementwise", "src/model/layers/logits.zig:47-59"),
    "argmax_no_alloc": KernelEntry(argmax_no_alloc, "elementwise",
                                   "src/model/layers/logits.zig:47-59"),
    "scale_cap": KernelEntry(scale_cap, "elementwise", "own: logit scale and tanh cap"),
    "advance_decode": KernelEntry(advance_decode, "elementwise",
                                  "own: positions and slots of the next decode step"),
    "cast": KernelEntry(cast, "elementwise", "src/tensor/formats/bfloat16.zig:3-13"),
    "poison_pages": KernelEntry(poison_pages, "elementwise", "own: NaN into pages given back"),
    "gemm": KernelEntry(gemm, "gemm", _LINEAR),
    "gemm_partials": KernelEntry(gemm_partials, "gemm", _LINEAR),
    "gemm_swiglu": KernelEntry(gemm_swiglu, "gemm", _LINEAR + "; src/kernel/core/cpu.zig:130-147"),
    "norm_gemm": KernelEntry(norm_gemm, "gemm", _RMSNORM + "; " + _LINEAR),
    "gemm_emit": KernelEntry(gemm_emit, "gemm", _LINEAR + "; " + _RMSNORM),
    "gemm_given": KernelEntry(gemm_given, "gemm", _RMSNORM + "; " + _LINEAR),
    "gemm_sum_norm": KernelEntry(gemm_sum_norm, "gemm", _LINEAR + "; " + _RMSNORM),
    "paged_attention": KernelEntry(paged_attention, "attention", _ATTENTION),
    "decode_attention_fused": KernelEntry(decode_attention_fused, "attention",
                                          _QK + "; " + _ATTENTION),
    "apply_penalties": KernelEntry(apply_penalties, "sampling",
                                   "src/sampling/sampler.zig:186-201"),
    "sample_topk": KernelEntry(sample_topk, "sampling", "src/sampling/sampler.zig:18-91"),
    "randinit": KernelEntry(randinit, "randinit", "own: counter-based random weights"),
    "check_tables": KernelEntry(check_tables, "elementwise",
                                "own: a step's block tables and slots against the pool"),
    "stream_read": KernelEntry(stream_read, "elementwise",
                               "own: the read stream bandwidths are measured against"),
    "norm_rows": KernelEntry(norm_rows, "norms", "own: layer norm / RMS norm with a bias, stored "
                             "or added to the stream"),
    "norm_add_norm": KernelEntry(norm_add_norm, "norms", "own: the norm behind a sublayer, the "
                                 "residual sum and the norm before the next sublayer"),
    "embed_position": KernelEntry(embed_position, "norms", "own: embedding plus a learned "
                                  "position row"),
    "kv_rows_write": KernelEntry(kv_rows_write, "sink_attention", "own: key rows into pages"),
    "shared_kv_attention": KernelEntry(shared_kv_attention, "sink_attention",
                                       "own: attention whose values are its keys, with a "
                                       "silent soft-max term and an output gate"),
    "tied_attention_mfma": KernelEntry(tied_attention_mfma, "sink_attention",
                                       "own: the same attention in MFMA tiles (bfloat16)"),
    "moe_route": KernelEntry(moe_route, "moe", "own: router logits, top-k, soft-max of the chosen "
                             "or sigmoid scores chosen by corrected scores within the best groups"),
    "moe_gate_up": KernelEntry(moe_gate_up, "moe", "own: the chosen experts' gated activations"),
    "moe_down": KernelEntry(moe_down, "moe", "own: the chosen experts' outputs, weighted"),
    "moe_grouped": KernelEntry(moe_grouped, "moe", "own: the chosen experts over tokens sorted "
                               "by expert, MFMA tiles"),
    "gated_act": KernelEntry(gated_act, "moe", "own: the experts' activation alone"),
    "activation": KernelEntry(activation, "elementwise", "own: gelu (erf or tanh form), silu or "
                              "squared relu alone"),
    "norm_add_store": KernelEntry(norm_add_store, "norms", "own: the norm behind a sublayer, the "
                                  "residual sum, and the sum in the products' type"),
    "project_rows": KernelEntry(project_rows, "masked_attention", "own: a projection's rows "
                                "normed over whole segments, rotated in part, into rows or pages"),
    "masked_attention": KernelEntry(masked_attention, "masked_attention", "own: attention with a "
                                    "score cap, a learned sink, chunks or a window, a gate; the "
                                    "values a pool or the keys' leading columns"),
    "masked_attention_mfma": KernelEntry(masked_attention_mfma, "masked_attention",
                                         "own: the same attention in MFMA tiles (bfloat16)"),
    "head_products": KernelEntry(head_products, "masked_attention", "own: a matrix a head"),
    "embed_sinusoid": KernelEntry(embed_sinusoid, "elementwise", "own: embedding plus a position "
                                  "vector of sines and cosines"),
    "concat_rows": KernelEntry(concat_rows, "elementwise", "own: two streams side by side for a "
                               "product over both"),
    "token_shift_mix": KernelEntry(token_shift_mix, "recurrent", "own: blends of a row with the "
                                   "row before it, the last row kept as state"),
    "decay_recurrence": KernelEntry(decay_recurrence, "recurrent", "own: a matrix a head, decayed "
                                    "a key channel and grown by k v^T, token by token"),
    "head_norm_gate": KernelEntry(head_norm_gate, "recurrent", "own: RMS norm a head, gain and "
                                  "silu gate"),
    "streams_step": KernelEntry(streams_step, "norms", "own: a residual stream in several "
                                "copies: a sublayer's output joins them, the next one's input "
                                "is read from them and normed"),
    "short_conv": KernelEntry(short_conv, "delta", "own: causal convolutions over time a channel "
                              "with silu and unit heads, the last rows kept as state"),
    "delta_recurrence": KernelEntry(delta_recurrence, "delta", "own: a matrix a head, decayed "
                                    "and corrected towards every token's value"),
    "mfma_loop": KernelEntry(mfma_loop, "gemm",
                             "own: MFMAs alone, the rate the tiled products are measured against"),
}
