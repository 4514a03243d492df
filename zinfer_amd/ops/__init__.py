"""The engine's operations: thin wrappers that check shapes on the host and launch the
hand-written HIP kernels on torch's current stream.  There is no other implementation: a
tensor that is not on the GPU, or a kernel library that cannot be built or loaded, is an
error.  Kernels take every size a configuration allows or refuse it with a clear message.
"""
from __future__ import annotations

import ctypes
import functools
from typing import Optional, Tuple

import torch

from ..errors import KernelUnavailable
from . import build

_DT = {torch.float32: 0, torch.bfloat16: 1}
_vp = ctypes.c_void_p


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    """torch's current HIP stream of the current device (the capture stream inside a graph
    capture); read through torch's raw-handle call where it has one: a launch costs a few
    microseconds of host time, and building a Stream object was half of that."""
    if _raw_stream is not None:
        return _vp(_raw_stream(torch.cuda.current_device()))
    return _vp(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return _vp(None) if t is None else _vp(t.data_ptr())


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelUnavailable(
                "the HIP kernels run on GPU tensors only; got a tensor on "
                f"{t.device} (there is no CPU path)")
        if t is not None and not t.is_contiguous():
            raise KernelUnavailable(f"kernel operands must be contiguous; got strides {t.stride()}")


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelUnavailable(f"kernels take float32 or bfloat16, not {t.dtype}") from None


def _check(code: int, what: str) -> None:
    if code != 0:
        raise KernelUnavailable(f"{what}: launch failed with code {code}")


def _i32(t: torch.Tensor, what: str) -> None:
    if t.dtype != torch.int32:
        raise KernelUnavailable(f"{what} must be int32, is {t.dtype}")


# ------------------------------------------------------------------------- kernel classes
# Every launcher belongs to a class of a step's work; the per-class benchmark
# (``Engine.class_times``, the reference's per-op harness is `src/app/cli/tools/bench/
# ops.zig:516-543`) runs a step with only one class's kernels launched, the others left out.
# The outputs of such a run mean nothing; only its time does.
KERNEL_CLASSES = ("products", "attention", "norm_rope_write", "head_sampling", "other")
_class_filter = None        # None: everything launches; else the set of classes that do
_class_override = None      # a caller's label for the launches inside it (the head's product)
_launch_count = 0           # launcher calls that went through


def launch_count() -> int:
    return _launch_count


class only_classes:
    """Within this context only kernels of ``classes`` are launched."""

    def __init__(self, classes):
        unknown = set(classes) - set(KERNEL_CLASSES)
        if unknown:
            raise KernelUnavailable(f"unknown kernel classes {sorted(unknown)}")
        self.classes = frozenset(classes)

    def __enter__(self):
        global _class_filter
        self._before, _class_filter = _class_filter, self.classes

    def __exit__(self, *exc):
        global _class_filter
        _class_filter = self._before


class kernel_class:
    """Launches inside this context count as ``name`` whatever their launcher's own class."""

    def __init__(self, name: str):
        self.name = name

    def __enter__(self):
        global _class_override
        self._before, _class_override = _class_override, self.name

    def __exit__(self, *exc):
        global _class_override
        _class_override = self._before


def _left_out(cls: str) -> bool:
    return _class_filter is not None and (_class_override or cls) not in _class_filter


def _launches(cls: str):
    """Marks a launcher with its class; under ``only_classes`` a launcher of another class
    returns without launching."""
    def deco(fn):
        @functools.wraps(fn)
        def launcher(*args, **kwargs):
            global _launch_count
            if _class_filter is not None and (_class_override or cls) not in _class_filter:
                return None
            _launch_count += 1
            return fn(*args, **kwargs)
        launcher.kernel_class = cls
        return launcher
    return deco


# ------------------------------------------------------------------------- elementwise
@_launches("other")
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[t, :] = table[ids[t], :] widened to float32, times ``scale``."""
    _need_gpu(table, ids, out)
    _i32(ids, "ids")
    T, H = out.shape
    if table.shape[1] != H or ids.shape[0] != T or out.dtype != torch.float32:
        raise KernelUnavailable(f"embed: table {tuple(table.shape)}, ids {tuple(ids.shape)}, "
                                f"out {tuple(out.shape)} {out.dtype}")
    lib = build.load("elementwise")
    _check(lib.zf_embed(_ptr(table), _dt(table), _ptr(ids), _ptr(out), T, H,
                        ctypes.c_float(scale), _stream()), "embed")


@_launches("other")
def embed_sinusoid(table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor,
                   freq: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[t, :] = table[ids[t], :] * scale plus a position vector formed where it is used:
    entry 2i gets sin(p * freq[i]), entry 2i + 1 cos(p * freq[i]), p = positions[t]; the angle
    is the 32-bit product.  ``freq`` float32 [ceil(H / 2)]."""
    _need_gpu(table, ids, positions, freq, out)
    _i32(ids, "ids")
    _i32(positions, "positions")
    T, H = out.shape
    if table.shape[1] != H or ids.shape[0] != T or positions.shape[0] != T \
            or out.dtype != torch.float32 or freq.dtype != torch.float32 \
            or freq.shape != ((H + 1) // 2,):
        raise KernelUnavailable(f"embed_sinusoid: table {tuple(table.shape)}, out "
                                f"{tuple(out.shape)} {out.dtype}, freq {tuple(freq.shape)} "
                                f"{freq.dtype}")
    lib = build.load("elementwise")
    _check(lib.zf_embed_sinusoid(_ptr(table), _dt(table), _ptr(ids), _ptr(positions), _ptr(freq),
                                 _ptr(out), T, H, ctypes.c_float(scale), _stream()),
           "embed_sinusoid")


@_launches("other")
def concat_rows(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> None:
    """out[t] = [a[t] | b[t]] for two float32 matrices [T, H], in ``out``'s type [T, 2 H]."""
    _need_gpu(a, b, out)
    T, H = a.shape
    if b.shape != a.shape or out.shape != (T, 2 * H) or a.dtype != torch.float32 \
            or b.dtype != torch.float32:
        raise KernelUnavailable(f"concat_rows: float32 {tuple(a.shape)} and {tuple(b.shape)} "
                                f"into {tuple(out.shape)}")
    lib = build.load("elementwise")
    _check(lib.zf_concat_rows(_ptr(a), _ptr(b), _ptr(out), _dt(out), T, H, _stream()),
           "concat_rows")


@_launches("head_sampling")
def scale_cap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> None:
    """In place on float32: x = x * scale, then with cap > 0: x = cap * tanh(x / cap)."""
    _need_gpu(x)
    if x.dtype != torch.float32 or cap < 0.0:
        raise KernelUnavailable("scale_cap: a float32 tensor and a cap that is not negative")
    lib = build.load("elementwise")
    _check(lib.zf_scale_cap(_ptr(x), ctypes.c_longlong(x.numel()), ctypes.c_float(scale),
                            ctypes.c_float(cap), _stream()), "scale_cap")


@_launches("norm_rope_write")
def rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """out = x * gain / sqrt(mean(x^2) + eps) over the last axis; x and gain float32."""
    _need_gpu(x, gain, out)
    T, W = x.shape
    if x.dtype != torch.float32 or gain.dtype != torch.float32 or gain.shape != (W,) \
            or out.shape != x.shape:
        raise KernelUnavailable(f"rmsnorm: x {tuple(x.shape)} {x.dtype}, gain "
                                f"{tuple(gain.shape)} {gain.dtype}, out {tuple(out.shape)}")
    lib = build.load("elementwise")
    _check(lib.zf_rmsnorm(_ptr(x), _ptr(gain), _ptr(out), _dt(out), T, W, ctypes.c_float(eps),
                          _stream()), "rmsnorm")


@_launches("norm_rope_write")
def qk_norm_rope_kv_write(qkv, q_gain, k_gain, eps, cos, sin, positions, slot_mapping, k_pool,
                          v_pool, q_out, n_heads, n_kv_heads, head_dim, page_size) -> None:
    """Per token and head of ``qkv`` [T, (nH + 2 nKV) hd]: optional RMSNorm of q and k heads
    with the [hd] gains, optional half-split rotation from the [max_pos, hd/2] tables at
    ``positions``; q goes to ``q_out`` [T, nH hd] (in place if None), k and v go into the
    pools at ``slot_mapping`` (k in place if None).  Pools of a shape the MFMA attention
    kernels cover (``mfma_attention_covers``) are written in those kernels' own order.

    ``qkv`` may also be the float32 partials [ksplit, T, (nH + 2 nKV) hd] of a product split
    along K (``gemm_partials``): the kernel adds them in split order and rounds to bfloat16
    on its way, as the kernel that only adds them would have (bfloat16 pools, ``q_out`` and
    ``slot_mapping`` given)."""
    partials = qkv if qkv.dim() == 3 else None
    if partials is not None:
        if partials.dtype != torch.float32 or not partials.is_contiguous() or q_out is None \
                or slot_mapping is None or k_pool.dtype != torch.bfloat16 \
                or head_dim % 8 != 0 or head_dim > 512:
            raise KernelUnavailable("qk_norm_rope_kv_write: partials must be contiguous float32 "
                                    "[ksplit, T, width], with q_out, slot_mapping and bfloat16 "
                                    "pools, head_dim a multiple of 8 up to 512")
        qkv = partials[0]
    _need_gpu(qkv, q_gain, k_gain, cos, sin, positions, slot_mapping, k_pool, v_pool, q_out)
    T = qkv.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if qkv.shape[1] != width or head_dim % 2 != 0:
        raise KernelUnavailable(f"qk_norm_rope_kv_write: qkv {tuple(qkv.shape)} for "
                                f"{n_heads}+2*{n_kv_heads} heads of {head_dim} (even)")
    if (q_gain is None) != (k_gain is None) or (cos is None) != (sin is None):
        raise KernelUnavailable("qk_norm_rope_kv_write: gains and tables come in pairs")
    for g in (q_gain, k_gain):
        if g is not None and (g.dtype != torch.float32 or g.shape != (head_dim,)):
            raise KernelUnavailable("qk_norm_rope_kv_write: a gain must be float32 [head_dim]")
    if cos is not None and (cos.dtype != torch.float32 or cos.shape[1] != head_dim // 2
                            or cos.shape != sin.shape):
        raise KernelUnavailable("qk_norm_rope_kv_write: tables must be float32 [*, head_dim/2]")
    _i32(positions, "positions")
    row_dtype = torch.bfloat16 if partials is not None else qkv.dtype
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        if k_pool.dtype != row_dtype or v_pool.dtype != row_dtype:
            raise KernelUnavailable("qk_norm_rope_kv_write: pools and qkv differ in dtype")
    if q_out is not None and (q_out.dtype != row_dtype
                              or q_out.shape != (T, n_heads * head_dim)):
        raise KernelUnavailable("qk_norm_rope_kv_write: q_out must be [T, nH * hd] of qkv's dtype")
    lib = build.load("elementwise")
    _check(lib.zf_qk_norm_rope_kv_write(
        _ptr(None if partials is not None else qkv), 1 if partials is not None else _dt(qkv),
        _ptr(q_gain), _ptr(k_gain),
        ctypes.c_float(eps), _ptr(cos),
        _ptr(sin), _ptr(positions), _ptr(slot_mapping), _ptr(k_pool), _ptr(v_pool), _ptr(q_out),
        T, n_heads, n_kv_heads, head_dim, page_size,
        1 if mfma_attention_covers(row_dtype, n_heads, n_kv_heads, head_dim, page_size) else 0,
        0 if cos is None else cos.shape[0],
        _ptr(partials), 0 if partials is None else partials.shape[0],
        _stream()), "qk_norm_rope_kv_write")


@_launches("norm_rope_write")
def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, j] = silu(gate_up[t, j]) * gate_up[t, I + j]."""
    _need_gpu(gate_up, out)
    T, I = out.shape
    if gate_up.shape != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelUnavailable(f"swiglu: gate_up {tuple(gate_up.shape)}, out {tuple(out.shape)}")
    lib = build.load("elementwise")
    _check(lib.zf_swiglu(_ptr(gate_up), _ptr(out), _dt(out), T, I, _stream()), "swiglu")


@_launches("other")
def cast(src: torch.Tensor, out: torch.Tensor) -> None:
    """out = src in the other storage type (bfloat16 <-> float32), element by element."""
    _need_gpu(src, out)
    if src.shape != out.shape or src.dtype == out.dtype:
        raise KernelUnavailable(f"cast: {tuple(src.shape)} {src.dtype} -> {tuple(out.shape)} "
                                f"{out.dtype}")
    lib = build.load("elementwise")
    _check(lib.zf_cast(_ptr(src), _dt(src), _ptr(out), _dt(out), ctypes.c_longlong(src.numel()),
                       _stream()), "cast")


@_launches("other")
def poison_pages(pool: torch.Tensor, pages: torch.Tensor) -> None:
    """pool[:, pages, :] = NaN: ``pool`` [runs, pages, row] float32 or bfloat16, ``pages`` int32."""
    _need_gpu(pool, pages)
    _i32(pages, "pages")
    if pool.dim() != 3 or pages.dim() != 1:
        raise KernelUnavailable("poison_pages: a pool [runs, pages, row] and a list of pages")
    lib = build.load("elementwise")
    _check(lib.zf_poison_pages(_ptr(pool), _dt(pool), _ptr(pages), pages.shape[0], pool.shape[0],
                               ctypes.c_longlong(pool.shape[1]), ctypes.c_longlong(pool.shape[2]),
                               _stream()), "poison_pages")


@_launches("head_sampling")
def gather_rows(x: torch.Tensor, idx: torch.Tensor, out: torch.Tensor) -> None:
    _need_gpu(x, idx, out)
    _i32(idx, "idx")
    n, H = out.shape
    if x.shape[1] != H or idx.shape[0] != n or x.dtype != torch.float32 or out.dtype != x.dtype:
        raise KernelUnavailable("gather_rows: float32 [T, H] -> [n, H]")
    lib = build.load("elementwise")
    _check(lib.zf_gather_rows(_ptr(x), _ptr(idx), _ptr(out), n, H, _stream()), "gather_rows")


@_launches("head_sampling")
def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = index of the first maximum of logits[r, :]."""
    _need_gpu(logits, out)
    _i32(out, "out")
    n, V = logits.shape
    if logits.dtype != torch.float32 or out.shape != (n,):
        raise KernelUnavailable("argmax: float32 [n, V] -> int32 [n]")
    lib = build.load("elementwise")
    ws = _workspace("argmax", 2 * n * ((V + 4095) // 4096), torch.float32, logits.device)
    _check(lib.zf_argmax(_ptr(logits), _ptr(out), _ptr(ws), n, V, _stream()), "argmax")


ARGMAX_NO_ALLOC_MAX_PARTIALS = 32768    # ZF_ARGMAX_NO_ALLOC_MAX_PARTIALS in zf_no_alloc.h


@_launches("head_sampling")
def argmax_no_alloc(logits: torch.Tensor, out: torch.Tensor) -> None:
    """``argmax`` for callers that cannot allocate: the partial results live in a fixed device
    array of the library (shared by all calls on a GPU: overlapping calls race), so at most
    n * ceil(V / 4096) = 32768 of them."""
    _need_gpu(logits, out)
    _i32(out, "out")
    n, V = logits.shape
    if logits.dtype != torch.float32 or out.shape != (n,):
        raise KernelUnavailable("argmax_no_alloc: float32 [n, V] -> int32 [n]")
    if n * ((V + 4095) // 4096) > ARGMAX_NO_ALLOC_MAX_PARTIALS:
        raise KernelUnavailable(f"argmax_no_alloc: {n} rows of {V} logits need more than "
                                f"{ARGMAX_NO_ALLOC_MAX_PARTIALS} partial results")
    lib = build.load("elementwise")
    _check(lib.zf_argmax_no_alloc(_ptr(logits), _ptr(out), n, V, _stream()), "argmax_no_alloc")


@_launches("other")
def advance_decode(token_ids: torch.Tensor, positions: torch.Tensor, ctx_len: torch.Tensor,
                   sampled: torch.Tensor, slot_mapping: torch.Tensor, block_table: torch.Tensor,
                   page_size: int, advance: bool) -> None:
    """One decode step on, on the device: with ``advance`` token_ids = sampled, positions and
    ctx_len + 1; always slot_mapping[i] = block_table[i, p // page_size] * page_size +
    p % page_size at the (new) position p.  The caller guarantees that the table holds a page
    there."""
    _need_gpu(token_ids, positions, ctx_len, sampled, slot_mapping, block_table)
    for t, name in ((token_ids, "token_ids"), (positions, "positions"), (ctx_len, "ctx_len"),
                    (sampled, "sampled"), (slot_mapping, "slot_mapping"),
                    (block_table, "block_table")):
        _i32(t, name)
    n = token_ids.shape[0]
    if block_table.dim() != 2 or block_table.shape[0] != n or not block_table.is_contiguous() \
            or any(t.shape != (n,) for t in (positions, ctx_len, sampled, slot_mapping)):
        raise KernelUnavailable("advance_decode: int32 [n] vectors and a contiguous [n, pages] "
                                "block table")
    lib = build.load("elementwise")
    _check(lib.zf_advance_decode(_ptr(token_ids), _ptr(positions), _ptr(ctx_len), _ptr(sampled),
                                 _ptr(slot_mapping), _ptr(block_table), n, block_table.shape[1],
                                 int(page_size), 1 if advance else 0, _stream()),
           "advance_decode")


@_launches("other")
def randinit(out: torch.Tensor, key: int, start: int, kind: str, std: float = 0.02) -> None:
    """out[i] = element ``start + i`` of the random tensor with ``key``
    (`weights/counter_rng.py`: 'normal' = N(0, std), 'gain' = 1 + U(-0.1, 0.1), 'zeros')."""
    from ..weights.counter_rng import KIND
    _need_gpu(out)
    if out.dim() != 1 or kind not in KIND:
        raise KernelUnavailable(f"randinit: a flat tensor and a kind of {sorted(KIND)}")
    lib = build.load("randinit")
    _check(lib.zf_randinit(_ptr(out), _dt(out), ctypes.c_ulonglong(key & ((1 << 64) - 1)),
                           ctypes.c_ulonglong(start), ctypes.c_ulonglong(out.numel()),
                           KIND[kind], ctypes.c_double(std), _stream()), "randinit")


@_launches("other")
def check_tables(block_table: torch.Tensor, ctx_len: torch.Tensor,
                 slot_mapping: Optional[torch.Tensor], page_size: int, num_pages: int,
                 report: torch.Tensor) -> None:
    """Debugging: marks in ``report`` (int32 [4], zeroed by the caller: kind, sequence or token,
    index, value) a block-table entry among those a step's kernels will look up that is no
    page of the pool (kind 1), a context longer than the table's row, or a slot that is no row
    of the pool (kind 2).  The kernels themselves trust their tables; this is the check to
    switch on when they are in doubt (``Engine(debug_tables=True)``)."""
    _need_gpu(block_table, ctx_len, slot_mapping, report)
    for t, name in ((block_table, "block_table"), (ctx_len, "ctx_len"), (report, "report")):
        _i32(t, name)
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
    if block_table.dim() != 2 or ctx_len.shape != (block_table.shape[0],) or report.numel() < 4:
        raise KernelUnavailable("check_tables: int32 [n, pages] table, [n] contexts, [4] report")
    lib = build.load("elementwise")
    _check(lib.zf_check_tables(_ptr(block_table), _ptr(ctx_len), _ptr(slot_mapping),
                               block_table.shape[0], block_table.shape[1], int(page_size),
                               int(num_pages), 0 if slot_mapping is None else slot_mapping.shape[0],
                               _ptr(report), _stream()), "check_tables")


@_launches("other")
def stream_read(buf: torch.Tensor, sink: torch.Tensor, workgroups: int = 2048) -> None:
    """Reads ``buf`` once (16-byte non-temporal loads, 8 in flight a lane) and xors it into
    ``sink`` (int32, one word per workgroup): the read stream the weight-streaming kernels are
    measured against (``measure_read_bandwidth``)."""
    _need_gpu(buf, sink)
    _i32(sink, "sink")
    nbytes = buf.numel() * buf.element_size()
    if nbytes % 16 != 0 or sink.numel() < workgroups or not 1 <= workgroups <= 65536:
        raise KernelUnavailable("stream_read: a buffer of a multiple of 16 bytes and a sink of "
                                "one int32 per workgroup (1 to 65536)")
    lib = build.load("elementwise")
    _check(lib.zf_stream_read(_ptr(buf), ctypes.c_longlong(nbytes), _ptr(sink), int(workgroups),
                              _stream()), "stream_read")


def measure_read_bandwidth(device, nbytes: int = 2 << 30, repeats: int = 3) -> float:
    """Bytes a second of the best of ``repeats`` passes of ``stream_read`` over a buffer of
    ``nbytes`` (far more than the last-level cache holds, so it comes from HBM), each pass
    timed by a pair of events; the best of 256 to 4096 workgroups."""
    buf = torch.empty((nbytes // 4,), dtype=torch.int32, device=device)
    buf.zero_()
    sink = torch.zeros((4096,), dtype=torch.int32, device=device)
    best = 0.0
    for wgs in (256, 512, 768, 1024, 2048, 4096):
        stream_read(buf, sink, wgs)                       # warm-up
        for _ in range(repeats):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            stream_read(buf, sink, wgs)
            b.record()
            b.synchronize()
            best = max(best, nbytes / (a.elapsed_time(b) * 1e-3))
    del buf
    return best


@_launches("other")
def mfma_loop(operands: torch.Tensor, out: torch.Tensor, workgroups: int, iters: int) -> None:
    """``iters`` rounds of eight 32x32x16 MFMAs between the operands in ``operands`` (bfloat16
    [6, 64, 8]: four token operands, two weight operands, as the lanes of a wave hold them) in
    every wave of ``workgroups`` workgroups of four; ``out`` float32 [8, 32, 32] takes the first
    wave's accumulators (accumulator n: ``iters`` times tokens n % 4 against weights n / 4).
    Nothing but MFMAs: the rate the matrix cores sustain (``measure_mfma_rate``)."""
    _need_gpu(operands, out)
    if operands.dtype != torch.bfloat16 or tuple(operands.shape) != (6, 64, 8) \
            or not operands.is_contiguous() or out.dtype != torch.float32 \
            or tuple(out.shape) != (8, 32, 32) or not out.is_contiguous():
        raise KernelUnavailable("mfma_loop: operands bfloat16 [6, 64, 8], out float32 [8, 32, 32]")
    lib = build.load("gemm")
    _check(lib.zf_mfma_loop(_ptr(operands), _ptr(out), int(workgroups), int(iters), _stream()),
           "mfma_loop")


MFMA_LOOP_FLOPS = 2.0 * 32 * 32 * 16 * 8 * 4       # a workgroup's flops in one round


def measure_mfma_rate(device, random_operands: bool = True, seconds: float = 0.03) -> float:
    """Flops a second of ``mfma_loop`` on the whole chip, sustained over about ``seconds``
    (launches of a few milliseconds, the first ones untimed: the clock settles under the
    load).  On random operands the chip's power limit sets it, on zeros its clock."""
    g = torch.Generator(device="cpu").manual_seed(5)
    operands = (torch.randn((6, 64, 8), generator=g) if random_operands
                else torch.zeros((6, 64, 8))).to(torch.bfloat16).to(device)
    out = torch.zeros((8, 32, 32), dtype=torch.float32, device=device)
    workgroups, iters = 1024, 8000                  # about 5 ms a launch
    for _ in range(3):
        mfma_loop(operands, out, workgroups, iters)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = 0
    a.record()
    while True:
        mfma_loop(operands, out, workgroups, iters)
        n += 1
        b.record()
        b.synchronize()
        dt = a.elapsed_time(b) * 1e-3
        if dt >= seconds or n >= 64:
            return MFMA_LOOP_FLOPS * workgroups * iters * n / dt


# ------------------------------------------------------------------------- work buffers
_workspaces = {}
_workspace_generation = 0


def workspace_generation() -> int:
    """Goes up whenever a work buffer is (re)allocated: a captured graph that used the old
    buffer must not be replayed."""
    return _workspace_generation


def _workspace(name: str, numel: int, dtype: torch.dtype, device) -> torch.Tensor:
    """A persistent device buffer of at least ``numel`` elements (grown when needed, never
    inside a stream capture once sizes have settled)."""
    global _workspace_generation
    key = (name, str(device), dtype)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < numel:
        buf = torch.empty((max(numel, 1),), dtype=dtype, device=device)
        _workspaces[key] = buf
        _workspace_generation += 1
    return buf


# ------------------------------------------------------------------------- matrix product
_EPI_STORE_BF16, _EPI_STORE_F32, _EPI_ACC_F32, _EPI_SWIGLU = 0, 1, 2, 3
SKINNY_MAX_M = 64
NORM_FOLD_MAX_M = 16


def _skinny_plan(M: int, N: int, K: int, tiled: bool):
    """Row groups of 16 per workgroup and workgroups along K for the weight-streaming kernel:
    enough workgroups to fill 256 CUs, as many rows per workgroup as that allows (the tokens
    are re-read once per workgroup).  Measured on MI355X at the Qwen3-8B sizes."""
    if tiled:
        if M <= 16:
            # one workgroup per CU streams best: the fewest row groups per workgroup that
            # still leave at most 256 workgroups, if that keeps half the CUs busy (384 row
            # groups: 192 workgroups of 2; 320: 160 of 2; 640: 160 of 4); a wide output takes 2
            for rg in (1, 2, 4):
                if N % (16 * rg) == 0 and 128 <= N // (16 * rg) <= 256:
                    return rg, 1
            return (2 if N >= 6144 else 1), 1
        # 17 to 64 tokens.  A wide output fills the chip by its row groups alone.  A narrow one
        # takes about 256 workgroups: the longer K is, the more rows a workgroup keeps (the
        # tokens are read again by every workgroup), and a split along K makes up for the
        # workgroups that costs (4096 x 1024: 256 of one row group; 1024 x 2048: 64 x 4 along
        # K; 2048 x 6144: 64 of two row groups x 4; 4096 x 12288: 64 of four x 4).  Measured on
        # MI355X at the projection widths of the Qwen3 0.6B to 8B shapes.
        if N >= 16384:
            return 4, 1
        if N >= 6144:
            return 2, 1
        rg = 1 if K < 4096 else 2 if K < 8192 else 4
        while rg > 1 and N % (16 * rg) != 0:
            rg //= 2
        wgs, ks = N // (16 * rg), 1
        while 2 * ks * wgs <= 256 and 2 * ks <= 16 and K >= 1024 * ks:
            ks *= 2
        return rg, ks
    if M <= 16:
        rg = 4 if N // 64 >= 256 else 1
        ks = 2 if (rg == 4 and N // 64 < 1024) else 1
    else:
        rg, ks = 4, 1
        while (N // 64) * ks < 192 and ks < 16:
            ks *= 2
    return rg, ks


MID_MAX_M = 128


def _mid_plan(M: int, N: int, K: int, w_tiled: bool, swiglu: bool = False):
    """Workgroups along K if the kernel for 17 to 128 tokens (128 outputs per workgroup, the
    tokens through LDS) covers the product, else None: above 32 tokens, and from 17 on a wide
    output, it beats the weight-streaming kernel, which re-reads the tokens for every few
    rows of the weight, and from 65 to 128 tokens the 128 x 128 tiles, two of whose waves load
    each part of the weight.  Split along K until up to 256 workgroups run, each keeping 1024
    of K.  Measured on MI355X at the Qwen3-8B sizes."""
    if not (w_tiled and 16 < M <= MID_MAX_M and N % 16 == 0
            and K % (256 if M <= 32 else 128) == 0):
        return None
    if M <= 32 and N < 16384:
        return None
    if swiglu:
        return 1
    tiles = (N + 127) // 128
    # up to 64 tokens a workgroup has half the work per k-tile: it may keep as little as 512 of K
    if M <= 64:
        return max(1, min(256 // tiles, K // 512))
    # above, 1024 of K a workgroup, or as little as 512 where that is what it takes to have
    # 128 workgroups (narrow outputs on a short K: 2048 x 2048 at 80 tokens 15.0 -> 12.4 us,
    # 1024 x 3072 15.2 -> 12.7, 2560 x 4096 16.7 -> 15.3)
    return max(1, min(256 // tiles, K // 512, max(K // 1024, (128 + tiles - 1) // tiles)))


_measured = None


def _measured_plans() -> dict:
    global _measured
    if _measured is None:
        import json
        import os
        with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "plans_mi355x.json")) as f:
            _measured = json.load(f)
    return _measured


PLAN_FILE = "kernel_plans.json"     # a model folder may bring plans measured at its own widths
PLAN_BUCKETS = (17, 24, 32, 48, 64)


def plan_bucket(M: int) -> int:
    """The bucket of a number of tokens in 17..64: a plan is kept per bucket, not per M."""
    return 17 if M <= 20 else 24 if M <= 28 else 32 if M <= 32 else 48 if M <= 56 else 64


def check_plans(plans: dict) -> None:
    """Raises ``KernelUnavailable`` unless every entry of a plan table names a configuration
    the launchers accept (what ``load_plans`` takes, and what the tuner writes)."""
    def bad(why):
        raise KernelUnavailable(f"kernel plans: {why}")
    for key, entry in plans.get("plans", {}).items():
        shape, _, kind = key.partition(":")
        try:
            N, K = (int(x) for x in shape.split("x"))
        except ValueError:
            bad(f"{key!r} is not 'NxK' or 'NxK:swiglu'")
        if kind not in ("", "swiglu"):
            bad(f"{key!r}: unknown kind {kind!r}")
        for bucket, plan in entry.items():
            M = int(bucket)
            if M not in PLAN_BUCKETS:
                bad(f"{key}: bucket {bucket} is none of {PLAN_BUCKETS}")
            if plan[0] == "mid" and len(plan) == 2:
                # k-tiles of 256 (up to 32 tokens) or 128, dealt over the workgroups along K
                ks, tk = int(plan[1]), (256 if M <= 32 else 128)
                ok = K % tk == 0 and 1 <= ks <= K // tk and N % 16 == 0
            elif plan[0] == "skinny" and len(plan) == 3:
                rg, ks = int(plan[1]), int(plan[2])
                ok = rg in (1, 2, 4) and N % (16 * rg) == 0 and 1 <= ks <= 16 and K % 64 == 0
            else:
                ok = False
            if ok and kind == "swiglu":
                ok = plan[-1] == 1 and (plan[0] == "mid" or plan[1] >= 2) and N % 32 == 0
            if not ok:
                bad(f"{key} at {bucket} tokens: {plan} is no plan the kernels take")
    for key, plan in plans.get("decode_acc", {}).items():
        if key == "_":
            continue
        N, K = (int(x) for x in key.split("x"))
        if plan is not None and not (
                len(plan) == 3 and plan[0] == "skinny" and plan[1] in (1, 2, 4)
                and N % (16 * plan[1]) == 0 and 2 <= plan[2] <= 16 and N <= 8192 and K % 64 == 0):
            bad(f"decode_acc {key}: {plan} is no plan the kernels take")


def load_plans(path: str) -> int:
    """Merges a plan file (``bench-ops --tune`` writes one) over the built-in table: its
    entries win for their widths.  Returns the number of entries taken."""
    import json
    with open(path, "r", encoding="utf-8") as f:
        plans = json.load(f)
    check_plans(plans)
    table = _measured_plans()
    n = 0
    for key, entry in plans.get("plans", {}).items():
        table["plans"][key] = {str(b): list(p) for b, p in entry.items()}
        n += 1
    for key, plan in plans.get("decode_acc", {}).items():
        if key != "_":
            table["decode_acc"][key] = None if plan is None else list(plan)
            n += 1
    return n


def _small_plan(M: int, N: int, K: int, w_tiled: bool, swiglu: bool = False):
    """Which kernel takes a product of 17 to 128 tokens (None: the tiled kernels):
    ('mid', workgroups along K) or ('skinny', row groups per workgroup, workgroups along K).
    The widths of the served models have measured entries in ``plans_mi355x.json``; other
    widths follow the rules of ``_mid_plan`` and ``_skinny_plan``."""
    if w_tiled and 16 < M <= SKINNY_MAX_M:
        bucket = plan_bucket(M)
        entry = _measured_plans()["plans"].get(f"{N}x{K}" + (":swiglu" if swiglu else ""))
        if entry is not None:
            # a width measured at fewer numbers of tokens: the nearest one on the same side of
            # 32 tokens (the kernels change there)
            same = [int(b) for b in entry if (int(b) <= 32) == (bucket <= 32)]
            if same:
                plan = entry[str(min(same, key=lambda b: abs(b - bucket)))]
                return tuple(plan)
    mid = _mid_plan(M, N, K, w_tiled, swiglu)
    # a short K: what the weight-streaming kernel reads again per workgroup is little, and it
    # stays ahead of the kernel that stages the tokens up to 56 tokens (64 at K <= 1024)
    short_k = w_tiled and 32 < M <= SKINNY_MAX_M and K <= 2048 and (M <= 56 or K <= 1024)
    if mid is not None and not short_k:
        return ("mid", mid)
    if M <= SKINNY_MAX_M:
        if swiglu:
            return ("skinny", 4 if (M > 16 and N >= 12288 and N % 64 == 0) else 2, 1)
        return ("skinny",) + tuple(_skinny_plan(M, N, K, w_tiled))
    return None


def _decode_acc_plan(M: int, N: int, K: int):
    """('skinny', row groups, workgroups along K) if, at 1 to 16 tokens, a residual sum that an
    RMSNorm follows is measured to run faster split along K (the reduce adds the residual and
    norms) than with the one-launch epilogue; else None."""
    if not 0 < M <= NORM_FOLD_MAX_M:
        return None
    plan = _measured_plans()["decode_acc"].get(f"{N}x{K}")
    return tuple(plan) if plan is not None else None


def _tile_variant(M: int, N: int, w_tiled: bool = False, accumulate: bool = False,
                  K: int = 0) -> int:
    """Which tiled kernel: with pre-tiled weights the kernels that take W straight from
    memory (10: 128 x 256 tiles, two workgroups to a CU, when they fill the chip; 12: the same
    tiles with two groups of waves a workgroup where a CU holds one; else 128 x
    128 tiles, 16: with the waves side by side and k-tiles of 128 (weights from HBM, 512
    tokens: qkv of the 8B shape 43 -> 38 us), 6: with 2 x 2 waves, where K is no multiple of
    128); otherwise the kernels that stage both operands through LDS
    (4: 256 x 256 when they still fill the chip, else 0: 128 x 128).  Measured on MI355X at the
    Qwen3-8B and Qwen3-14B sizes."""
    if w_tiled:
        tiles_m = (M + 127) // 128
        tiles = tiles_m * ((N + 255) // 256)
        # from 144 large tiles on they win or draw (140 to 152 tiles: 0.84 to 1.05 of the
        # 128 x 128 tiles' time).  Between one and two 128 x 256 tiles per CU half the CUs hold
        # two workgroups and half one: there the 256-token tiles are measured against the
        # 128 x 128 ones (2048 tokens into 6144 outputs); with few tiles along the tokens (512
        # tokens into 24576 outputs) the large tiles still win (five rows of tiles: 544 tokens
        # into 24576 outputs, 480 large tiles, 143 -> 115 us)
        if tiles >= 144 and not (256 < tiles < 512 and tiles_m > 5):
            # one workgroup to a CU whatever is done: two groups of waves in it, each over
            # half of a long K (o_proj and down at 1280 to 2048 tokens: 3 to 12 % less; at
            # K <= 2048 the blocks handed over at the end cost more than the waves gain)
            if 160 <= tiles <= TILE_PLACES // 2 and K >= 4096 and K % 256 == 0:
                return 12
            return 10
        # (the 128 x 128 tiles of 2 x 2 waves, where two waves load each part of W, only
        # where k-tiles of 128 do not divide K: in 24 products of 136 to 4096 tokens that had
        # them, the waves side by side were level or faster, 12 % in all)
        return 16 if K > 0 and K % 128 == 0 else 6
    tiles = ((M + 255) // 256) * ((N + 255) // 256)
    return 4 if tiles >= 160 else 0


def _tile_ksplit(M: int, N: int, K: int, accumulate: bool = True) -> int:
    """Workgroups per 128 x 128 tile along K: products of a few hundred tokens on a narrow
    output have too few tiles for 256 CUs, or a number that fills them unevenly (160 tiles:
    96 CUs idle; 320: a second round for a quarter of them).  Two workgroups fit a CU, so the
    split is chosen to fill 256 or a multiple of 512 places as evenly as it can, each
    workgroup keeping at least 8 k-tiles of 64.  Every split costs partials of M * N floats,
    written and read again (against the product's own time that is about 400 / K a split),
    and the first one a second launch.  A product that is stored, not added to the residual,
    stays whole once its tiles need a second round anyway (257 and more: 768 tokens of the 8B
    shape's qkv 66 -> 59 us); the residual sum gains from the split up to 383 tiles, since the
    kernel that adds the partials is the norm's as well.  Measured on MI355X at the Qwen3-8B,
    14B and 32B sizes, 256 to 1024 tokens, the weights from HBM."""
    tiles = ((M + 127) // 128) * ((N + 127) // 128)
    if tiles >= 384 or (tiles > 256 and not accumulate):
        return 1
    # one round of 128 x 256 tiles with two groups of waves a workgroup needs no partials: on
    # a short K it beats the split even with the norm's kernel behind it (1280 tokens into
    # 4096 outputs, K = 4096: 64 + 6 against 76 us; 2048 into 2560: 59 + 8 against 75); on a
    # long K the split stays ahead (1024 into 5120, K = 17408: 205 against 237)
    if K < 8192 and _tile_variant(M, N, True, accumulate, K) == 12:
        return 1
    best, best_cost = 1, None
    for ks in range(1, min(8, K // 64 // 8) + 1):
        wgs = tiles * ks
        places = 256 if wgs <= 256 else (wgs + 511) // 512 * 512
        cost = places / wgs + (ks * 400.0 / K + 0.05 if ks > 1 else 0.0)
        if best_cost is None or cost < best_cost - 1e-9:
            best, best_cost = ks, cost
    return best


# Rates per CU (flop/s) of the tiled kernels on pre-tiled weights, from gate/up of the 8B shape
# at 16384 tokens: the 256-token tiles of 256, 192 and 128 outputs (one workgroup to a CU),
# and the 128-token tiles two to a CU ("pair") or one ("alone").
_TILE256_RATE = {20: 5.18e12, 21: 4.52e12, 22: 3.73e12}
_TILE256_WIDTH = {20: 256, 21: 192, 22: 128}
_TILE128_RATE = {10: (5.13e12, 3.85e12), 12: (5.13e12, 4.05e12), 16: (3.8e12, 2.9e12), 6: (3.77e12, 2.7e12)}


@functools.lru_cache(maxsize=None)
def _tile64_covers(M: int, N: int, K: int, accumulate: bool) -> bool:
    """A few hundred tokens on a narrow output, no residual sum: tiles of 64 tokens x 128
    outputs, unsplit.  A CU finishes one such tile in about two thirds of the time of a
    128 x 128 tile, and a second round doubles that, so they are taken where one round holds
    them (up to 288: the last few share CUs), or where the 128-token tiles would need a
    second round themselves while these stay within two.  Measured on MI355X with weights
    that come from HBM (more copies in turn than the last-level cache holds): qkv of the
    8B shape at 272 tokens 36 -> 26 us, o_proj-like 5120 x 8192 at 384 tokens 72 -> 51 us,
    qkv of the 14B shape at 528 to 576 tokens 70 -> 58 us; with 300 to 512 tiles against one
    round of the larger ones they lose (14B qkv at 384 tokens 47 -> 57 us).  A residual sum
    keeps its split along K, whose second kernel is also the norm."""
    if accumulate or not (128 < M <= 640 and K % 128 == 0 and N % 16 == 0 and K <= 8192):
        return False
    cols = (N + 127) // 128
    tiles64, tiles128 = ((M + 63) // 64) * cols, ((M + 127) // 128) * cols
    return tiles64 <= 288 or (tiles128 > 256 and tiles64 <= 512)


def _tile256_time(variant: int, M: int, N: int, K: int) -> float:
    """Estimated seconds of the 256-token tile kernel: rounds of up to 256 tiles, one to a CU."""
    bn = _TILE256_WIDTH[variant]
    tiles = ((M + 255) // 256) * ((N + bn - 1) // bn)
    rounds = (tiles + 255) // 256
    t = rounds * 2.0 * 256 * bn * K / _TILE256_RATE[variant]
    # on a narrow output the 256-token tiles fall behind this estimate once every CU takes
    # more than one (o_proj and down at 8192 tokens and more: by 6 to 20 %)
    return t * (1.08 if (rounds > 1 and N <= 5120) else 1.0) + 4e-6


TILE_PLACES = 512       # workgroups of the 128 x 256 tiles the chip holds at once: two to a CU


def _tile_tail_split(M: int, N: int, K: int):
    """(whole, split) if the 128 x 256 tiles of a product on pre-tiled weights should run with
    their last, short round split along K, else None: ``whole`` tiles fill whole rounds of the
    chip's ``TILE_PLACES`` places, and each of the others goes to ``split`` workgroups.  A
    round of a few tiles takes as long as a full one (512 tokens into the 14B shape's 34816
    gate and up outputs: 544 tiles, 210 us, of which the last 32 take 80); split in four it
    takes a quarter of that, plus what the partials cost: 128 KB a workgroup, written and read
    again, and a second kernel.  The split that the estimate below likes best is taken if it
    saves a fifth of the round or more, which on MI355X (Qwen3-8B and 14B widths, 512 to 4096
    tokens) is where the measured gain begins: 210 -> 165 us above, 768 tokens into 24576
    outputs 156 -> 131, 1024 into 34816 339 -> 307; a last round of more than about 100 tiles
    stays whole (168 tiles in three parts: 210 -> 255 us).  Only splits that leave every part
    an even number of k-tiles, which the kernel's deeper prefetch of W needs."""
    if K % 128 != 0:
        return None
    tiles = ((M + 127) // 128) * ((N + 255) // 256)
    whole = tiles // TILE_PLACES * TILE_PLACES
    tail = tiles - whole
    if whole == 0 or tail == 0 or whole > 2 * TILE_PLACES:
        return None         # (behind three rounds and more the workgroups no longer end together)
    kt = K // 64
    per = 2.0 * 128 * 256 * K
    pair, alone = _TILE128_RATE[10]

    def last_round(workgroups: int, flop: float) -> float:
        return flop / alone if workgroups <= 256 else 2 * flop / pair
    best, best_t = None, 0.8 * last_round(tail, per)
    for split in (2, 4, 8):
        if tail * split > TILE_PLACES or kt % (2 * split) != 0 or kt // split < 8:
            continue
        t = last_round(tail * split, per / split) + 8e-6 + tail * split * 128 * 256 * 4 * 2 / 3e12
        if t < best_t:
            best, best_t = split, t
    return None if best is None else (whole, best)


def _tile128_time(M: int, N: int, K: int, variant: int, ksplit: int) -> float:
    """Estimated seconds of the 128-token tile kernels: rounds of up to 512 tiles, two to a CU
    (a last round of up to 256 tiles runs one to a CU, each faster than two)."""
    bn = 256 if variant in (10, 12) else 128
    tiles = ((M + 127) // 128) * ((N + bn - 1) // bn) * ksplit
    per = 2.0 * 128 * bn * (K / ksplit)
    pair, alone = _TILE128_RATE[variant if ksplit == 1 else 6]
    rem = tiles % 512
    tail = _tile_tail_split(M, N, K) if variant == 10 and ksplit == 1 else None
    if tail is not None:    # the last round split along K, its partials written and read again
        part, wgs = per / tail[1], rem * tail[1]
        last = (part / alone if wgs <= 256 else 2 * part / pair) + 8e-6 \
            + wgs * 128 * 256 * 4 * 2 / 3e12
    else:
        last = 0.0 if rem == 0 else per / alone if rem <= 256 else 2 * per / pair
    t = (tiles // 512) * 2 * per / pair + last
    if ksplit > 1:      # the partials, written and read again, and the second launch
        t += 4e-6 + M * N * 4.0 * ksplit * 2 / 4e12
    return t + 4e-6


@functools.lru_cache(maxsize=None)
def _tile256_variant(M: int, N: int, K: int, accumulate: bool = False):
    """The 256-token tile kernel (20: 256 outputs a tile, 21: 192, 22: 128) if it is expected
    to beat what ``_tile_variant`` and ``_tile_ksplit`` choose by 5 % or more, else None.  One
    workgroup per CU and tile: what counts is how evenly the tiles fill 256 CUs (2048 tokens
    into 6144 outputs are 256 tiles of 256 x 192, where 128 x 128 tiles fill 512 places one
    and a half times: 101 -> 83 us; 14B down at 3072 tokens: 603 -> 441).  Where both kinds
    fill the chip many times over they run equally fast (gate/up at 8192 tokens: 1250 us).
    Times are estimated from rates measured on MI355X; against a sweep of the Qwen3-8B, 14B
    and 32B widths at 512 to 16384 tokens the choice is within 1 % of the best on the whole.
    A residual sum that is split along K keeps its split (the kernel that adds the partials
    also norms)."""
    if M <= 128 or K % 128 != 0 or N % 16 != 0:
        return None
    ks = _tile_ksplit(M, N, K, accumulate)
    if ks > 1 and accumulate:
        return None
    now = _tile128_time(M, N, K, _tile_variant(M, N, True, accumulate, K), ks)
    best = min((20, 21, 22), key=lambda v: _tile256_time(v, M, N, K))
    return best if _tile256_time(best, M, N, K) < 0.95 * now else None


def can_pretile(w: torch.Tensor) -> bool:
    return w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[0] % 64 == 0 \
        and w.shape[1] % 64 == 0


def pretile_weight(w: torch.Tensor) -> torch.Tensor:
    """The bfloat16 kernels' own weight layout, made once at load: [N / 16][K / 64][2][64][8],
    the 16 rows x 64 k of a tile together (2 KB) in the order the lanes of the 16x16x32 MFMA
    pair consume them, so that the weight-streaming kernel reads 1 KB of consecutive memory
    per wave load.  Returned with shape [N, K]; only the kernels know what lies where."""
    N, K = w.shape
    if not can_pretile(w):
        raise KernelUnavailable(f"pretile_weight: bfloat16 [N % 64 == 0, K % 64 == 0], got "
                                f"{tuple(w.shape)} {w.dtype}")
    t = w.view(N // 16, 16, K // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5).contiguous()
    return t.view(N, K)


def _gemm_tile_tail(lib, a, w, out, M: int, N: int, K: int, epi: int, tail) -> None:
    whole, split = tail
    tiles = ((M + 127) // 128) * ((N + 255) // 256)
    if not (0 <= whole < tiles and split >= 2):
        raise KernelUnavailable(f"gemm: tail split {tail} of {tiles} tiles")
    ws = _workspace("gemm_tile_tail", (tiles - whole) * split * 128 * 256, torch.float32, a.device)
    _check(lib.zf_gemm_bf16_tile_tail(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N, K, epi, whole,
                                      split, _stream()), "gemm (tiled, last round split along K)")


@_launches("products")
def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
         w_tiled: bool = False, tile_variant: Optional[int] = None,
         tile_tail: Optional[Tuple[int, int]] = None) -> None:
    """out = a w^T (w is [N, K]); with ``accumulate`` out += a w^T, in 32-bit.  ``w_tiled``:
    ``w`` went through ``pretile_weight``.  ``tile_variant`` (tests and measurements): this
    tiled kernel, whatever the number of rows; ``tile_tail`` (whole, split): the 128 x 256
    tiles with the tiles from ``whole`` on split along K (``_tile_tail_split``).

    bfloat16 operands with K a multiple of 8 go to the MFMA kernels (weight streaming for up
    to 16 rows of ``a``, and up to 64 where the kernel for 17 to 128 rows does not cover the
    sizes; LDS-tiled above); everything else, the whole 32-bit path included,
    goes to the FMA kernel, whose results do not depend on how rows are batched."""
    _need_gpu(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N):
        raise KernelUnavailable(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, "
                                f"out {tuple(out.shape)}")
    if accumulate and out.dtype != torch.float32:
        raise KernelUnavailable("gemm: accumulation needs a float32 output")
    lib = build.load("gemm")
    if w_tiled and not (a.dtype == torch.bfloat16 and can_pretile(w)):
        raise KernelUnavailable("gemm: a pre-tiled weight needs bfloat16 operands")
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and K % 8 == 0 and M > 0:
        epi = _EPI_ACC_F32 if accumulate else \
            (_EPI_STORE_BF16 if out.dtype == torch.bfloat16 else _EPI_STORE_F32)
        plan = _small_plan(M, N, K, w_tiled) if M > 16 else None
        if tile_tail is not None:
            _gemm_tile_tail(lib, a, w, out, M, N, K, epi, tile_tail)
        elif tile_variant is not None:
            _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, epi, tile_variant,
                                         1 if w_tiled else 0, _stream()), "gemm (tiled)")
        elif plan is not None and plan[0] == "mid":
            mid = plan[1]
            ws = _workspace("gemm_splitk", mid * M * N, torch.float32, a.device) if mid > 1 else None
            _check(lib.zf_gemm_bf16_mid(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N, K, epi, mid,
                                        _stream()), "gemm (17 to 128 tokens)")
        elif M <= SKINNY_MAX_M:
            rg, ks = plan[1:] if plan is not None else _skinny_plan(M, N, K, w_tiled)
            ws = _workspace("gemm_splitk", ks * M * N, torch.float32, a.device) if ks > 1 else None
            _check(lib.zf_gemm_bf16_skinny(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N, K, epi,
                                           rg, ks, 1 if w_tiled else 0, _stream()),
                   "gemm (weight streaming)")
        elif w_tiled and _tile64_covers(M, N, K, accumulate):
            _check(lib.zf_gemm_bf16_mid(_ptr(a), _ptr(w), _ptr(out), _ptr(None), M, N, K, epi, 1,
                                        _stream()), "gemm (64-token tiles)")
        else:
            wide = _wide_ksplit(M, N, K) if w_tiled and accumulate else None
            if wide is not None:        # as gemm_sum_norm runs it: the same bits
                ws = _workspace("gemm_splitk", wide * M * N, torch.float32, a.device)
                _check(lib.zf_gemm_bf16_wide_splitk(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N, K,
                                                    epi, wide, _stream()),
                       "gemm (128 x 256 tiles, split along K)")
                return
            big = _tile256_variant(M, N, K, accumulate) if w_tiled else None
            if big is not None:
                _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, epi, big, 1,
                                             _stream()), "gemm (256-token tiles)")
                return
            ksplit = _tile_ksplit(M, N, K, accumulate) if w_tiled else 1
            if ksplit > 1:
                ws = _workspace("gemm_splitk", ksplit * M * N, torch.float32, a.device)
                _check(lib.zf_gemm_bf16_tile_splitk(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N,
                                                    K, epi, ksplit, _stream()),
                       "gemm (tiled, split along K)")
                return
            variant = _tile_variant(M, N, w_tiled, accumulate, K)
            tail = _tile_tail_split(M, N, K) if variant == 10 else None
            if tail is not None:
                _gemm_tile_tail(lib, a, w, out, M, N, K, epi, tail)
                return
            _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, epi, variant,
                                         1 if w_tiled else 0, _stream()),
                   "gemm (tiled)")
        return
    _check(lib.zf_gemm_fma(_ptr(a), _dt(a), _ptr(w), _dt(w), _ptr(out), _dt(out), M, N, K,
                           1 if accumulate else 0, _stream()), "gemm")


def gemm_partials_plan(M: int, N: int, K: int, w: torch.Tensor, w_tiled: bool):
    """Workgroups along K if ``gemm`` would run a stored product a w^T through the kernel for
    17 to 128 tokens split along K (whose partials a second kernel then adds), else None: the
    partials can instead go to a kernel of the caller's that adds them on its way
    (``gemm_partials``)."""
    if not (w_tiled and w.dtype == torch.bfloat16 and w.is_cuda and 16 < M <= MID_MAX_M):
        return None
    plan = _small_plan(M, N, K, True)
    return plan[1] if plan is not None and plan[0] == "mid" and plan[1] > 1 else None


def gemm_partials(a: torch.Tensor, w: torch.Tensor, ksplit: int) -> torch.Tensor:
    """The float32 partials [ksplit, M, N] of a w^T (``w`` pre-tiled, 17 to 128 rows of
    ``a``) in a work buffer that the next split product overwrites; their sum in split order,
    rounded, is what ``gemm`` stores."""
    _need_gpu(a, w)
    M, K = a.shape
    N = w.shape[0]
    if a.dtype != torch.bfloat16 or w.shape[1] != K or not can_pretile(w) \
            or gemm_partials_plan(M, N, K, w, True) != ksplit:
        raise KernelUnavailable("gemm_partials: not a product that gemm_partials_plan covers")
    ws = _workspace("gemm_splitk", ksplit * M * N, torch.float32, a.device)
    lib = build.load("gemm")
    if not _left_out("products"):
        global _launch_count
        _launch_count += 1
        _check(lib.zf_gemm_bf16_mid_partials(_ptr(a), _ptr(w), _ptr(ws), M, N, K, ksplit,
                                             _stream()), "gemm_partials")
    return ws[:ksplit * M * N].view(ksplit, M, N)


gemm_partials.kernel_class = "products"     # (it hands its work buffer on even when left out)


def norm_gemm_plan(M: int, N: int, K: int, w: torch.Tensor, w_tiled: bool):
    """Row groups per workgroup if ``norm_gemm`` covers the product (the weight-streaming
    kernel without a split over workgroups on a pre-tiled bfloat16 weight), else None."""
    # beyond 16 tokens the lanes' extra work (32-bit rows, gains, conversions for every group
    # of 16 tokens) costs more than the norm kernel it saves (measured)
    if not (w_tiled and 0 < M <= NORM_FOLD_MAX_M and w.dtype == torch.bfloat16):
        return None
    rg, ks = _skinny_plan(M, N, K, True)
    return rg if ks == 1 else None


@_launches("products")
def norm_gemm(x: torch.Tensor, gain: torch.Tensor, eps: float, w: torch.Tensor,
              out: torch.Tensor, swiglu: bool = False) -> None:
    """out = rmsnorm(x, gain, eps) w^T with the norm folded into the weight-streaming product
    (``w`` pre-tiled; with ``swiglu`` the rows of ``w`` alternate gate / up as for
    ``gemm_swiglu`` and out is [M, N / 2]).  x float32 [M <= 64, K]; the sum of squares, the
    scale and the product's sums are 32-bit, the MFMA operands bfloat16(x * gain)."""
    _need_gpu(x, gain, w, out)
    M, K = x.shape
    N = w.shape[0]
    rg = norm_gemm_plan(M, N, K, w, True)
    if swiglu and 0 < M <= SKINNY_MAX_M:
        rg = 4 if (M > 16 and N >= 16384) else 2
    if rg is None or x.dtype != torch.float32 or gain.dtype != torch.float32 \
            or gain.shape != (K,) or w.shape[1] != K or not can_pretile(w) \
            or out.shape != (M, N // 2 if swiglu else N) \
            or (swiglu and out.dtype != torch.bfloat16):
        raise KernelUnavailable(f"norm_gemm: x {tuple(x.shape)} {x.dtype}, w {tuple(w.shape)}, "
                                f"out {tuple(out.shape)} {out.dtype}")
    epi = _EPI_SWIGLU if swiglu else \
        (_EPI_STORE_BF16 if out.dtype == torch.bfloat16 else _EPI_STORE_F32)
    lib = build.load("gemm")
    _check(lib.zf_norm_gemm_bf16_skinny(_ptr(x), _ptr(gain), ctypes.c_float(eps), _ptr(w),
                                        _ptr(out), M, N, K, epi, rg, _stream()), "norm_gemm")


def sum_norm_plan(M: int, N: int, K: int, w: torch.Tensor, w_tiled: bool):
    """The plan if ``gemm_sum_norm`` covers residual += a w^T: a product that is split along K
    anyway (by measurement at 1 to 64 tokens, by rule at 17 to 128, or a few hundred tokens on
    a narrow output), whose partials one kernel can add, sum into the residual and norm; else
    None.  ('mid' | 'tile' | 'wide' | 'skinny', [row groups per workgroup,] workgroups along K)."""
    if not (w_tiled and w.dtype == torch.bfloat16 and w.is_cuda and N % 16 == 0 and N <= 8192):
        return None
    if M <= NORM_FOLD_MAX_M:
        return _decode_acc_plan(M, N, K)
    if M <= MID_MAX_M:
        plan = _small_plan(M, N, K, True)
        return plan if plan is not None and plan[-1] >= 2 else None
    wide = _wide_ksplit(M, N, K)
    if wide is not None:
        return ("wide", wide)
    ks = _tile_ksplit(M, N, K)
    return ("tile", ks) if ks >= 2 else None


def _wide_ksplit(M: int, N: int, K: int):
    """Workgroups along K if a residual sum with the norm behind it should run through 128 x
    256 tiles split along K: 641 to 1280 tokens on a long K, where those tiles alone leave
    half the chip idle (1024 tokens into 4096 outputs: 128 of them) and the 128 x 128 tiles,
    split or not, are slower per flop.  Two to four parts of an even number of k-tiles each,
    as close to 512 workgroups as they get.  Measured on MI355X against what ran before (the
    norm's kernel included): K = 12288 into 4096 at 768 / 1024 / 1280 tokens 113 -> 107, 133
    -> 113, 171 -> 143 us; K = 17408 into 5120 174 -> 149, 222 -> 209, 254 -> 244; K = 25600
    253 -> 205 and 314 -> 289.  With K = 4096 or 5120 the partials cost what the split gains,
    and from 1536 tokens on the tiles fill the chip without it."""
    if not (640 < M <= 1280 and K >= 8192 and K % 128 == 0 and N % 16 == 0):
        return None
    tiles = ((M + 127) // 128) * ((N + 255) // 256)
    fits = [ks for ks in (2, 3, 4) if (K // 64) % (2 * ks) == 0]
    return min(fits, key=lambda ks: abs(tiles * ks - TILE_PLACES)) if fits else None


@_launches("products")
def gemm_sum_norm(a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, gain: torch.Tensor,
                  eps: float, normed: torch.Tensor) -> None:
    """residual += a w^T in 32-bit (``w`` pre-tiled) and normed = bfloat16(rmsnorm(residual,
    gain, eps)), the norm from the kernel that adds the product's partials."""
    _need_gpu(a, w, residual, gain, normed)
    M, K = a.shape
    N = w.shape[0]
    plan = sum_norm_plan(M, N, K, w, True)
    if plan is None or a.dtype != torch.bfloat16 or w.shape[1] != K or not can_pretile(w) \
            or residual.shape != (M, N) or residual.dtype != torch.float32 \
            or gain.shape != (N,) or gain.dtype != torch.float32 \
            or normed.shape != (M, N) or normed.dtype != torch.bfloat16 \
            or not all(t.is_contiguous() for t in (a, residual, normed)):
        raise KernelUnavailable(f"gemm_sum_norm: a {tuple(a.shape)} {a.dtype}, w "
                                f"{tuple(w.shape)}, residual {tuple(residual.shape)} "
                                f"{residual.dtype}")
    ks = plan[-1]
    ws = _workspace("gemm_splitk", ks * M * N, torch.float32, a.device)
    lib = build.load("gemm")
    if plan[0] == "wide":
        _check(lib.zf_gemm_bf16_wide_splitk_sum_norm(_ptr(a), _ptr(w), _ptr(residual), _ptr(ws),
                                                     _ptr(gain), ctypes.c_float(eps), _ptr(normed),
                                                     M, N, K, ks, _stream()),
               "gemm_sum_norm (128 x 256 tiles)")
    elif plan[0] == "skinny":
        _check(lib.zf_gemm_bf16_skinny_sum_norm(_ptr(a), _ptr(w), _ptr(residual), _ptr(ws),
                                                _ptr(gain), ctypes.c_float(eps), _ptr(normed), M, N,
                                                K, plan[1], ks, _stream()),
               "gemm_sum_norm (weight streaming)")
    else:
        _check(lib.zf_gemm_bf16_splitk_sum_norm(_ptr(a), _ptr(w), _ptr(residual), _ptr(ws),
                                                _ptr(gain), ctypes.c_float(eps), _ptr(normed), M, N,
                                                K, ks, _stream()), "gemm_sum_norm")


def norm_emit_plan(M: int, N: int, K: int, w: torch.Tensor, w_tiled: bool):
    """Row groups per workgroup if ``gemm_emit`` covers out += a w^T (weight-streaming kernel,
    up to 16 tokens, pre-tiled bfloat16 weight, no split over workgroups), else None."""
    if not (w_tiled and 0 < M <= NORM_FOLD_MAX_M and w.dtype == torch.bfloat16 and w.is_cuda):
        return None
    if N <= 8192 and _decode_acc_plan(M, N, K) is not None:
        return None             # measured: the split along K with the norm in its reduce is faster
    rg, ks = _skinny_plan(M, N, K, True)
    return rg if (ks == 1 and rg <= 2) else None


@_launches("products")
def gemm_emit(a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, gain: torch.Tensor,
              xg: torch.Tensor, sq: torch.Tensor) -> None:
    """residual += a w^T in 32-bit (``w`` pre-tiled) and, for the RMSNorm that reads the sum
    next, from the same epilogue: xg = bfloat16(residual * gain) [M, N] and sq [N / 16, 16] =
    the sums of residual^2 over each 16 columns per token, which ``gemm_given`` takes."""
    _need_gpu(a, w, residual, gain, xg, sq)
    M, K = a.shape
    N = w.shape[0]
    rg = norm_emit_plan(M, N, K, w, True)
    if rg is None or a.dtype != torch.bfloat16 or w.shape[1] != K or not can_pretile(w) \
            or residual.shape != (M, N) or residual.dtype != torch.float32 \
            or gain.shape != (N,) or gain.dtype != torch.float32 \
            or xg.shape != (M, N) or xg.dtype != torch.bfloat16 \
            or sq.shape != (N // 16, 16) or sq.dtype != torch.float32 \
            or not all(t.is_contiguous() for t in (a, residual, xg, sq)):
        raise KernelUnavailable(f"gemm_emit: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)}, "
                                f"residual {tuple(residual.shape)} {residual.dtype}")
    lib = build.load("gemm")
    _check(lib.zf_gemm_bf16_skinny_emit(_ptr(a), _ptr(w), _ptr(residual), _ptr(gain), _ptr(xg),
                                        _ptr(sq), M, N, K, rg, _stream()), "gemm_emit")


@_launches("products")
def gemm_given(xg: torch.Tensor, sq: torch.Tensor, eps: float, w: torch.Tensor,
               out: torch.Tensor, swiglu: bool = False) -> None:
    """out = rmsnorm(x) w^T from what ``gemm_emit`` left of x: xg = bfloat16(x * gain) and the
    partial sums of squares sq [groups, 16]; the token's 1 / sqrt(mean(x^2) + eps) scales the
    32-bit sums of the product.  With ``swiglu`` as ``gemm_swiglu``."""
    _need_gpu(xg, sq, w, out)
    M, K = xg.shape
    N = w.shape[0]
    rg = norm_gemm_plan(M, N, K, w, True)
    if swiglu and 0 < M <= NORM_FOLD_MAX_M:
        rg = 2
    if rg is None or xg.dtype != torch.bfloat16 or sq.dtype != torch.float32 \
            or sq.dim() != 2 or sq.shape[1] != 16 or sq.shape[0] * 16 != K \
            or w.shape[1] != K or not can_pretile(w) \
            or out.shape != (M, N // 2 if swiglu else N) \
            or (swiglu and out.dtype != torch.bfloat16) \
            or not all(t.is_contiguous() for t in (xg, sq, out)):
        raise KernelUnavailable(f"gemm_given: xg {tuple(xg.shape)} {xg.dtype}, w {tuple(w.shape)}, "
                                f"out {tuple(out.shape)} {out.dtype}")
    epi = _EPI_SWIGLU if swiglu else \
        (_EPI_STORE_BF16 if out.dtype == torch.bfloat16 else _EPI_STORE_F32)
    lib = build.load("gemm")
    _check(lib.zf_gemm_bf16_skinny_given(_ptr(xg), _ptr(sq), sq.shape[0], ctypes.c_float(eps),
                                         _ptr(w), _ptr(out), M, N, K, epi, rg, _stream()),
           "gemm_given")


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of the gate and the up projection alternating in groups of 16 (gate 0..15, up
    0..15, gate 16..31, ...): the order ``gemm_swiglu`` wants.  Needs I % 16 == 0."""
    I, K = gate.shape
    return torch.stack([gate.view(I // 16, 16, K), up.view(I // 16, 16, K)], dim=1) \
        .reshape(2 * I, K).contiguous()


def can_fuse_swiglu(w: torch.Tensor) -> bool:
    return w.is_cuda and w.dtype == torch.bfloat16 and w.shape[0] % 64 == 0 and w.shape[1] % 8 == 0


@_launches("products")
def gemm_swiglu(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, w_tiled: bool = False,
                tile_variant: Optional[int] = None,
                tile_tail: Optional[Tuple[int, int]] = None) -> None:
    """out[M, I] = silu(a Wg^T) * (a Wu^T) as bfloat16, with ``w`` [2 I, K] from
    ``interleave_gate_up`` (then possibly ``pretile_weight``): the activation is applied to
    the 32-bit sums in the product's epilogue, nothing of width 2 I is written."""
    _need_gpu(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N // 2) or out.dtype != torch.bfloat16 \
            or a.dtype != torch.bfloat16 or not can_fuse_swiglu(w):
        raise KernelUnavailable(f"gemm_swiglu: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} "
                                f"{w.dtype}, out {tuple(out.shape)} {out.dtype}")
    if M == 0:
        return
    lib = build.load("gemm")
    plan = _small_plan(M, N, K, w_tiled, swiglu=True) if M > 16 else None
    if tile_tail is not None:
        _gemm_tile_tail(lib, a, w, out, M, N, K, _EPI_SWIGLU, tile_tail)
    elif tile_variant is not None:
        _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, _EPI_SWIGLU,
                                     tile_variant, 1 if w_tiled else 0, _stream()),
               "gemm_swiglu (tiled)")
    elif plan is not None and plan[0] == "mid":
        _check(lib.zf_gemm_bf16_mid(_ptr(a), _ptr(w), _ptr(out), _ptr(None), M, N, K, _EPI_SWIGLU,
                                    1, _stream()), "gemm_swiglu (17 to 128 tokens)")
    elif M <= SKINNY_MAX_M:
        rg = plan[1] if plan is not None else 2
        _check(lib.zf_gemm_bf16_skinny(_ptr(a), _ptr(w), _ptr(out), _ptr(None), M, N, K,
                                       _EPI_SWIGLU, rg, 1, 1 if w_tiled else 0, _stream()),
               "gemm_swiglu (weight streaming)")
    else:
        big = _tile256_variant(M, N, K) if w_tiled else None
        variant = big if big is not None else _tile_variant(M, N, w_tiled, False, K)
        tail = _tile_tail_split(M, N, K) if variant == 10 else None
        if tail is not None:
            _gemm_tile_tail(lib, a, w, out, M, N, K, _EPI_SWIGLU, tail)
            return
        _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, _EPI_SWIGLU, variant,
                                     1 if w_tiled else 0, _stream()),
               "gemm_swiglu (tiled)")


# ------------------------------------------------------------------------- attention
MAX_HEAD_DIM = 512          # the wave kernel keeps a head in registers: 8 values a lane
DECODE_SPLIT_KEYS = 256     # keys per split of the decode kernel (DEC_SPLIT in attention.hip)
PREFILL_QUERY_TILE = 32     # queries per tile of the kernels for prompt portions


def mfma_attention_covers(dtype, n_heads, n_kv_heads, head_dim, page_size) -> bool:
    """Whether the bfloat16 MFMA attention kernels serve this shape.  If so, the pools are
    kept in those kernels' own order inside every group of 16 rows (keys ``[hd / 32][16 *
    ((d % 32) / 8) + row][d % 8]``, values ``[hd / 16][16 * (row / 4) + d % 16][row % 4]``);
    otherwise keys are ``[row][hd]`` and values ``[hd][row]`` inside a (page, kv head) block."""
    return dtype == torch.bfloat16 and head_dim in (32, 64, 128, 256) and page_size % 16 == 0 \
        and n_heads // n_kv_heads <= 16


# Up to this many sequences a decode step's attention does the work of qk_norm_rope_kv_write
# itself.  Measured on MI355X (Qwen3-8B shape, context 2100, per layer, against the two kernels
# one after the other): 11.2 -> 8.2 us at batch 1, 15.0 -> 13.1 at 4, 19.1 -> 18.2 at 8,
# 30.2 -> 29.3 at 16, 51.0 -> 50.0 at 32, but 94.6 -> 95.7 at 64, where the chip is busy
# streaming keys and values and a workgroup's longer start costs more than a launch.  At
# context 32768 it gains at batch 1, 8 and 16 alike (245 -> 255, 853 -> 864, 1008 -> 1012
# tokens/s): there one workgroup in 128 also norms and stores a key, at context 2100 one in 9.
FUSED_DECODE_MAX_SEQS = 32


@_launches("attention")
def decode_attention_fused(qkv, q_gain, k_gain, eps, cos, sin, positions, slot_mapping, k_pool,
                           v_pool, block_table, q_start, ctx_len, out, scale, window, n_heads,
                           n_kv_heads, head_dim, page_size, max_ctx_len) -> None:
    """A decode step's attention straight from the q/k/v product: every sequence has exactly
    one token (token s is sequence s's), ``qkv`` [n_seqs, (nH + 2 nKV) hd] is read and not
    changed.  What ``qk_norm_rope_kv_write`` and ``paged_attention`` do one after the other
    (per-head RMSNorm of q and k, rotation at ``positions``, the token's key and value into the
    pools at ``slot_mapping``, attention over the cache) in one kernel less, with the same
    arithmetic and so the same bits.  Only for shapes ``mfma_attention_covers``."""
    _need_gpu(qkv, q_gain, k_gain, cos, sin, positions, slot_mapping, k_pool, v_pool, block_table,
              q_start, ctx_len, out)
    n_seqs = ctx_len.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if not mfma_attention_covers(qkv.dtype, n_heads, n_kv_heads, head_dim, page_size):
        raise KernelUnavailable("decode_attention_fused: bfloat16, head_dim 32/64/128/256, pages "
                                "of a multiple of 16 rows and at most 16 query heads per kv head")
    if qkv.shape != (n_seqs, width) or out.shape != (n_seqs, n_heads * head_dim) \
            or out.dtype != qkv.dtype or k_pool.dtype != qkv.dtype or v_pool.dtype != qkv.dtype:
        raise KernelUnavailable("decode_attention_fused: qkv must be [n_seqs, (nH + 2 nKV) * hd] "
                                "and out [n_seqs, nH * hd], of the pools' dtype")
    if (q_gain is None) != (k_gain is None) or (cos is None) != (sin is None):
        raise KernelUnavailable("decode_attention_fused: gains and tables come in pairs")
    for g in (q_gain, k_gain):
        if g is not None and (g.dtype != torch.float32 or g.shape != (head_dim,)):
            raise KernelUnavailable("decode_attention_fused: a gain must be float32 [head_dim]")
    if cos is not None and (cos.dtype != torch.float32 or cos.shape[1] != head_dim // 2
                            or cos.shape != sin.shape):
        raise KernelUnavailable("decode_attention_fused: tables must be float32 [*, head_dim/2]")
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (ctx_len, "ctx_len"),
                    (positions, "positions"), (slot_mapping, "slot_mapping")):
        _i32(t, name)
    if q_start.shape[0] != n_seqs + 1 or block_table.shape[0] != n_seqs \
            or positions.shape[0] != n_seqs or slot_mapping.shape[0] != n_seqs:
        raise KernelUnavailable("decode_attention_fused: per-sequence arrays disagree in length")
    if max_ctx_len > block_table.shape[1] * page_size:
        raise KernelUnavailable("decode_attention_fused: block table shorter than the context")
    max_splits = (max_ctx_len + DECODE_SPLIT_KEYS - 1) // DECODE_SPLIT_KEYS
    ws_o = _workspace("attn_o", n_seqs * n_heads * max_splits * head_dim, torch.float32,
                      qkv.device)
    ws_ml = _workspace("attn_ml", n_seqs * n_heads * max_splits * 2, torch.float32, qkv.device)
    lib = build.load("attention")
    _check(lib.zf_attn_decode_fused_bf16(
        _ptr(qkv), _ptr(q_gain), _ptr(k_gain), ctypes.c_float(eps), _ptr(cos), _ptr(sin),
        0 if cos is None else cos.shape[0],
        _ptr(positions), _ptr(slot_mapping), _ptr(k_pool), _ptr(v_pool), _ptr(block_table),
        _ptr(q_start), _ptr(ctx_len), _ptr(out), _ptr(ws_o), _ptr(ws_ml), ctypes.c_float(scale),
        int(window), n_seqs, n_heads, n_kv_heads, head_dim, page_size, block_table.shape[1],
        max_splits, _stream()), "decode_attention_fused")


def _prefill_key_split(n_query_tiles: int, n_kv_heads: int, max_ctx_len: int):
    """(keys per split, splits) if a prompt portion's attention should also split its keys over
    workgroups: few query tiles behind a long context (a 512-token portion at context 4096: 128
    workgroups that walk up to 128 key tiles each) leave half the chip idle and the rest
    waiting on one chain of tiles.  Splits of at least 512 keys, about 512 workgroups; from
    2048 keys on (measured, 481 queries of 40 heads on 8: 4096 keys 223 -> 151 us, 8192 keys
    443 -> 259 us; at 1024 keys the partials cost what the split gains)."""
    wgs = n_query_tiles * n_kv_heads
    if wgs <= 0 or wgs >= 384 or max_ctx_len < 2048:
        return None
    want = (512 + wgs - 1) // wgs
    keys = max(512, ((max_ctx_len + want - 1) // want + 63) // 64 * 64)
    splits = (max_ctx_len + keys - 1) // keys
    return (keys, splits) if splits >= 2 else None


@_launches("attention")
def paged_attention(q, k_pool, v_pool, block_table, q_start, ctx_len, seq_index, out, scale,
                    window, n_heads, n_kv_heads, head_dim, page_size, max_q_len,
                    max_ctx_len, n_single=None, n_query_tiles=None, q_tile_map=None,
                    prefill_max_ctx=None, prefill_variant=0) -> None:
    """Causal grouped-query attention of the step's tokens over the paged cache.  Token t of
    sequence s = seq_index[t] has position ctx_len[s] - q_len[s] + (t - q_start[s]) and reads
    the positions up to its own (the last ``window`` of them if window > 0).  ``n_single`` is
    the number of sequences with exactly one token in this step (None: unknown),
    ``n_query_tiles`` the number of 32-query tiles of the others, ``q_tile_map`` their int32
    (sequence, tile) pairs [n_query_tiles, 2] and ``prefill_max_ctx`` the longest context among
    those sequences (None: unknown): they only decide how the work is cut.
    ``prefill_variant`` picks the kernel for the portions (0: by size; 1: every wave fetches
    its keys and values; 2: they are staged in LDS for a group's heads), for measurements and
    tests.

    bfloat16 with head_dim 32/64/128/256 and a page size that is a multiple of 16 runs the
    MFMA kernels: split-context decode for single tokens, the tiled kernel for portions.
    Everything else runs the 32-bit wave kernel."""
    _need_gpu(q, k_pool, v_pool, block_table, q_start, ctx_len, seq_index, out)
    T = q.shape[0]
    if q.shape != (T, n_heads * head_dim) or out.shape != q.shape or out.dtype != q.dtype \
            or k_pool.dtype != q.dtype or v_pool.dtype != q.dtype:
        raise KernelUnavailable("paged_attention: q/out must be [T, nH * hd] of the pools' dtype")
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (ctx_len, "ctx_len"),
                    (seq_index, "seq_index")):
        _i32(t, name)
    if n_heads % n_kv_heads != 0:
        raise KernelUnavailable("paged_attention: InvalidGrouping")
    if head_dim > MAX_HEAD_DIM:
        raise KernelUnavailable(f"paged_attention: head_dim {head_dim} > {MAX_HEAD_DIM} is not "
                                "covered")
    if max_ctx_len > block_table.shape[1] * page_size:
        raise KernelUnavailable("paged_attention: block table shorter than the context")
    n_seqs = ctx_len.shape[0]
    if q_start.shape[0] != n_seqs + 1 or block_table.shape[0] != n_seqs or seq_index.shape[0] != T:
        raise KernelUnavailable("paged_attention: per-sequence arrays disagree in length")
    lib = build.load("attention")
    max_pages = block_table.shape[1]
    if mfma_attention_covers(q.dtype, n_heads, n_kv_heads, head_dim, page_size):
        if n_single is None:
            n_single = n_seqs if max_q_len == 1 else -1      # -1: some, not known how many
        if n_single != 0:
            max_splits = (max_ctx_len + DECODE_SPLIT_KEYS - 1) // DECODE_SPLIT_KEYS
            ws_o = _workspace("attn_o", n_seqs * n_heads * max_splits * head_dim, torch.float32,
                              q.device)
            ws_ml = _workspace("attn_ml", n_seqs * n_heads * max_splits * 2, torch.float32,
                               q.device)
            _check(lib.zf_attn_decode_bf16(
                _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), _ptr(q_start),
                _ptr(ctx_len), _ptr(out), _ptr(ws_o), _ptr(ws_ml), ctypes.c_float(scale),
                int(window), n_seqs, n_heads, n_kv_heads, head_dim, page_size, max_pages,
                max_splits, _stream()), "paged_attention (decode)")
        if n_single != n_seqs and max_q_len > 1:
            if q_tile_map is not None:
                _i32(q_tile_map, "q_tile_map")
                if n_query_tiles is None or q_tile_map.shape != (n_query_tiles, 2) \
                        or not q_tile_map.is_cuda or not q_tile_map.is_contiguous():
                    raise KernelUnavailable("paged_attention: q_tile_map must be int32 "
                                            "[n_query_tiles, 2] on the device")
            split = _prefill_key_split(n_query_tiles, n_kv_heads,
                                       prefill_max_ctx if prefill_max_ctx is not None
                                       else max_ctx_len) \
                if n_query_tiles is not None else None
            if split is not None and T * n_heads * split[1] * (head_dim + 2) * 4 > (1 << 28):
                split = None
            ws_o = ws_ml = None
            if split is not None:
                ws_o = _workspace("attn_pre_o", T * n_heads * split[1] * head_dim, torch.float32,
                                  q.device)
                ws_ml = _workspace("attn_pre_ml", T * n_heads * split[1] * 2, torch.float32,
                                   q.device)
            _check(lib.zf_attn_prefill_bf16(
                _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), _ptr(q_start),
                _ptr(ctx_len), _ptr(out), ctypes.c_float(scale), int(window), n_seqs,
                max_q_len, n_heads, n_kv_heads, head_dim, page_size, max_pages,
                1 if n_single != 0 else 0, 1 if max_ctx_len <= 2 * max_q_len else 0,
                _ptr(seq_index), T, _ptr(ws_o), _ptr(ws_ml),
                split[0] if split is not None else 0, split[1] if split is not None else 0,
                _ptr(q_tile_map), n_query_tiles if q_tile_map is not None else 0,
                int(prefill_variant), _stream()), "paged_attention (prefill)")
        return
    _check(lib.zf_paged_attention_wave(
        _ptr(q), _ptr(k_pool), _ptr(v_pool), _dt(q), _ptr(block_table), _ptr(q_start),
        _ptr(ctx_len), _ptr(seq_index), _ptr(out), ctypes.c_float(scale), int(window), T,
        n_heads, n_kv_heads, head_dim, page_size, max_pages, _stream()),
        "paged_attention")


# ------------------------------------------------------------------------- norms with a bias
@_launches("norm_rope_write")
def norm_rows(x: torch.Tensor, gain: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
              out: torch.Tensor, centred: bool = True, add: bool = False) -> None:
    """Row by row over float32 ``x`` [T, W], all in 32-bit: centred,
    n = (x - mean) / sqrt(mean((x - mean)^2) + eps) * gain + bias (a layer norm); not centred,
    n = x / sqrt(mean(x^2) + eps) * gain (+ bias).  ``out`` = n (float32 or bfloat16), or with
    ``add`` out += n (float32: a branch's normed output joins the residual stream)."""
    _need_gpu(x, gain, bias, out)
    T, W = x.shape
    if x.dtype != torch.float32 or gain.dtype != torch.float32 or gain.shape != (W,) \
            or out.shape != x.shape or (bias is not None and (bias.dtype != torch.float32
                                                              or bias.shape != (W,))) \
            or (add and out.dtype != torch.float32):
        raise KernelUnavailable(f"norm_rows: x {tuple(x.shape)} {x.dtype}, gain "
                                f"{tuple(gain.shape)} {gain.dtype}, out {tuple(out.shape)} "
                                f"{out.dtype} (float32 when added to)")
    lib = build.load("norms")
    _check(lib.zf_norm_rows(_ptr(x), _ptr(gain), _ptr(bias), _ptr(out), _dt(out), T, W,
                            ctypes.c_float(eps), 1 if centred else 0, 1 if add else 0,
                            _stream()), "norm_rows")


NORM_ADD_NORM_MAX_WIDTH = 8192


def norm_add_norm_covers(width: int) -> bool:
    return width % 4 == 0 and 0 < width <= NORM_ADD_NORM_MAX_WIDTH


@_launches("norm_rope_write")
def norm_add_norm(y: torch.Tensor, gain_a, bias_a, eps_a: float, centred_a: bool,
                  x: torch.Tensor, gain_b, bias_b, eps_b: float, centred_b: bool,
                  out: torch.Tensor) -> None:
    """x += norm_a(y); out = norm_b(x), row by row in 32-bit (``norm_rows`` with ``add`` and then
    ``norm_rows``, in one kernel, the same numbers): the norm behind a sublayer and the norm
    before the next one.  ``y`` and ``x`` float32 [T, W], W a multiple of 4 up to 8192."""
    _need_gpu(y, gain_a, bias_a, x, gain_b, bias_b, out)
    T, W = x.shape
    vecs = [v for v in (gain_a, bias_a, gain_b, bias_b) if v is not None]
    if y.shape != x.shape or out.shape != x.shape or y.dtype != torch.float32 \
            or x.dtype != torch.float32 or gain_a is None or gain_b is None \
            or any(v.dtype != torch.float32 or v.shape != (W,) for v in vecs) \
            or not norm_add_norm_covers(W):
        raise KernelUnavailable(f"norm_add_norm: float32 rows {tuple(y.shape)} and "
                                f"{tuple(x.shape)}, float32 [W] gains and biases, W a multiple "
                                f"of 4 up to {NORM_ADD_NORM_MAX_WIDTH}")
    lib = build.load("norms")
    _check(lib.zf_norm_add_norm(_ptr(y), _ptr(gain_a), _ptr(bias_a), ctypes.c_float(eps_a),
                                1 if centred_a else 0, _ptr(x), _ptr(gain_b), _ptr(bias_b),
                                ctypes.c_float(eps_b), 1 if centred_b else 0, _ptr(out), _dt(out),
                                T, W, _stream()), "norm_add_norm")


@_launches("other")
def embed_position(table: torch.Tensor, ids: torch.Tensor, pos_table: torch.Tensor,
                   positions: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[t, :] = table[ids[t], :] * scale + pos_table[positions[t], :], in float32."""
    _need_gpu(table, ids, pos_table, positions, out)
    _i32(ids, "ids")
    _i32(positions, "positions")
    T, H = out.shape
    if table.shape[1] != H or pos_table.shape[1] != H or table.dtype != pos_table.dtype \
            or ids.shape[0] != T or positions.shape[0] != T or out.dtype != torch.float32:
        raise KernelUnavailable(f"embed_position: table {tuple(table.shape)} {table.dtype}, "
                                f"positions' table {tuple(pos_table.shape)} {pos_table.dtype}, "
                                f"out {tuple(out.shape)} {out.dtype}")
    lib = build.load("norms")
    _check(lib.zf_embed_position(_ptr(table), _ptr(pos_table), _dt(table), _ptr(ids),
                                 _ptr(positions), _ptr(out), T, H, ctypes.c_float(scale),
                                 _stream()), "embed_position")


# ------------------------------------------------------------------------- attention whose values are its keys
def _columns(t: torch.Tensor, what: str) -> int:
    """Row stride (in elements) of a 2-D tensor whose rows are contiguous: a slice of columns
    of a wider product."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelUnavailable(f"{what} must be a matrix with contiguous rows")
    return t.stride(0)


@_launches("norm_rope_write")
def kv_rows_write(rows: torch.Tensor, slot_mapping: torch.Tensor, k_pool: torch.Tensor,
                  n_kv_heads: int, head_dim: int, page_size: int) -> None:
    """rows [T, nKV * hd] (contiguous rows, any row stride: columns of a wider product) go
    into the pool laid out [page, kv head, row, hd] at ``slot_mapping``."""
    for t in (rows, slot_mapping, k_pool):
        if not t.is_cuda:
            raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    _i32(slot_mapping, "slot_mapping")
    T = rows.shape[0]
    stride = _columns(rows, "kv_rows_write: rows")
    if rows.shape[1] != n_kv_heads * head_dim or rows.dtype != k_pool.dtype \
            or slot_mapping.shape[0] != T or not k_pool.is_contiguous() \
            or k_pool.numel() % (n_kv_heads * head_dim * page_size) != 0:
        raise KernelUnavailable(f"kv_rows_write: rows {tuple(rows.shape)} {rows.dtype} for "
                                f"{n_kv_heads} heads of {head_dim}, pool {k_pool.dtype}")
    lib = build.load("sink_attention")
    _check(lib.zf_kv_rows_write(_ptr(rows), _dt(rows), ctypes.c_longlong(stride), 0,
                                _ptr(slot_mapping), _ptr(k_pool), T, n_kv_heads, head_dim,
                                page_size, _stream()), "kv_rows_write")


@_launches("attention")
def shared_kv_attention(q: torch.Tensor, gate: Optional[torch.Tensor], k_pool: torch.Tensor,
                        block_table, q_start, ctx_len, seq_index, out: torch.Tensor,
                        scale: float, window: int, sink: bool, n_heads: int, n_kv_heads: int,
                        head_dim: int, page_size: int, max_ctx_len: int) -> None:
    """Causal grouped-query attention whose values are the keys, over a paged pool of keys
    [page, kv head, row, hd].  Token t of sequence s = seq_index[t] has position ctx_len[s] -
    q_len[s] + (t - q_start[s]) and reads the positions up to its own (the last ``window`` of
    them if window > 0).  ``sink``: the soft-max's denominator holds one more term, exp(0).
    ``gate`` [T, nH * hd]: the output is multiplied by sigmoid(gate).  ``q`` and ``gate`` may
    be column slices of a wider product.  Scores and weights are 32-bit in both dtypes."""
    for t in (q, gate, k_pool, block_table, q_start, ctx_len, seq_index, out):
        if t is not None and not t.is_cuda:
            raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    T = q.shape[0]
    qs = _columns(q, "shared_kv_attention: q")
    gs = _columns(gate, "shared_kv_attention: gate") if gate is not None else 0
    if q.shape[1] != n_heads * head_dim or out.shape != (T, n_heads * head_dim) \
            or not out.is_contiguous() or out.dtype != q.dtype or k_pool.dtype != q.dtype \
            or (gate is not None and (gate.shape != q.shape or gate.dtype != q.dtype)):
        raise KernelUnavailable("shared_kv_attention: q, gate and out must be [T, nH * hd] of "
                                "the pool's dtype")
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (ctx_len, "ctx_len"),
                    (seq_index, "seq_index")):
        _i32(t, name)
    if n_kv_heads <= 0 or n_heads % n_kv_heads != 0:
        raise KernelUnavailable("shared_kv_attention: InvalidGrouping")
    if not 0 < head_dim <= MAX_HEAD_DIM:
        raise KernelUnavailable(f"shared_kv_attention: head_dim {head_dim} is not in 1.."
                                f"{MAX_HEAD_DIM}")
    if max_ctx_len > block_table.shape[1] * page_size:
        raise KernelUnavailable("shared_kv_attention: block table shorter than the context")
    n_seqs = ctx_len.shape[0]
    if q_start.shape[0] != n_seqs + 1 or block_table.shape[0] != n_seqs \
            or seq_index.shape[0] != T or not block_table.is_contiguous():
        raise KernelUnavailable("shared_kv_attention: per-sequence arrays disagree in length")
    lib = build.load("sink_attention")
    _check(lib.zf_shared_kv_attention(
        _ptr(q), ctypes.c_longlong(qs), _ptr(gate), ctypes.c_longlong(gs), _ptr(k_pool), _dt(q),
        _ptr(block_table), _ptr(q_start), _ptr(ctx_len), _ptr(seq_index), _ptr(out),
        ctypes.c_float(scale), int(window), 1 if sink else 0, T, n_heads, n_kv_heads, head_dim,
        page_size, block_table.shape[1], _stream()), "shared_kv_attention")


TIED_MFMA_HEAD_DIMS = (32, 64, 96, 128, 192, 256)
TIED_MFMA_ROWS = 128          # (position, head) pairs a workgroup of the MFMA kernel takes
TIED_SPLIT_KEYS = 256         # least keys a split of a decode step's context holds
TIED_SPLIT_WORKGROUPS = 512   # splits are made until about this many workgroups run
TIED_ROWS_WAVES = 2048        # a prompt portion's keys are cut in parts until this many waves run
TIED_ROWS_MAX_PARTS = 4
TIED_DECODE_WORKGROUPS = 1024  # the same for the decode kernel (whose every wave is a split)


def tied_attention_mfma_covers(dtype, n_heads: int, n_kv_heads: int, head_dim: int) -> bool:
    """Whether the bfloat16 MFMA kernel for attention whose values are its keys takes the
    shape; otherwise (and in 32-bit) ``shared_kv_attention``'s kernel runs."""
    return dtype == torch.bfloat16 and head_dim in TIED_MFMA_HEAD_DIMS \
        and n_heads // n_kv_heads <= TIED_MFMA_ROWS


def tied_attention(q, gate, k_pool, block_table, q_start, ctx_len, seq_index, out, scale, window,
                   sink, n_heads, n_kv_heads, head_dim, page_size, max_q_len, max_ctx_len) -> None:
    """``shared_kv_attention`` through the fastest kernel that takes the shape: in bfloat16,
    for the head sizes of ``TIED_MFMA_HEAD_DIMS``, MFMA tiles of 128 (position, head) pairs
    (``tied_attention_mfma``); else the 32-bit kernel.  Same arguments, same result up to
    rounding."""
    if tied_attention_mfma_covers(q.dtype, n_heads, n_kv_heads, head_dim):
        tied_attention_mfma(q, gate, k_pool, block_table, q_start, ctx_len, out, scale, window,
                            sink, n_heads, n_kv_heads, head_dim, page_size, max_q_len, max_ctx_len)
    else:
        shared_kv_attention(q, gate, k_pool, block_table, q_start, ctx_len, seq_index, out, scale,
                            window, sink, n_heads, n_kv_heads, head_dim, page_size, max_ctx_len)


@_launches("attention")
def tied_attention_mfma(q, gate, k_pool, block_table, q_start, ctx_len, out, scale, window, sink,
                        n_heads, n_kv_heads, head_dim, page_size, max_q_len, max_ctx_len,
                        n_splits: Optional[int] = None, shared_tiles: Optional[bool] = None) -> None:
    """The bfloat16 MFMA form of ``shared_kv_attention`` (see there for the arguments).  Scores
    and the soft-max are 32-bit; a weight enters the second product as the sum of two bfloat16
    numbers.  A step in which every sequence brings one token runs the decode kernel (head
    sizes up to 128, at most 32 heads a kv head): each context is split over ``n_splits``
    workgroups of four waves that are splits of their own (None: by the block table's width and
    the window, never by the contexts themselves, so that a captured step replays for other
    contexts), and the partial results are merged.  Prompt portions of those shapes run the
    same waves-on-their-own scheme, a wave per 32 (position, head) rows; ``shared_tiles`` True
    (and every other shape) runs the kernel whose workgroup stages the keys once for 128 rows."""
    for t in (q, gate, k_pool, block_table, q_start, ctx_len, out):
        if t is not None and not t.is_cuda:
            raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    T = q.shape[0]
    qs = _columns(q, "tied_attention_mfma: q")
    gs = _columns(gate, "tied_attention_mfma: gate") if gate is not None else 0
    if not tied_attention_mfma_covers(q.dtype, n_heads, n_kv_heads, head_dim):
        raise KernelUnavailable(f"tied_attention_mfma: bfloat16, head_dim of "
                                f"{TIED_MFMA_HEAD_DIMS}, at most {TIED_MFMA_ROWS} heads a kv head")
    if q.shape[1] != n_heads * head_dim or out.shape != (T, n_heads * head_dim) \
            or not out.is_contiguous() or out.dtype != q.dtype or k_pool.dtype != q.dtype \
            or (gate is not None and (gate.shape != q.shape or gate.dtype != q.dtype)) \
            or qs % 8 != 0 or gs % 8 != 0 or q.data_ptr() % 16 != 0 \
            or (gate is not None and gate.data_ptr() % 16 != 0):
        raise KernelUnavailable("tied_attention_mfma: q, gate and out must be [T, nH * hd] of "
                                "the pool's dtype, rows aligned to 16 bytes")
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (ctx_len, "ctx_len")):
        _i32(t, name)
    if n_kv_heads <= 0 or n_heads % n_kv_heads != 0:
        raise KernelUnavailable("tied_attention_mfma: InvalidGrouping")
    n_seqs = ctx_len.shape[0]
    max_pages = block_table.shape[1]
    if max_ctx_len > max_pages * page_size or q_start.shape[0] != n_seqs + 1 \
            or block_table.shape[0] != n_seqs or not block_table.is_contiguous():
        raise KernelUnavailable("tied_attention_mfma: block table or per-sequence arrays do not fit")
    G = n_heads // n_kv_heads
    lib = build.load("sink_attention")
    keys = max_pages * page_size if window <= 0 else min(max_pages * page_size, window)
    if max_q_len == 1 and T == n_seqs and head_dim <= 128 and G <= 32 and not shared_tiles:
        # a decode step: every wave of a workgroup is a split of its own
        # (``tied_attention_decode_kernel``); about 1024 workgroups, at least 64 keys a wave
        span = keys + 31                      # the first chunk starts at a multiple of 32
        blocks = n_splits if n_splits is not None else \
            max(1, min(TIED_DECODE_WORKGROUPS // max(1, n_seqs * n_kv_heads),
                       (span + 255) // 256, 16))
        if not 1 <= blocks <= 16:
            raise KernelUnavailable("tied_attention_mfma: 1 to 16 workgroups a context")
        wave_keys = ((span + 4 * blocks - 1) // (4 * blocks) + 31) // 32 * 32
        ws_o = _workspace("tied_o", T * n_heads * 4 * blocks * head_dim, torch.float32, q.device)
        ws_ml = _workspace("tied_ml", T * n_heads * 4 * blocks * 2, torch.float32, q.device)
        _check(lib.zf_tied_attention_decode(
            _ptr(q), ctypes.c_longlong(qs), _ptr(gate), ctypes.c_longlong(gs), _ptr(k_pool),
            _ptr(block_table), _ptr(ctx_len), _ptr(out), _ptr(ws_o), _ptr(ws_ml),
            ctypes.c_float(scale), int(window), 1 if sink else 0, n_seqs, n_heads, n_kv_heads,
            head_dim, page_size, max_pages, blocks, wave_keys, _stream()),
            "tied_attention_mfma (decode)")
        return
    QT = max(1, TIED_MFMA_ROWS // G)
    n_tiles = (T + QT - 1) // QT + n_seqs
    if shared_tiles is None:
        shared_tiles = not (head_dim <= 128 and G <= 32)
    if not shared_tiles:
        # prompt portions: every wave walks the keys of its own 32 rows
        if head_dim > 128 or G > 32:
            raise KernelUnavailable("tied_attention_mfma: waves on their own take head sizes up "
                                    "to 128 and 32 heads a kv head")
        # few waves behind long contexts: every wave's keys in parts, so that the last rows of
        # a prompt do not run alone at the end and a SIMD holds more than one wave
        parts = n_splits
        if parts is None:
            waves = (T * n_heads + 31) // 32
            parts = 1
            while parts < TIED_ROWS_MAX_PARTS and waves * parts < TIED_ROWS_WAVES \
                    and min(keys, max_ctx_len) >= 256 * parts:
                parts *= 2
        ws_o = ws_ml = None
        if parts > 1:
            ws_o = _workspace("tied_o", T * n_heads * parts * head_dim, torch.float32, q.device)
            ws_ml = _workspace("tied_ml", T * n_heads * parts * 2, torch.float32, q.device)
        _check(lib.zf_tied_attention_rows(
            _ptr(q), ctypes.c_longlong(qs), _ptr(gate), ctypes.c_longlong(gs), _ptr(k_pool),
            _ptr(block_table), _ptr(q_start), _ptr(ctx_len), _ptr(out), _ptr(ws_o), _ptr(ws_ml),
            ctypes.c_float(scale), int(window), 1 if sink else 0, T, n_seqs, n_tiles, n_heads,
            n_kv_heads, head_dim, page_size, max_pages, parts, _stream()),
            "tied_attention_mfma (rows)")
        return
    if n_splits is None:
        n_splits = 1
        if max_q_len == 1 and n_seqs * n_kv_heads < 256:
            n_splits = max(1, min(keys // TIED_SPLIT_KEYS,
                                  TIED_SPLIT_WORKGROUPS // (n_seqs * n_kv_heads), 64))
    split_keys = ((keys + 32 + n_splits - 1) // n_splits + 31) // 32 * 32
    ws_o = ws_ml = None
    if n_splits > 1:
        ws_o = _workspace("tied_o", T * n_heads * n_splits * head_dim, torch.float32, q.device)
        ws_ml = _workspace("tied_ml", T * n_heads * n_splits * 2, torch.float32, q.device)
    _check(lib.zf_tied_attention_mfma(
        _ptr(q), ctypes.c_longlong(qs), _ptr(gate), ctypes.c_longlong(gs), _ptr(k_pool),
        _ptr(block_table), _ptr(q_start), _ptr(ctx_len), _ptr(out), _ptr(ws_o), _ptr(ws_ml),
        ctypes.c_float(scale), int(window), 1 if sink else 0, T, n_seqs, n_tiles, n_heads,
        n_kv_heads, head_dim, page_size, max_pages, n_splits, split_keys, _stream()),
        "tied_attention_mfma")


# ------------------------------------------------------------------------- mixture of experts
MOE_MAX_EXPERTS = 1024


ROUTER_SCORINGS = {"softmax": 0, "sigmoid": 1, "softmax_all": 2}


@_launches("other")
def moe_route(h: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor],
              ids: torch.Tensor, weights: torch.Tensor, scoring: str = "softmax",
              correction: Optional[torch.Tensor] = None,
              groups: Optional[Tuple[int, int]] = None, group_mark: int = 2,
              normalize: bool = True, weight_scale: float = 1.0,
              extra: Optional[torch.Tensor] = None) -> None:
    """Per row of ``h`` [T, W]: z = router h + bias in 32-bit (router float32 [E, W]); ``ids``
    [T, top] int32 receives the ``top`` chosen experts (the lower index wins a tie).
    ``scoring`` "softmax": the largest z are chosen and ``weights`` [T, top] float32 is the
    soft-max over those alone.  "sigmoid": s = sigmoid(z); the choice goes by s + ``correction``
    (float32 [E], or none); with ``groups`` = (count, keep) the experts form ``count`` equal
    groups of neighbours, a group is marked by its two largest choice scores added, and only
    experts of the ``keep`` best groups can be chosen; the weights are the chosen s over their
    sum (+ 1e-20).  "softmax_all": the same with s = softmax(z) over all E outputs.
    ``group_mark`` 1: a group is marked by its largest choice score alone.  ``normalize`` False:
    the weights are the chosen s themselves; either way times ``weight_scale``.  ``extra``
    float32 [T, n]: the router has n more rows behind its E outputs, which are no experts; the
    sigmoids of their products with h go there (a gate a token that rides with the router)."""
    _need_gpu(h, router, bias, ids, weights, correction, extra)
    _i32(ids, "ids")
    T, W = h.shape
    n_extra = 0
    if extra is not None:
        if extra.dim() != 2 or extra.shape[0] != T or extra.dtype != torch.float32 \
                or not extra.is_contiguous() or extra.shape[1] >= router.shape[0]:
            raise KernelUnavailable(f"moe_route: extra {tuple(extra.shape)} {extra.dtype} must be "
                                    "float32 [T, n], n rows of the router behind the experts'")
        n_extra = extra.shape[1]
    E = router.shape[0] - n_extra
    top = ids.shape[1] if ids.dim() == 2 else 0
    count, keep = groups if groups is not None else (0, 0)
    if router.dtype != torch.float32 or router.shape != (E + n_extra, W) \
            or not router.is_contiguous() or ids.shape != (T, top) \
            or weights.shape != (T, top) or weights.dtype != torch.float32 \
            or not 0 < top <= E or E + n_extra > MOE_MAX_EXPERTS \
            or scoring not in ROUTER_SCORINGS or group_mark not in (1, 2) \
            or (scoring == "softmax" and (not normalize or n_extra)) \
            or (bias is not None and (bias.dtype != torch.float32 or bias.shape != (E,))) \
            or (correction is not None and (correction.dtype != torch.float32
                                            or correction.shape != (E,))) \
            or (scoring == "softmax" and (correction is not None or groups is not None)) \
            or (groups is not None and not (0 < keep <= count <= E and E % count == 0
                                            and top <= keep * (E // count))):
        raise KernelUnavailable(f"moe_route: h {tuple(h.shape)}, router {tuple(router.shape)} "
                                f"{router.dtype}, ids {tuple(ids.shape)}, at most "
                                f"{MOE_MAX_EXPERTS} experts, scoring {scoring!r}, groups {groups}")
    lib = build.load("moe")
    _check(lib.zf_moe_route(_ptr(h), _dt(h), _ptr(router), _ptr(bias), _ptr(ids), _ptr(weights),
                            T, W, E, top, ROUTER_SCORINGS[scoring], _ptr(correction), int(count),
                            int(keep), int(group_mark), 1 if normalize else 0,
                            ctypes.c_float(weight_scale), n_extra, _ptr(extra), _stream()),
           "moe_route")


@_launches("products")
def moe_gate_up(h: torch.Tensor, gate_up: torch.Tensor, ids: Optional[torch.Tensor],
                y: torch.Tensor, limit: float, alpha: float, shift: float,
                act: Optional[str] = None, n_identity: int = 0) -> None:
    """y[t, s, :] = act(expert ids[t, s] of ``gate_up`` [E, 2 ff, W] applied to h[t]) with
    g = min(gate, limit), u = clamp(up, -limit, limit) (no clamp if limit <= 0) and
    act = g * sigmoid(alpha g) * (u + shift).  With ``act`` (one of ``ACTIVATIONS``) the experts
    have no gate: ``gate_up`` is [E, ff, W] and y = act(up h).  ``ids`` None: expert 0 for every
    token.  ``n_identity``: ids from E up to E + n_identity - 1 name no expert; their rows of y
    are left alone."""
    _need_gpu(h, gate_up, ids, y)
    T, W = h.shape
    if y.dim() != 3 or gate_up.dim() != 3:
        raise KernelUnavailable("moe_gate_up: y [T, slots, ff], gate_up [E, 2 ff, W]")
    slots, ff = y.shape[1], y.shape[2]
    if ids is not None:
        _i32(ids, "ids")
    rows = ff if act is not None else 2 * ff
    if y.shape[0] != T or gate_up.shape[1:] != (rows, W) or gate_up.dtype != h.dtype \
            or y.dtype != h.dtype or (ids is not None and ids.shape != (T, slots)) \
            or (ids is None and gate_up.shape[0] != 1) or W > 16384 \
            or (act is not None and act not in ACTIVATIONS):
        raise KernelUnavailable(f"moe_gate_up: h {tuple(h.shape)} {h.dtype}, gate_up "
                                f"{tuple(gate_up.shape)} {gate_up.dtype}, y {tuple(y.shape)}, "
                                f"activation {act!r}")
    lib = build.load("moe")
    _check(lib.zf_moe_gate_up(_ptr(h), _ptr(gate_up), _dt(h), _ptr(ids), _ptr(y), T, W, ff,
                              slots, ctypes.c_float(limit), ctypes.c_float(alpha),
                              ctypes.c_float(shift), 0 if act is not None else 1,
                              ACTIVATIONS[act] if act is not None else 0,
                              gate_up.shape[0] if n_identity else (1 << 30), _stream()),
           "moe_gate_up")


@_launches("products")
def moe_down(y: torch.Tensor, down: torch.Tensor, ids: Optional[torch.Tensor],
             weights: Optional[torch.Tensor], out: torch.Tensor, add: bool = False,
             identity: Optional[torch.Tensor] = None) -> None:
    """out[t] (=, or with ``add`` +=) sum over s of weights[t, s] * down[ids[t, s]] y[t, s], in
    slot order and 32-bit; ``down`` [E, W, ff], ``out`` float32 [T, W].  ``ids`` None: expert
    0; ``weights`` None: 1.  ``identity`` [T, W] (the experts' input): an id from E on names no
    expert, and its term is weights[t, s] * identity[t]."""
    _need_gpu(y, down, ids, weights, out, identity)
    if y.dim() != 3 or down.dim() != 3:
        raise KernelUnavailable("moe_down: y [T, slots, ff], down [E, W, ff]")
    T, slots, ff = y.shape
    W = down.shape[1]
    if ids is not None:
        _i32(ids, "ids")
    if down.shape[2] != ff or down.dtype != y.dtype or out.shape != (T, W) \
            or out.dtype != torch.float32 or (ids is not None and ids.shape != (T, slots)) \
            or (ids is None and down.shape[0] != 1) \
            or (weights is not None and (weights.shape != (T, slots)
                                         or weights.dtype != torch.float32)) \
            or (identity is not None and (identity.shape != (T, W) or identity.dtype != y.dtype
                                          or not identity.is_contiguous())):
        raise KernelUnavailable(f"moe_down: y {tuple(y.shape)} {y.dtype}, down "
                                f"{tuple(down.shape)} {down.dtype}, out {tuple(out.shape)}")
    lib = build.load("moe")
    _check(lib.zf_moe_down(_ptr(y), _ptr(down), _dt(y), _ptr(ids), _ptr(weights), _ptr(out), T,
                           W, ff, slots, 1 if add else 0,
                           down.shape[0] if identity is not None else (1 << 30), _ptr(identity),
                           _stream()), "moe_down")


@_launches("norm_rope_write")
def gated_act(gate_up: torch.Tensor, out: torch.Tensor, limit: float, alpha: float,
              shift: float, row_factor: Optional[torch.Tensor] = None) -> None:
    """out[t, j] = g * sigmoid(alpha g) * (u + shift) with g = min(gate_up[t, j], limit) and
    u = clamp(gate_up[t, ff + j], -limit, limit) (no clamp if limit <= 0); times
    ``row_factor[t]`` (float32 [T] or a column of a float32 matrix) if given."""
    _need_gpu(gate_up, out)
    T, ff = out.shape
    if gate_up.shape != (T, 2 * ff) or gate_up.dtype != out.dtype \
            or (row_factor is not None and (not row_factor.is_cuda
                                            or row_factor.dtype != torch.float32
                                            or row_factor.dim() != 1 or row_factor.shape[0] != T)):
        raise KernelUnavailable(f"gated_act: gate_up {tuple(gate_up.shape)}, out {tuple(out.shape)}")
    lib = build.load("moe")
    _check(lib.zf_gated_act(_ptr(gate_up), _ptr(out), _dt(out), T, ff, ctypes.c_float(limit),
                            ctypes.c_float(alpha), ctypes.c_float(shift), _ptr(row_factor),
                            int(row_factor.stride(0)) if row_factor is not None else 0,
                            _stream()), "gated_act")


MOE_TILE_ROWS = 128           # MOE_TILE_ROWS in moe.hip
MOE_STREAM_MAX_TOKENS = 16    # up to here every (token, expert) streams its own matrices


def moe_grouped_covers(h: torch.Tensor, gate_up: torch.Tensor, act: Optional[str] = None) -> bool:
    """Whether the MFMA kernels over tokens sorted by expert take these operands: bfloat16,
    both reduction lengths multiples of 8."""
    ff = gate_up.shape[1] if act is not None else gate_up.shape[1] // 2
    return h.dtype == torch.bfloat16 and gate_up.dtype == torch.bfloat16 \
        and gate_up.shape[2] % 8 == 0 and ff % 8 == 0


def moe_experts(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, ids: torch.Tensor,
                weights: torch.Tensor, y: torch.Tensor, out: torch.Tensor, limit: float,
                alpha: float, shift: float, add: bool = False,
                act: Optional[str] = None, n_identity: int = 0) -> None:
    """out[t] (=, +=) sum over s of weights[t, s] * expert ids[t, s] applied to h[t]
    (``moe_gate_up`` then ``moe_down``), with ``y`` [T, top, ff] as work space.  A few tokens
    stream each chosen expert's matrices (one workgroup row per token and slot); more tokens,
    in bfloat16, are sorted by expert and run through MFMA tiles of ``MOE_TILE_ROWS`` pairs
    (``moe_sort``, ``moe_grouped`` twice, ``moe_combine``).  Either way a token's result
    depends on that token alone.  ``act``: experts without a gate (see ``moe_gate_up``).
    ``n_identity``: ids from E up to E + n_identity - 1 name no expert; such a term of the sum is
    the weight times h[t] itself."""
    T, W = h.shape
    if T > MOE_STREAM_MAX_TOKENS and moe_grouped_covers(h, gate_up, act):
        moe_grouped(h, gate_up, down, ids, weights, y, out, limit, alpha, shift, add, act,
                    n_identity)
        return
    moe_gate_up(h, gate_up, ids, y, limit, alpha, shift, act, n_identity)
    moe_down(y, down, ids, weights, out, add=add, identity=h if n_identity else None)


@_launches("products")
def moe_grouped(h, gate_up, down, ids, weights, y, out, limit, alpha, shift, add=False,
                act: Optional[str] = None, n_identity: int = 0) -> None:
    """The many-token form of ``moe_experts`` (bfloat16; see there)."""
    _need_gpu(h, gate_up, down, ids, weights, y, out)
    _i32(ids, "ids")
    T, W = h.shape
    E, rows, _ = gate_up.shape
    ff = rows if act is not None else rows // 2
    top = ids.shape[1]
    if not moe_grouped_covers(h, gate_up, act) or down.dtype != torch.bfloat16 \
            or gate_up.shape != (E, ff if act is not None else 2 * ff, W) \
            or down.shape != (E, W, ff) \
            or ids.shape != (T, top) or weights.shape != (T, top) \
            or weights.dtype != torch.float32 or y.dtype != torch.bfloat16 \
            or y.numel() != T * top * ff or not y.is_contiguous() \
            or out.shape != (T, W) or out.dtype != torch.float32 \
            or not 0 < E <= E + n_identity <= MOE_MAX_EXPERTS or not h.is_contiguous() \
            or (act is not None and act not in ACTIVATIONS):
        raise KernelUnavailable(f"moe_grouped: h {tuple(h.shape)} {h.dtype}, gate_up "
                                f"{tuple(gate_up.shape)}, down {tuple(down.shape)}, ids "
                                f"{tuple(ids.shape)}, y {tuple(y.shape)} {y.dtype}")
    P = T * top
    EA = E + n_identity           # the sort's buckets: the ids that name no expert have theirs
    max_tiles = (P + MOE_TILE_ROWS - 1) // MOE_TILE_ROWS + EA
    # places of the pairs, the tiles' list and the experts' 32-bit outputs, kept across steps
    table = _workspace("moe_table", 2 * P + 3 * max_tiles + 4, torch.int32, h.device)
    o = _workspace("moe_out", P * W, torch.float32, h.device)
    sorted_, place = table[:P], table[P:2 * P]
    t0 = 2 * P
    tile_expert, tile_row0 = table[t0:t0 + max_tiles], table[t0 + max_tiles:t0 + 2 * max_tiles]
    tile_rows = table[t0 + 2 * max_tiles:t0 + 3 * max_tiles]
    n_tiles = table[t0 + 3 * max_tiles:]
    lib = build.load("moe")
    st = _stream()
    _check(lib.zf_moe_sort(_ptr(ids), P, EA, _ptr(sorted_), _ptr(place), _ptr(tile_expert),
                           _ptr(tile_row0), _ptr(tile_rows), _ptr(n_tiles), st), "moe_sort")
    lim, al, sh = ctypes.c_float(limit), ctypes.c_float(alpha), ctypes.c_float(shift)
    kind = ACTIVATIONS[act] if act is not None else 0
    _check(lib.zf_moe_grouped(_ptr(h), ctypes.c_longlong(W), _ptr(sorted_), top, _ptr(gate_up),
                              _ptr(tile_expert), _ptr(tile_row0), _ptr(tile_rows), _ptr(n_tiles),
                              _ptr(y), max_tiles, ff, W, 2 if act is not None else 1, lim, al, sh,
                              kind, E, st), "moe_grouped (gate, up)")
    _check(lib.zf_moe_grouped(_ptr(y), ctypes.c_longlong(ff), _ptr(sorted_), top, _ptr(down),
                              _ptr(tile_expert), _ptr(tile_row0), _ptr(tile_rows), _ptr(n_tiles),
                              _ptr(o), max_tiles, W, ff, 0, lim, al, sh, 0, E, st),
           "moe_grouped (down)")
    _check(lib.zf_moe_combine(_ptr(o), _ptr(place), _ptr(weights), _ptr(out), T, W, top,
                              1 if add else 0, _ptr(ids) if n_identity else None, E,
                              _ptr(h) if n_identity else None, st), "moe_combine")


# ------------------------------------------------------------------------- sampling
SAMPLE_MAX_TOP_K = 1024
SAMPLE_ROW_DTYPE = [("temperature", "<f4"), ("top_p", "<f4"), ("min_p", "<f4"), ("top_k", "<i4"),
                    ("u", "<f8")]


@_launches("head_sampling")
def apply_penalties(logits, rows, tokens, counts, params) -> None:
    """In place, for every triple (rows[i], tokens[i], counts[i]): the repetition, presence
    and frequency penalties of ``params[row] = (repetition, presence, frequency)``."""
    _need_gpu(logits, rows, tokens, counts, params)
    for t, name in ((rows, "rows"), (tokens, "tokens"), (counts, "counts")):
        _i32(t, name)
    n, V = rows.shape[0], logits.shape[1]
    if logits.dtype != torch.float32 or params.dtype != torch.float32 \
            or params.shape != (logits.shape[0], 3) or tokens.shape[0] != n or counts.shape[0] != n:
        raise KernelUnavailable("apply_penalties: float32 logits [n, V], params [n, 3], int32 triples")
    lib = build.load("sampling")
    _check(lib.zf_apply_penalties(_ptr(logits), _ptr(rows), _ptr(tokens), _ptr(counts),
                                  _ptr(params), n, V, _stream()), "apply_penalties")


@_launches("head_sampling")
def sample_topk(logits: torch.Tensor, params: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = a token of row r drawn as the reference's sampler draws it: the top_k
    (1..1024) largest logits, temperature, min-p, top-p, and the uniform number u of the
    row.  ``params`` is a uint8 tensor holding one SAMPLE_ROW_DTYPE record per row."""
    _need_gpu(logits, params, out)
    _i32(out, "out")
    n, V = logits.shape
    if logits.dtype != torch.float32 or params.dtype != torch.uint8 \
            or params.numel() != n * 24 or out.shape != (n,):
        raise KernelUnavailable("sample_topk: float32 logits [n, V], 24-byte records, int32 out [n]")
    lib = build.load("sampling")
    _check(lib.zf_sample_topk(_ptr(logits), _ptr(params), _ptr(out), n, V, _stream()),
           "sample_topk")


# ------------------------------------------------------------------------- an activation alone
ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2, "relu2": 3, "tanh": 4}


@_launches("norm_rope_write")
def activation(x: torch.Tensor, out: torch.Tensor, kind: str) -> None:
    """out = act(x) element by element, in 32-bit on values of either storage type: "gelu"
    (the exact form with erf), "gelu_tanh", "silu", "relu2" (max(x, 0)^2), "tanh".  ``out``
    may be ``x``."""
    _need_gpu(x, out)
    if x.shape != out.shape or x.dtype != out.dtype or kind not in ACTIVATIONS:
        raise KernelUnavailable(f"activation: {tuple(x.shape)} {x.dtype} -> {tuple(out.shape)} "
                                f"{out.dtype}, kind {kind!r} of {sorted(ACTIVATIONS)}")
    lib = build.load("elementwise")
    _check(lib.zf_activation(_ptr(x), _ptr(out), _dt(x), ctypes.c_longlong(x.numel()),
                             ACTIVATIONS[kind], _stream()), "activation")


@_launches("norm_rope_write")
def norm_add_store(y: torch.Tensor, gain: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
                   centred: bool, x: torch.Tensor, out: torch.Tensor) -> None:
    """x += norm(y); out = x rounded to ``out``'s type, row by row in 32-bit (``norm_rows`` with
    ``add`` and a cast, in one kernel, the same numbers).  ``y`` and ``x`` float32 [T, W], W a
    multiple of 4 up to 8192."""
    _need_gpu(y, gain, bias, x, out)
    T, W = x.shape
    if y.shape != x.shape or out.shape != x.shape or y.dtype != torch.float32 \
            or x.dtype != torch.float32 or gain.dtype != torch.float32 or gain.shape != (W,) \
            or (bias is not None and (bias.dtype != torch.float32 or bias.shape != (W,))) \
            or not norm_add_norm_covers(W):
        raise KernelUnavailable(f"norm_add_store: float32 rows {tuple(y.shape)} and "
                                f"{tuple(x.shape)}, float32 [W] gain and bias, W a multiple of 4 "
                                f"up to {NORM_ADD_NORM_MAX_WIDTH}")
    lib = build.load("norms")
    _check(lib.zf_norm_add_store(_ptr(y), _ptr(gain), _ptr(bias), ctypes.c_float(eps),
                                 1 if centred else 0, _ptr(x), _ptr(out), _dt(out), T, W,
                                 _stream()), "norm_add_store")


# ------------------------------------------------------------------------- attention with a cap, a sink, chunks or a window, a gate
class RowSegment:
    """Columns [src_off, src_off + width) of a projection's rows and what happens to them on the
    way out (``project_rows``): ``gain`` [width] float32: an RMS norm over the whole segment with
    ``eps``; the segment is ``width / hd`` heads, of each the elements [rot_off, rot_off +
    rot_dims) are rotated by the token's position in the pairs (i, i + rot_dims / 2) with the
    angles position * ``freq`` [rot_dims / 2] (float32), cosine and sine times ``mag``; the
    elements of a head below ``skip`` are not written.  The rest goes to ``dst``: plain rows
    [T, ...] where head h starts at column dst_off + h * dst_hd (dst_hd None: hd - skip), or
    (``pool_heads`` given) a pool of blocks [page, kv head] of rows of dst_hd elements (laid out as
    ``masked_pool_from_rows`` says) at the token's slot, from column dst_off of the row on.
    ``bias`` [width] float32 is added to the source's values before anything else.  ``per_head``:
    the norm runs over every head on its own and ``gain`` is [hd], one for all heads.
    ``interleaved``: the rotated pairs are the neighbours (2i, 2i + 1), pair i by freq[i]."""

    def __init__(self, src_off: int, width: int, dst: torch.Tensor, *, gain=None, eps: float = 0.0,
                 hd: Optional[int] = None, rot_off: int = 0, rot_dims: int = 0, freq=None,
                 mag: float = 1.0, skip: int = 0, dst_off: int = 0, dst_hd: Optional[int] = None,
                 pool_heads: Optional[int] = None, bias=None, per_head: bool = False,
                 interleaved: bool = False):
        self.src_off, self.width, self.dst = int(src_off), int(width), dst
        self.gain, self.eps = gain, float(eps)
        self.hd = int(hd) if hd is not None else int(width)
        self.rot_off, self.rot_dims, self.freq, self.mag = int(rot_off), int(rot_dims), freq, float(mag)
        self.skip, self.dst_off = int(skip), int(dst_off)
        self.dst_hd = int(dst_hd) if dst_hd is not None else self.hd - self.skip
        self.pool_heads = pool_heads
        self.bias, self.per_head, self.interleaved = bias, bool(per_head), bool(interleaved)


PROJECT_ROWS_MAX_SEGMENTS = 4


@_launches("norm_rope_write")
def project_rows(src: torch.Tensor, positions: torch.Tensor, slot_mapping: Optional[torch.Tensor],
                 page_size: int, segments) -> None:
    """Every row of ``src`` [T, C] (contiguous rows, any row stride), segment by segment as
    ``RowSegment`` says: norm, rotation by ``positions`` [T], then into rows or pages.  All
    arithmetic is 32-bit; a row's result depends on that row and its position alone."""
    for t in (src, positions, slot_mapping):
        if t is not None and not t.is_cuda:
            raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    _i32(positions, "positions")
    T, C = src.shape
    stride = _columns(src, "project_rows: src")
    n = len(segments)
    if not 0 < n <= PROJECT_ROWS_MAX_SEGMENTS or positions.shape[0] != T:
        raise KernelUnavailable(f"project_rows: 1 to {PROJECT_ROWS_MAX_SEGMENTS} segments and a "
                                "position a row")
    ints, floats, ptrs, strides = [], [], [], []
    for g in segments:
        pool = g.pool_heads is not None
        ok = 0 <= g.src_off and g.src_off + g.width <= C and g.width > 0 and g.hd > 0 \
            and g.width % g.hd == 0 and g.rot_dims % 2 == 0 and 0 <= g.rot_off \
            and g.rot_off + g.rot_dims <= g.hd and 0 <= g.skip < g.hd \
            and g.dst.is_cuda and g.dst.dtype == src.dtype and g.dst_off >= 0 \
            and (g.gain is None or (g.gain.is_cuda and g.gain.dtype == torch.float32
                                    and g.gain.shape == ((g.hd if g.per_head else g.width),)
                                    and g.gain.is_contiguous())) \
            and (g.bias is None or (g.bias.is_cuda and g.bias.dtype == torch.float32
                                    and g.bias.shape == (g.width,) and g.bias.is_contiguous())) \
            and (g.rot_dims == 0 or (g.freq is not None and g.freq.is_cuda
                                     and g.freq.dtype == torch.float32
                                     and g.freq.shape == (g.rot_dims // 2,)))
        heads = g.width // max(g.hd, 1)
        if ok and pool:
            _i32(slot_mapping, "slot_mapping")
            ok = slot_mapping.shape[0] == T and g.dst.is_contiguous() and heads == g.pool_heads \
                and g.dst_off + g.hd - g.skip <= g.dst_hd \
                and g.dst.numel() % (g.pool_heads * page_size * g.dst_hd) == 0
            strides.append(0)
        elif ok:
            ok = g.dst.dim() == 2 and g.dst.stride(1) == 1 and g.dst.shape[0] == T \
                and g.dst_off + (heads - 1) * g.dst_hd + g.hd - g.skip <= g.dst.shape[1]
            strides.append(g.dst.stride(0) if ok else 0)
        if not ok:
            raise KernelUnavailable(f"project_rows: a segment of columns {g.src_off}.."
                                    f"{g.src_off + g.width} (heads of {g.hd}) does not fit its "
                                    f"source {tuple(src.shape)} or destination "
                                    f"{tuple(g.dst.shape)} {g.dst.dtype}")
        ints += [g.src_off, g.width, g.hd, g.rot_off, g.rot_dims, g.skip, 1 if pool else 0,
                 g.dst_off, g.dst_hd, g.pool_heads or 0,
                 (1 if g.per_head else 0) | (2 if g.interleaved else 0)]
        floats += [g.eps, g.mag]
        ptrs += [g.gain.data_ptr() if g.gain is not None else None,
                 g.freq.data_ptr() if g.rot_dims else None, g.dst.data_ptr(),
                 g.bias.data_ptr() if g.bias is not None else None]
    lib = build.load("masked_attention")
    _check(lib.zf_project_rows(
        _ptr(src), _dt(src), ctypes.c_longlong(stride), _ptr(positions), _ptr(slot_mapping), T,
        int(page_size), n, (ctypes.c_int * len(ints))(*ints),
        (ctypes.c_float * len(floats))(*floats), (ctypes.c_void_p * len(ptrs))(*ptrs),
        (ctypes.c_longlong * len(strides))(*strides), _stream()), "project_rows")


def masked_pool_from_rows(rows: torch.Tensor) -> torch.Tensor:
    """A pool [pages, heads * page_size * W] in the layout ``project_rows`` writes and the
    ``masked_attention`` kernels read, from rows [pages, heads, page_size, W]: with W a multiple
    of 8 a block [page, head] is laid out [W / 8][page_size][8] (the 16 bytes of 8 elements of
    a row beside the same 16 bytes of the next row: what 16 lanes of a wave load for an MFMA
    operand is 256 consecutive bytes), else in plain rows."""
    P, H, ps, W = rows.shape
    if W % 8 == 0:
        rows = rows.view(P, H, ps, W // 8, 8).permute(0, 1, 3, 2, 4)
    return rows.contiguous().view(P, H * ps * W)


def masked_pool_rows(pool: torch.Tensor, n_heads: int, page_size: int, width: int) -> torch.Tensor:
    """The rows [pages, heads, page_size, W] a pool of that layout holds (a copy)."""
    P = pool.shape[0]
    if width % 8 == 0:
        return pool.view(P, n_heads, width // 8, page_size, 8).permute(0, 1, 3, 2, 4) \
            .reshape(P, n_heads, page_size, width)
    return pool.view(P, n_heads, page_size, width).clone()


GATE_MODES = {None: 0, "element": 1, "head": 2}


def _masked_attention_checks(what, q, gate, gate_mode, k_pool, v_pool, sink, block_table, q_start,
                             ctx_len, seq_index, out, n_heads, n_kv_heads, key_width,
                             value_width, page_size, max_ctx_len):
    for t in (q, gate, k_pool, v_pool, sink, block_table, q_start, ctx_len, seq_index, out):
        if t is not None and not t.is_cuda:
            raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    T = q.shape[0]
    if gate_mode not in GATE_MODES or (gate_mode is None) != (gate is None):
        raise KernelUnavailable(f"{what}: gate mode {gate_mode!r} of {list(GATE_MODES)}, with a "
                                "gate exactly when there is a mode")
    gate_cols = {None: 0, "element": n_heads * value_width, "head": n_heads}[gate_mode]
    if q.shape[1] != n_heads * key_width or out.shape != (T, n_heads * value_width) \
            or not out.is_contiguous() or out.dtype != q.dtype or k_pool.dtype != q.dtype \
            or (v_pool is not None and v_pool.dtype != q.dtype) \
            or (gate is not None and (gate.shape != (T, gate_cols) or gate.dtype != q.dtype)) \
            or (sink is not None and (sink.dtype != torch.float32 or sink.shape != (n_heads,))):
        raise KernelUnavailable(f"{what}: q [T, nH * key width], out [T, nH * value width], the "
                                "gate [T, nH * value width] or [T, nH], all of the pools' dtype; "
                                "the sink float32 [nH]")
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (ctx_len, "ctx_len"),
                    (seq_index, "seq_index")):
        if t is not None:
            _i32(t, name)
    if n_kv_heads <= 0 or n_heads % n_kv_heads != 0:
        raise KernelUnavailable(f"{what}: InvalidGrouping")
    if key_width < 1 or not 0 < value_width <= MAX_HEAD_DIM \
            or (v_pool is None and value_width > key_width):
        raise KernelUnavailable(f"{what}: key rows of {key_width}, value rows of {value_width} "
                                f"(1..{MAX_HEAD_DIM}; without a value pool at most the key's)")
    if max_ctx_len > block_table.shape[1] * page_size:
        raise KernelUnavailable(f"{what}: block table shorter than the context")
    n_seqs = ctx_len.shape[0]
    if q_start.shape[0] != n_seqs + 1 or block_table.shape[0] != n_seqs \
            or (seq_index is not None and seq_index.shape[0] != T) \
            or not block_table.is_contiguous() \
            or not k_pool.is_contiguous() or (v_pool is not None and not v_pool.is_contiguous()):
        raise KernelUnavailable(f"{what}: per-sequence arrays disagree in length")


@_launches("attention")
def masked_attention(q: torch.Tensor, gate: Optional[torch.Tensor], gate_mode: Optional[str],
                     k_pool: torch.Tensor, v_pool: Optional[torch.Tensor],
                     sink: Optional[torch.Tensor], block_table, q_start, ctx_len, seq_index,
                     out: torch.Tensor, scale: float, cap: float, window: int, chunk: int,
                     n_heads: int, n_kv_heads: int, key_width: int, value_width: int,
                     page_size: int, max_ctx_len: int) -> None:
    """Causal grouped-query attention over paged pools of blocks [page, kv head] of rows (laid
    out as ``masked_pool_from_rows`` says): keys of ``key_width``, values of ``value_width``
    elements, or with ``v_pool`` None the first ``value_width`` columns of the key rows.  Token t of sequence s = seq_index[t] has position p = ctx_len[s] -
    q_len[s] + (t - q_start[s]) and reads the keys j <= p with p - j < window (window > 0) and
    floor(j / chunk) == floor(p / chunk) (chunk > 0).  Scores are scale * q . k, then with
    cap > 0 cap * tanh(score / cap).  ``sink`` [nH] float32: the soft-max's denominator holds
    exp(sink_h) once more.  ``gate`` with mode "element" [T, nH * value width] or "head" [T, nH]:
    the output is multiplied by sigmoid(gate).  ``q`` and ``gate`` may be column slices of a
    wider product.  All arithmetic is 32-bit in both dtypes."""
    _masked_attention_checks("masked_attention", q, gate, gate_mode, k_pool, v_pool, sink,
                             block_table, q_start, ctx_len, seq_index, out, n_heads, n_kv_heads,
                             key_width, value_width, page_size, max_ctx_len)
    qs = _columns(q, "masked_attention: q")
    gs = _columns(gate, "masked_attention: gate") if gate is not None else 0
    lib = build.load("masked_attention")
    code = lib.zf_masked_attention(
        _ptr(q), ctypes.c_longlong(qs), _ptr(gate), ctypes.c_longlong(gs), GATE_MODES[gate_mode],
        _ptr(k_pool), _ptr(v_pool), _dt(q), _ptr(sink), _ptr(block_table), _ptr(q_start),
        _ptr(ctx_len), _ptr(seq_index), _ptr(out), ctypes.c_float(scale), ctypes.c_float(cap),
        int(window), int(chunk), q.shape[0], n_heads, n_kv_heads, key_width, value_width,
        page_size, block_table.shape[1], _stream())
    if code == -3:
        raise KernelUnavailable(f"masked_attention: key rows of {key_width} are wider than the "
                                "kernel's staging area takes")
    _check(code, "masked_attention")


@_launches("products")
def head_products(a: torch.Tensor, a_off: int, a_hd: int, w: torch.Tensor,
                  gate: Optional[torch.Tensor], out: torch.Tensor, out_off: int,
                  out_hd: int) -> None:
    """A matrix a head: out[t, out_off + h * out_hd + n] = sum_k a[t, a_off + h * a_hd + k] *
    w[h, n, k] for w [H, N, K], times sigmoid(gate[t, h * N + n]) if a gate is given.  ``a``,
    ``out`` and ``gate`` are matrices with contiguous rows (any row stride).  32-bit sums in
    ascending k whatever the dtypes: a row's result does not depend on the rows beside it."""
    for t in (a, w, gate, out):
        if t is not None and not t.is_cuda:
            raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    T = a.shape[0]
    if w.dim() != 3 or not w.is_contiguous():
        raise KernelUnavailable("head_products: w must be [H, N, K], contiguous")
    H, N, K = w.shape
    a_stride = _columns(a, "head_products: a")
    o_stride = _columns(out, "head_products: out")
    g_stride = _columns(gate, "head_products: gate") if gate is not None else 0
    if out.shape[0] != T or out.dtype != a.dtype or a_hd < K or out_hd < N or a_off < 0 \
            or out_off < 0 or a_off + (H - 1) * a_hd + K > a.shape[1] \
            or out_off + (H - 1) * out_hd + N > out.shape[1] \
            or (gate is not None and (gate.shape != (T, H * N) or gate.dtype != a.dtype)):
        raise KernelUnavailable(f"head_products: a {tuple(a.shape)}, w {tuple(w.shape)}, out "
                                f"{tuple(out.shape)} do not fit together")
    lib = build.load("masked_attention")
    _check(lib.zf_head_products(
        _ptr(a), _dt(a), ctypes.c_longlong(a_stride), int(a_off), int(a_hd), _ptr(w), _dt(w),
        _ptr(gate), ctypes.c_longlong(g_stride), _ptr(out), ctypes.c_longlong(o_stride),
        int(out_off), int(out_hd), T, H, N, K, _stream()), "head_products")


# (key width, value width) the MFMA kernels are built for: values of their own, and the keys'
# leading columns as values
MASKED_MFMA_SHAPES = {False: ((64, 64), (96, 96), (128, 128)),
                      True: ((64, 64), (96, 96), (128, 128), (96, 64), (160, 128), (192, 128))}
MASKED_MFMA_ROWS = 128           # (position, head) pairs a workgroup takes
MASKED_ROWS_WAVES = 2048         # a prompt portion's keys are cut in parts until this many waves run
MASKED_ROWS_MAX_PARTS = 4
MASKED_DECODE_WORKGROUPS = 1024  # a decode step's contexts are split until about this many run


def masked_attention_mfma_covers(dtype, n_heads: int, n_kv_heads: int, key_width: int,
                                 value_width: int, tied: bool) -> bool:
    """Whether the bfloat16 MFMA kernels take the shape; otherwise (and in 32-bit) the kernel
    for every size runs."""
    return dtype == torch.bfloat16 and (key_width, value_width) in MASKED_MFMA_SHAPES[bool(tied)] \
        and n_heads // n_kv_heads <= 32


def attend_masked(q, gate, gate_mode, k_pool, v_pool, sink, block_table, q_start, ctx_len,
                  seq_index, out, scale, cap, window, chunk, n_heads, n_kv_heads, key_width,
                  value_width, page_size, max_q_len, max_ctx_len) -> None:
    """``masked_attention`` through the fastest kernel that takes the shape: in bfloat16, for
    the widths of ``MASKED_MFMA_SHAPES``, the MFMA kernels (``masked_attention_mfma``); else
    the 32-bit kernel.  Same arguments, same result up to rounding."""
    if masked_attention_mfma_covers(q.dtype, n_heads, n_kv_heads, key_width, value_width,
                                    v_pool is None) \
            and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0:
        masked_attention_mfma(q, gate, gate_mode, k_pool, v_pool, sink, block_table, q_start,
                              ctx_len, out, scale, cap, window, chunk, n_heads, n_kv_heads,
                              key_width, value_width, page_size, max_q_len, max_ctx_len)
    else:
        masked_attention(q, gate, gate_mode, k_pool, v_pool, sink, block_table, q_start, ctx_len,
                         seq_index, out, scale, cap, window, chunk, n_heads, n_kv_heads,
                         key_width, value_width, page_size, max_ctx_len)


@_launches("attention")
def masked_attention_mfma(q, gate, gate_mode, k_pool, v_pool, sink, block_table, q_start, ctx_len,
                          out, scale, cap, window, chunk, n_heads, n_kv_heads, key_width,
                          value_width, page_size, max_q_len, max_ctx_len,
                          n_splits: Optional[int] = None) -> None:
    """The bfloat16 MFMA form of ``masked_attention`` (see there for the arguments).  Scores, cap
    and soft-max are 32-bit; a weight enters the second product as the sum of two bfloat16
    numbers.  Every wave takes 32 (position, head) rows and walks their keys on its own.  A step
    in which every sequence brings one token runs the decode form: each context is split over
    ``n_splits`` workgroups of four waves that are splits of their own (None: by the block
    table's width and the window or chunk, never by the contexts themselves, so that a captured
    step replays for other contexts) and the partial results are merged; a prompt portion's
    waves take their keys in ``n_splits`` parts where few waves stand behind long contexts."""
    _masked_attention_checks("masked_attention_mfma", q, gate, gate_mode, k_pool, v_pool, sink,
                             block_table, q_start, ctx_len, None, out, n_heads, n_kv_heads,
                             key_width, value_width, page_size, max_ctx_len)
    T = q.shape[0]
    qs = _columns(q, "masked_attention_mfma: q")
    gs = _columns(gate, "masked_attention_mfma: gate") if gate is not None else 0
    if not masked_attention_mfma_covers(q.dtype, n_heads, n_kv_heads, key_width, value_width,
                                        v_pool is None) or qs % 8 != 0 or q.data_ptr() % 16 != 0:
        raise KernelUnavailable(f"masked_attention_mfma: bfloat16, (key, value) widths of "
                                f"{MASKED_MFMA_SHAPES}, at most 32 heads a kv head, query rows "
                                "aligned to 16 bytes")
    n_seqs = ctx_len.shape[0]
    max_pages = block_table.shape[1]
    keys = max_pages * page_size
    for bound in (window, chunk):
        if bound > 0:
            keys = min(keys, bound)
    G = n_heads // n_kv_heads
    lib = build.load("masked_attention")
    decode = max_q_len == 1 and T == n_seqs
    if decode:
        span = keys + 31                      # the first chunk starts at a multiple of 32
        blocks = n_splits if n_splits is not None else \
            max(1, min(MASKED_DECODE_WORKGROUPS // max(1, n_seqs * n_kv_heads),
                       (span + 383) // 384, 16))
        if not 1 <= blocks <= 16:
            raise KernelUnavailable("masked_attention_mfma: 1 to 16 workgroups a context")
        wave_keys = ((span + 4 * blocks - 1) // (4 * blocks) + 31) // 32 * 32
        parts, splits, n_tiles = blocks, 4 * blocks, n_seqs
    else:
        QT = max(1, MASKED_MFMA_ROWS // G)
        n_tiles = (T + QT - 1) // QT + n_seqs
        parts = n_splits
        if parts is None:
            waves = (T * n_heads + 31) // 32
            parts = 1
            while parts < MASKED_ROWS_MAX_PARTS and waves * parts < MASKED_ROWS_WAVES \
                    and min(keys, max_ctx_len) >= 256 * parts:
                parts *= 2
        wave_keys, splits = 0, parts
    ws_o = ws_ml = None
    if decode or parts > 1:
        ws_o = _workspace("masked_o", T * n_heads * splits * value_width, torch.float32, q.device)
        ws_ml = _workspace("masked_ml", T * n_heads * splits * 2, torch.float32, q.device)
    code = lib.zf_masked_attention_mfma(
        _ptr(q), ctypes.c_longlong(qs), _ptr(gate), ctypes.c_longlong(gs), GATE_MODES[gate_mode],
        _ptr(k_pool), _ptr(v_pool), _ptr(sink), _ptr(block_table), _ptr(q_start), _ptr(ctx_len),
        _ptr(out), _ptr(ws_o), _ptr(ws_ml), ctypes.c_float(scale), ctypes.c_float(cap),
        int(window), int(chunk), T, n_seqs, n_tiles, n_heads, n_kv_heads, key_width, value_width,
        page_size, max_pages, 1 if decode else 0, parts, wave_keys, _stream())
    _check(code, "masked_attention_mfma")


# ------------------------------------------------------------------------- mixers with a state of fixed size
RECURRENCE_CHANNELS = 8          # REC_R in recurrent.hip: key channels a thread holds
RECURRENCE_MAX_KEY_DIM = 256
RECURRENCE_MAX_THREADS = 256
RECURRENCE_MAX_LDS = 65536
RECURRENCE_WORKGROUPS = 512      # value columns are dealt over workgroups until about this many run
RECURRENCE_SPAN = 64             # tokens of a span; a multiple of the 16 tokens the kernel stages
RECURRENCE_MAX_SPANS = 64        # longer portions have longer spans instead of more
DECAY_RULES = {"sigmoid_root": 0, "double_exp": 1}


def recurrence_state_size(n_heads: int, key_dim: int, value_dim: int) -> int:
    """32-bit numbers a request's state takes in ``decay_recurrence``: [head][value column]
    [channels padded to a multiple of ``RECURRENCE_CHANNELS``]."""
    padded = (key_dim + RECURRENCE_CHANNELS - 1) // RECURRENCE_CHANNELS * RECURRENCE_CHANNELS
    return n_heads * value_dim * padded


def recurrence_state_matrix(state: torch.Tensor, n_heads: int, key_dim: int,
                            value_dim: int) -> torch.Tensor:
    """The matrices S [.., head, key channel, value column] of states laid out as the kernel
    keeps them (tests and inspection)."""
    padded = recurrence_state_size(n_heads, key_dim, value_dim) // (n_heads * value_dim)
    s = state[..., :n_heads * value_dim * padded]
    s = s.reshape(s.shape[:-1] + (n_heads, value_dim, padded))
    return s[..., :key_dim].transpose(-1, -2)


@_launches("norm_rope_write")
def token_shift_mix(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, state_offset: int,
                    state_slots: torch.Tensor, seq_index: torch.Tensor, q_start: torch.Tensor,
                    out: torch.Tensor) -> None:
    """out[m, t] = h[t] + (h[t - 1] - h[t]) * mu[m] for the rows ``h`` [T, W] of a step
    (``mu`` float32 [n, W], ``out`` [n, T, W] in the rows' type).  The row before a sequence's
    first row of this step is the request's state: elements [state_offset, state_offset + W)
    of row state_slots[s] of ``state`` (float32 [slots, size]), which afterwards hold the
    sequence's last row of this step."""
    _need_gpu(h, mu, state, state_slots, seq_index, q_start, out)
    for t, name in ((state_slots, "state_slots"), (seq_index, "seq_index"), (q_start, "q_start")):
        _i32(t, name)
    T, W = h.shape
    n = mu.shape[0]
    if mu.dtype != torch.float32 or mu.shape != (n, W) or out.shape != (n, T, W) \
            or out.dtype != h.dtype or state.dtype != torch.float32 or state.dim() != 2 \
            or not 0 <= state_offset <= state.shape[1] - W or seq_index.shape[0] != T \
            or q_start.shape[0] != state_slots.shape[0] + 1:
        raise KernelUnavailable(f"token_shift_mix: h {tuple(h.shape)}, mu {tuple(mu.shape)} "
                                f"{mu.dtype}, out {tuple(out.shape)}, state {tuple(state.shape)} "
                                f"{state.dtype} from {state_offset}")
    lib = build.load("recurrent")
    base = _vp(state.data_ptr() + 4 * int(state_offset))
    _check(lib.zf_token_shift_mix(_ptr(h), _dt(h), _ptr(mu), base,
                                  ctypes.c_longlong(state.shape[1]), _ptr(state_slots),
                                  _ptr(seq_index), _ptr(q_start), _ptr(out), T, W, n, _stream()),
           "token_shift_mix")


def _recurrence_lds(key_dim: int, columns: int) -> int:
    """Bytes of LDS a workgroup of ``decay_recurrence`` with ``columns`` value columns takes."""
    groups = (key_dim + RECURRENCE_CHANNELS - 1) // RECURRENCE_CHANNELS
    padded = groups * RECURRENCE_CHANNELS
    staged = 8 if padded > 128 else 16
    partial = 0 if groups & (groups - 1) == 0 else groups | 1     # none where lanes add them
    return 4 * (3 * staged * padded + 2 * padded + staged * columns * (1 + partial))


def _recurrence_columns(n_seqs: int, n_heads: int, key_dim: int, value_dim: int,
                        single: bool = False):
    """(value columns a workgroup of ``decay_recurrence`` takes, columns a thread).  Portions:
    four columns a thread where that divides, as many columns as threads and LDS hold, fewer
    where that leaves the chip idle, though not fewer than fill a wave.  ``single`` (a token a
    sequence: the state is read and written, little else): a column a thread and small
    workgroups, so that many loads are in flight.  The results do not depend on either."""
    groups = (key_dim + RECURRENCE_CHANNELS - 1) // RECURRENCE_CHANNELS
    per = 1 if single else 4
    most = max(1, min(value_dim, per * RECURRENCE_MAX_THREADS // groups, 256))
    while most > 1 and _recurrence_lds(key_dim, most) > RECURRENCE_MAX_LDS:
        most -= 1
    if single:
        floor = 8
    else:
        if most >= 8:
            most -= most % 4
        elif groups * most > RECURRENCE_MAX_THREADS:
            most = max(1, RECURRENCE_MAX_THREADS // groups)
        floor = max(8, 4 * 64 // groups // 4 * 4)
    vb = most
    while vb > floor and n_seqs * n_heads * ((value_dim + vb - 1) // vb) < RECURRENCE_WORKGROUPS:
        vb = max(floor, (vb + 1) // 2 if single else vb // 2 // 4 * 4)
    return vb, (1 if single else (4 if vb % 4 == 0 else (2 if vb % 2 == 0 else 1)))


@_launches("attention")
def decay_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, z: torch.Tensor,
                     z_bias: torch.Tensor, bonus: Optional[torch.Tensor], state: torch.Tensor,
                     state_slots: torch.Tensor, q_start: torch.Tensor, out: torch.Tensor,
                     n_heads: int, key_dim: int, value_dim: int, rule: str, tau: float = 1.0,
                     q_scale: float = 1.0, columns: Optional[int] = None,
                     max_q_len: Optional[int] = None, span: Optional[int] = None) -> None:
    """The recurrence S_t = diag(a_t) S_(t-1) + k_t v_t^T a head, token by token in 32-bit, over
    the rows of a step: ``q``, ``k`` [T, H * d] and ``v`` [T, H * dv] (contiguous rows, any row
    stride), ``z`` float32 [T, H * d] with a_t = sigmoid(z_t + z_bias)^(1 / tau) (``rule``
    "sigmoid_root") or exp(-exp(z_t + z_bias)) ("double_exp").  Without ``bonus`` the output is
    o_t = S_t^T (q_t * q_scale); with ``bonus`` u (float32 [H * d]) it is
    o_t = (S_(t-1) + diag(u) k_t v_t^T)^T (q_t * q_scale).  ``out`` float32 [T, H * dv].
    Sequence s owns the rows q_start[s] .. q_start[s + 1] - 1; its state (row state_slots[s] of
    ``state``, float32 [slots, >= ``recurrence_state_size``]) is read before its first row and
    written behind its last.  A row's result depends on the state and the rows of its own
    sequence alone, and not on how the sequence was cut into steps, beyond rounding.

    ``max_q_len``: the most rows a sequence has in this step, where the caller knows it.  Above
    two spans (``span`` tokens, by default ``RECURRENCE_SPAN`` or what keeps a sequence within
    ``RECURRENCE_MAX_SPANS``) the portions are cut into spans that run side by side: each span's
    own sum from a zero state, the states at the spans' starts one after the other
    (S <- diag(product of the span's decays) S + the span's sum), then each span's outputs from
    the state at its start.  The same numbers up to 32-bit rounding; ``z`` is then overwritten
    with the decays.  ``span`` 0, or no ``max_q_len``: token by token from end to end."""
    _need_gpu(z, z_bias, bonus, state, state_slots, q_start, out)
    for t in (q, k, v):
        if not t.is_cuda:
            raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    _i32(state_slots, "state_slots")
    _i32(q_start, "q_start")
    T = q.shape[0]
    H, d, dv = int(n_heads), int(key_dim), int(value_dim)
    n_seqs = state_slots.shape[0]
    need = recurrence_state_size(H, d, dv)
    if rule not in DECAY_RULES or not 0 < d <= RECURRENCE_MAX_KEY_DIM or dv < 1 or H < 1 \
            or q.shape[1] < H * d or k.shape[1] < H * d or v.shape[1] < H * dv \
            or k.shape[0] != T or v.shape[0] != T or k.dtype != q.dtype or v.dtype != q.dtype \
            or z.shape != (T, H * d) or z.dtype != torch.float32 \
            or z_bias.shape != (H * d,) or z_bias.dtype != torch.float32 \
            or (bonus is not None and (bonus.shape != (H * d,) or bonus.dtype != torch.float32)) \
            or out.shape != (T, H * dv) or out.dtype != torch.float32 \
            or state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] < need \
            or q_start.shape[0] != n_seqs + 1 or not tau > 0.0:
        raise KernelUnavailable(f"decay_recurrence: q {tuple(q.shape)}, k {tuple(k.shape)}, v "
                                f"{tuple(v.shape)} {q.dtype}, z {tuple(z.shape)} {z.dtype}, out "
                                f"{tuple(out.shape)} {out.dtype}, state {tuple(state.shape)} for "
                                f"{H} heads of {d} x {dv} (key size up to "
                                f"{RECURRENCE_MAX_KEY_DIM}), rule {rule!r}")
    lib = build.load("recurrent")
    longest = int(max_q_len) if max_q_len is not None else 0
    if span is None:
        span = RECURRENCE_SPAN
        if longest > span * RECURRENCE_MAX_SPANS:
            span = ((longest + RECURRENCE_MAX_SPANS - 1) // RECURRENCE_MAX_SPANS + 15) // 16 * 16
    if span and (span % 16 or span < 16):
        raise KernelUnavailable(f"decay_recurrence: a span of {span} tokens is no multiple of 16")
    if span and longest > 2 * span and z.is_contiguous():
        max_spans = (longest + span - 1) // span
        works = n_seqs * max_spans
        vb, rv = (int(columns), 0) if columns is not None else _recurrence_columns(works, H, d, dv)
        span_state = _workspace("recurrence_span_state", works * need, torch.float32, q.device)
        span_decay = _workspace("recurrence_span_decay", works * (need // dv), torch.float32,
                                q.device)
        code = lib.zf_decay_recurrence_spans(
            _ptr(q), ctypes.c_longlong(_columns(q, "decay_recurrence: q")), _ptr(k),
            ctypes.c_longlong(_columns(k, "decay_recurrence: k")), _ptr(v),
            ctypes.c_longlong(_columns(v, "decay_recurrence: v")), _dt(q), _ptr(z), _ptr(z_bias),
            _ptr(bonus), _ptr(state), ctypes.c_longlong(state.shape[1]), _ptr(state_slots),
            _ptr(q_start), _ptr(out), T, n_seqs, H, d, dv, vb, rv, DECAY_RULES[rule],
            ctypes.c_float(1.0 / tau), ctypes.c_float(q_scale), int(span), max_spans,
            _ptr(span_state), _ptr(span_decay), _stream())
        _check(code, "decay_recurrence_spans")
        return
    vb, rv = (int(columns), 0) if columns is not None else \
        _recurrence_columns(n_seqs, H, d, dv, single=longest == 1)
    code = lib.zf_decay_recurrence(
        _ptr(q), ctypes.c_longlong(_columns(q, "decay_recurrence: q")), _ptr(k),
        ctypes.c_longlong(_columns(k, "decay_recurrence: k")), _ptr(v),
        ctypes.c_longlong(_columns(v, "decay_recurrence: v")), _dt(q), _ptr(z), _ptr(z_bias),
        _ptr(bonus), _ptr(state), ctypes.c_longlong(state.shape[1]), _ptr(state_slots),
        _ptr(q_start), _ptr(out), n_seqs, H, d, dv, vb, rv, DECAY_RULES[rule],
        ctypes.c_float(1.0 / tau), ctypes.c_float(q_scale), _stream())
    _check(code, "decay_recurrence")


@_launches("norm_rope_write")
def head_norm_gate(o: torch.Tensor, gain: torch.Tensor, gate: torch.Tensor, out: torch.Tensor,
                   n_heads: int, eps: float) -> None:
    """out[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * gain * silu(gate[t, h, :]):
    ``o`` float32 [T, H * dv]; ``gain`` float32 [dv] (one for all heads) or [H * dv]; ``gate``
    (contiguous rows, any row stride) and ``out`` [T, H * dv] in the products' type."""
    _need_gpu(o, gain, out)
    if not gate.is_cuda:
        raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    T, width = o.shape
    H = int(n_heads)
    dv = width // H if H > 0 else 0
    if H < 1 or dv * H != width or o.dtype != torch.float32 or gain.dtype != torch.float32 \
            or gain.shape not in ((dv,), (width,)) or gate.shape != (T, width) \
            or out.shape != (T, width) or gate.dtype != out.dtype:
        raise KernelUnavailable(f"head_norm_gate: o {tuple(o.shape)} {o.dtype}, gain "
                                f"{tuple(gain.shape)}, gate {tuple(gate.shape)} {gate.dtype}, out "
                                f"{tuple(out.shape)} {out.dtype}, {H} heads")
    lib = build.load("recurrent")
    per_head = 1 if gain.shape == (width,) and H > 1 else 0
    _check(lib.zf_head_norm_gate(_ptr(o), _ptr(gain), per_head, _ptr(gate),
                                 ctypes.c_longlong(_columns(gate, "head_norm_gate: gate")),
                                 _ptr(out), _dt(out), T, H, dv, ctypes.c_float(eps), _stream()),
           "head_norm_gate")


# ------------------------------------------------------------------------- the residual stream in several copies
STREAMS_MAX = 8               # STREAMS_MAX in norms.hip
STREAMS_MAX_WIDTH = 16384


@_launches("norm_rope_write")
def streams_step(x: torch.Tensor, branches=(), mix: Optional[torch.Tensor] = None,
                 out_coef: Optional[torch.Tensor] = None, *, read: bool = False,
                 in_coef: Optional[torch.Tensor] = None, gain: Optional[torch.Tensor] = None,
                 eps: float = 0.0, out: Optional[torch.Tensor] = None) -> None:
    """Around a sublayer of a model whose residual stream is kept in S copies ``x`` float32
    [S, T, W] (a view whose copies are contiguous [T, W] matrices a fixed distance apart), row by
    row, all 32-bit.  With ``branches`` = one or two (y float32 [T, W], factor): y = the sum of
    factor * y, and x_t <- sum_s mix[s, t] x_s + out_coef[t] * y for all t at once from the old
    copies (``mix`` float32 [S, S], ``out_coef`` float32 [S]).  With ``read``: u = sum_s
    in_coef[s] x_s over the (new) copies (``in_coef`` None: all ones), and ``out`` [T, W] =
    u / sqrt(mean(u^2) + eps) * gain in out's type, or (``gain`` None) u itself as float32.
    Both halves in one launch when both are asked for."""
    _need_gpu(x, mix, out_coef, in_coef, gain, out, *[y for y, _ in branches])
    if x.dim() != 3 or x.dtype != torch.float32 or x.stride(2) != 1 or x.stride(1) != x.shape[2]:
        raise KernelUnavailable(f"streams_step: x {tuple(x.shape)} {x.dtype} must be float32 "
                                "[S, T, W] with contiguous copies")
    S, T, W = x.shape
    ok = 1 <= S <= STREAMS_MAX and 0 < W <= STREAMS_MAX_WIDTH and len(branches) <= 2 \
        and (branches or read)
    for y, _ in branches:
        ok = ok and y.shape == (T, W) and y.dtype == torch.float32 and y.is_contiguous()
    if branches:
        ok = ok and mix is not None and out_coef is not None and mix.shape == (S, S) \
            and out_coef.shape == (S,) and mix.dtype == torch.float32 \
            and out_coef.dtype == torch.float32 and mix.is_contiguous()
    if read:
        ok = ok and out is not None and out.shape == (T, W) and out.is_contiguous() \
            and (in_coef is None or (in_coef.shape == (S,) and in_coef.dtype == torch.float32)) \
            and (gain is None or (gain.shape == (W,) and gain.dtype == torch.float32)) \
            and (gain is not None or out.dtype == torch.float32)
    if not ok:
        raise KernelUnavailable(f"streams_step: x {tuple(x.shape)}, {len(branches)} branches, "
                                f"read {read}: up to {STREAMS_MAX} copies of up to "
                                f"{STREAMS_MAX_WIDTH} columns, float32 coefficients [S], [S, S]")
    y0 = branches[0][0] if branches else None
    y1 = branches[1][0] if len(branches) > 1 else None
    c0 = float(branches[0][1]) if branches else 0.0
    c1 = float(branches[1][1]) if len(branches) > 1 else 0.0
    lib = build.load("norms")
    _check(lib.zf_streams_step(_ptr(x), ctypes.c_longlong(x.stride(0) if S > 1 else T * W), S,
                               _ptr(y0), _ptr(y1), ctypes.c_float(c0), ctypes.c_float(c1),
                               _ptr(mix), _ptr(out_coef), _ptr(in_coef), _ptr(gain),
                               ctypes.c_float(eps), _ptr(out), _dt(out) if out is not None else 0,
                               T, W, 1 if read else 0, _stream()), "streams_step")


# ------------------------------------------------------------------------- the gated delta rule
DELTA_MAX_KEY_DIM = 256
DELTA_CHANNELS = (8, 12, 16)      # key channels a thread holds (instantiations in delta.hip)
DELTA_MAX_LANES = 16              # lanes that share a column's key channels
SHORT_CONV_MAX_TAPS = 8           # DL_CONV_MAX_TAPS in delta.hip
SHORT_CONV_MAX_HEAD_DIM = 1024    # a head that leaves as a unit vector lies in one workgroup


def delta_plan(key_dim: int) -> Tuple[int, int]:
    """(channels a thread, lanes a column) for heads of ``key_dim``: the padded key size
    channels * lanes is the smallest of 8, 12, 16, 24, 32, 48, ... that holds the head, and as
    many lanes (a power of two, at most ``DELTA_MAX_LANES``) share a column as leave a thread
    at least 8 channels.  A function of the key size alone: a request's state is laid out by it."""
    best = None
    for r in DELTA_CHANNELS:
        lanes = 1
        while lanes <= DELTA_MAX_LANES:
            if r * lanes >= key_dim:
                if best is None or (r * lanes, -lanes) < (best[0] * best[1], -best[1]):
                    best = (r, lanes)
                break
            lanes *= 2
    if best is None:
        raise KernelUnavailable(f"delta rule: key size {key_dim} beyond {DELTA_MAX_KEY_DIM}")
    return best


def delta_state_size(n_heads: int, key_dim: int, value_dim: int) -> int:
    """Floats of a request's matrices: [head][value column][padded key size]."""
    r, lanes = delta_plan(key_dim)
    return n_heads * value_dim * r * lanes


def delta_state_matrix(state: torch.Tensor, n_heads: int, key_dim: int,
                       value_dim: int) -> torch.Tensor:
    """The matrices S [slots, H, d, dv] that the leading part of state rows holds (a copy)."""
    r, lanes = delta_plan(key_dim)
    P = r * lanes
    m = state[:, :n_heads * value_dim * P].reshape(state.shape[0], n_heads, value_dim, P)
    return m[..., :key_dim].transpose(2, 3).contiguous()


@_launches("norm_rope_write")
def short_conv(src: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, state_offset: int,
               state_slots: torch.Tensor, seq_index: torch.Tensor, q_start: torch.Tensor,
               out: torch.Tensor, unit_heads: int = 0, head_dim: int = 1, scaled_heads: int = 0,
               scale: float = 1.0, unit_eps: float = 0.0, single_tokens: bool = False) -> None:
    """out[t, c] = silu(sum_j taps[c, j] * x_(t - n + 1 + j)[c]) over the rows of a step: ``src``
    [T, >= C] (contiguous rows, any row stride), ``taps`` float32 [C, n] (the last column is the
    token's own), ``out`` float32 [T, C].  Rows before a sequence's portion come from its state:
    [n - 1, C] floats from ``state_offset`` on in row state_slots[s] of ``state`` (float32
    [slots, width]), oldest first; zeros for a new request.  After the step the state holds the
    last n - 1 rows seen.  The leading ``unit_heads`` * ``head_dim`` channels are heads that
    leave as unit vectors x / sqrt(sum x^2 + unit_eps), the first ``scaled_heads`` of them times
    ``scale``.  ``single_tokens``: every sequence brings one token (one launch instead of two)."""
    _need_gpu(taps, state, state_slots, seq_index, q_start, out)
    if not src.is_cuda:
        raise KernelUnavailable("the HIP kernels run on GPU tensors only")
    for t, name in ((state_slots, "state_slots"), (seq_index, "seq_index"), (q_start, "q_start")):
        _i32(t, name)
    T = src.shape[0]
    C, n = taps.shape
    n_seqs = state_slots.shape[0]
    if taps.dtype != torch.float32 or not taps.is_contiguous() or src.shape[1] < C \
            or out.shape != (T, C) or out.dtype != torch.float32 or not out.is_contiguous() \
            or state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 \
            or state_offset < 0 or state_offset + (n - 1) * C > state.shape[1] \
            or seq_index.shape[0] != T or q_start.shape[0] != n_seqs + 1 \
            or unit_heads < 0 or head_dim < 1 or unit_heads * head_dim > C \
            or n > SHORT_CONV_MAX_TAPS or head_dim > SHORT_CONV_MAX_HEAD_DIM \
            or scaled_heads > unit_heads or (single_tokens and T != n_seqs):
        raise KernelUnavailable(f"short_conv: src {tuple(src.shape)}, taps {tuple(taps.shape)} "
                                f"{taps.dtype}, out {tuple(out.shape)} {out.dtype}, state "
                                f"{tuple(state.shape)} from {state_offset}")
    lib = build.load("delta")
    _check(lib.zf_short_conv(_ptr(src), _dt(src), ctypes.c_longlong(_columns(src, "short_conv: src")),
                             _ptr(taps), n, _ptr(state), ctypes.c_longlong(state.stride(0)),
                             ctypes.c_longlong(state_offset), _ptr(state_slots), _ptr(seq_index),
                             _ptr(q_start), _ptr(out), T, n_seqs, C, int(unit_heads),
                             int(head_dim), int(scaled_heads), ctypes.c_float(scale),
                             ctypes.c_float(unit_eps), 1 if single_tokens else 0, _stream()),
           "short_conv")


@_launches("attention")
def delta_recurrence(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, ab: torch.Tensor,
                     decay_log: torch.Tensor, decay_bias: torch.Tensor, state: torch.Tensor,
                     state_slots: torch.Tensor, q_start: torch.Tensor, out: torch.Tensor,
                     n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int) -> None:
    """The gated delta rule a head, token by token in 32-bit, over the rows of a step:
    S <- g S; w = beta (v - S^T k); S <- S + k w^T; o = S^T q.  ``qkv`` float32 [T, C] holds
    ``n_kv_heads`` q heads of ``key_dim`` from column q_off, as many k heads from k_off and
    ``n_heads`` v heads of ``value_dim`` from v_off (value head n reads q/k head
    floor(n / (n_heads / n_kv_heads))); ``ab`` float32 [T, 2 H]: z_a, then z_b, with
    g = exp(-exp(decay_log) * softplus(z_a + decay_bias)) and beta = sigmoid(z_b)
    (``decay_log``, ``decay_bias`` float32 [H]).  ``out`` float32 [T, H * dv].  Sequence s owns
    the rows q_start[s] .. q_start[s + 1] - 1; its matrices (the leading ``delta_state_size``
    floats of row state_slots[s] of ``state``) are read before its first row and written behind
    its last.  A row's result depends on the state and the rows of its own sequence alone."""
    _need_gpu(qkv, ab, decay_log, decay_bias, state, state_slots, q_start, out)
    _i32(state_slots, "state_slots")
    _i32(q_start, "q_start")
    T, C = qkv.shape
    H, KH, d, dv = int(n_heads), int(n_kv_heads), int(key_dim), int(value_dim)
    n_seqs = state_slots.shape[0]
    if not 0 < d <= DELTA_MAX_KEY_DIM or H < 1 or KH < 1 or H % KH != 0 or dv < 1:
        raise KernelUnavailable(f"delta_recurrence: {H} heads on {KH} of {d} x {dv} (key size up "
                                f"to {DELTA_MAX_KEY_DIM})")
    r, lanes = delta_plan(d)
    need = H * dv * r * lanes
    if qkv.dtype != torch.float32 or not qkv.is_contiguous() or min(q_off, k_off, v_off) < 0 \
            or max(q_off, k_off) + KH * d > C or v_off + H * dv > C \
            or ab.shape != (T, 2 * H) or ab.dtype != torch.float32 or not ab.is_contiguous() \
            or decay_log.shape != (H,) or decay_bias.shape != (H,) \
            or decay_log.dtype != torch.float32 or decay_bias.dtype != torch.float32 \
            or out.shape != (T, H * dv) or out.dtype != torch.float32 or not out.is_contiguous() \
            or state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] < need \
            or state.stride(1) != 1 or state.stride(0) % 4 != 0 or state.data_ptr() % 16 != 0 \
            or q_start.shape[0] != n_seqs + 1:
        raise KernelUnavailable(f"delta_recurrence: qkv {tuple(qkv.shape)} {qkv.dtype}, ab "
                                f"{tuple(ab.shape)}, out {tuple(out.shape)}, state "
                                f"{tuple(state.shape)} (rows a multiple of 4 floats, at least "
                                f"{need})")
    # a workgroup: whole waves, at most 256 threads, no more columns than the head has
    cols = min(256, (dv * lanes + 63) // 64 * 64) // lanes
    lib = build.load("delta")
    _check(lib.zf_delta_recurrence(_ptr(qkv), C, int(q_off), int(k_off), int(v_off), _ptr(ab),
                                   _ptr(decay_log), _ptr(decay_bias), _ptr(state),
                                   ctypes.c_longlong(state.stride(0)), _ptr(state_slots),
                                   _ptr(q_start), _ptr(out), n_seqs, H, KH, d, dv, r, lanes, cols,
                                   _stream()), "delta_recurrence")
