#!/usr/bin/env python3
"""Throughput of the engine with random bfloat16 weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The default run (``--workload decode``) has the layer sizes of the Qwen3-8B configuration (36
layers, hidden 4096, 32 query heads on 8 kv heads of 128, intermediate 12288, vocabulary
151936), a batch of 8 requests with 2048-token prompts of random ids and pages of 16 tokens.
A "step" is one decode step of the batch; ``value`` is decoded tokens a second over exactly K
timed steps after W warm-up steps, through the engine's own scheduler, step function, cache
and kernels.  The same line reports a 2048-token prefill, the decode step's HBM roofline,
decode at batch 1 and 64, prefills of 512 and 8192 tokens and, unless ``--no-points``, the two
other workloads below in short form.

``--workload continuous``: the Qwen3-14B shape (40 layers, hidden 5120, 40 / 8 heads of 128,
intermediate 17408): 32 requests arrive together, prompt lengths uniform in [128, 4096], 256
greedy tokens each, prompts cut into 512-token portions that run beside the other requests'
decode tokens, through the product's scheduler.  ``value`` is all tokens (prompt and
generated) a second.

``--workload long-context``: the Qwen3-32B shape (64 layers, hidden 5120, 64 / 8 heads of 128,
intermediate 25600; 65.5 GB of weights): a 2048-token prefill, then decode at batch 1, 8 and
64 with every request's context just below 8192 tokens; the cache pool is sized for
64 x 8192 tokens (137 GB).

``--workload fezupel``, ``--workload lodenex``, ``--workload nupovik`` and ``--workload kugisun``: shapes of those
designs at layer sizes that resemble served models, each beside the dense Qwen3 decoder of equal
size (prefill of 2048 tokens, decode at batch 8), and their kernels alone beside the like
kernels of that decoder.

The reference publishes no numbers, so ``vs_baseline`` is null.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                      # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PAGE = 16


def _shape(layers, hidden, heads, inter, tied=False):
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=layers,
                hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=8,
                head_dim=128, intermediate_size=inter, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=tied, max_position_embeddings=40960,
                torch_dtype="bfloat16")


# (the three smaller shapes tie the head to the embedding)
SHAPES = {"0.6b": _shape(28, 1024, 16, 3072, True), "1.7b": _shape(28, 2048, 16, 6144, True),
          "4b": _shape(36, 2560, 32, 9728, True), "8b": _shape(36, 4096, 32, 12288),
          "14b": _shape(40, 5120, 40, 17408), "32b": _shape(64, 5120, 64, 25600)}
SHAPE_NAMES = {"0.6b": "Qwen3-0.6B", "1.7b": "Qwen3-1.7B", "4b": "Qwen3-4B", "8b": "Qwen3-8B",
               "14b": "Qwen3-14B", "32b": "Qwen3-32B"}


def build_llm(raw: dict, dtype: str, seed: int, pool_tokens: int, max_seqs: int, **sched):
    """The engine over the product's random-weights mode (matrices and the embedding
    N(0, 0.02), norm gains 1 + U(-0.1, 0.1), drawn on the device) with a pool for
    ``pool_tokens`` tokens."""
    from zinfer_amd.entrypoints import LLM
    return LLM(config=raw, random_seed=seed, dtype=dtype, device="cuda:0", page_size=PAGE,
               num_pages=(pool_tokens + PAGE - 1) // PAGE + 8, max_seqs=max_seqs, **sched)


def drop(llm) -> None:
    """Gives the model's and the pool's memory back before the next shape is built."""
    import gc
    import torch
    import zinfer_amd.ops as ops
    llm.engine._graphs.clear()
    llm.engine = llm.model = None
    ops._workspaces.clear()
    gc.collect()
    torch.cuda.empty_cache()


def weight_bytes_per_step(cfg, elem: int) -> int:
    """Bytes of weights a decode step has to read: every matrix once (layers and head) and
    the norm gains (32-bit); the embedding rows of the batch are negligible and left out."""
    H, I, hd = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * hd * H
    per_layer = qkv + H * cfg.num_attention_heads * hd + 2 * I * H + H * I
    gains = cfg.num_hidden_layers * (2 * H + 2 * hd) + H
    return (cfg.num_hidden_layers * per_layer + cfg.vocab_size * H) * elem + gains * 4


def kv_bytes_per_token(cfg, elem: int) -> int:
    return 2 * cfg.num_hidden_layers * cfg.num_key_value_heads * cfg.head_dim * elem


def linear_flops_per_token(cfg) -> float:
    H, I, hd, nH = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim, cfg.num_attention_heads
    qkv = (nH + 2 * cfg.num_key_value_heads) * hd * H
    return 2.0 * (qkv + H * nH * hd + 3 * I * H) * cfg.num_hidden_layers


def prefill_flops(cfg, T: int) -> float:
    """2 flops per multiply-add: the layers' matrices for T tokens, causal attention
    (QK^T and PV over T (T + 1) / 2 pairs), the head for one row."""
    attn = 2.0 * 2.0 * (T * (T + 1) / 2) * cfg.head_dim * cfg.num_attention_heads \
        * cfg.num_hidden_layers
    return linear_flops_per_token(cfg) * T + attn + 2.0 * cfg.vocab_size * cfg.hidden_size


def prefill_record(cfg, T: int, seconds: float, peak: float, mfma_rate=None) -> dict:
    """``frac``: of the published peak; ``frac_of_mfma_loop``: of what a loop of MFMAs alone
    reaches on random operands on this card (``ops.measure_mfma_rate``)."""
    flops = prefill_flops(cfg, T)
    out = {"value": round(T / seconds, 1), "tokens": T, "ms": round(seconds * 1e3, 3),
           "frac": round(flops / seconds / peak, 4)}
    if mfma_rate:
        out["mfma_loop_tflops"] = round(mfma_rate / 1e12, 1)
        out["frac_of_mfma_loop"] = round(flops / seconds / mfma_rate, 4)
    return out


def run_prefill(llm, cfg, T: int, seed: int) -> float:
    import torch
    from zinfer_amd.engine import StepEntry
    g = torch.Generator().manual_seed(seed)
    eng = llm.engine
    times = []
    for i in range(3):                       # the first pass warms caches and work buffers
        toks = torch.randint(0, cfg.vocab_size, (T,), generator=g).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = eng.step([StepEntry(f"prefill{i}", toks, [T - 1])], end=[f"prefill{i}"])
        eng.argmax(logits)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return min(times[1:])


def decode_lead(batch: int, prompt_len: int, step_tokens: int) -> int:
    """How many tokens the first request of ``batch`` may have decoded by the time the last
    one's prompt is through: a step's token budget is shared between one prompt's portion and
    the decode tokens of the requests already running."""
    room = max(1, step_tokens - batch)
    return batch * ((prompt_len + room - 1) // room)


def run_decode(llm, cfg, batch: int, prompt_len: int, steps: int, warmup: int, seed: int,
               classes: bool = False):
    """Prefills ``batch`` requests through the scheduler, runs ``warmup`` untimed decode
    steps, then times exactly ``steps`` steps.  Returns (seconds, mean context length), and
    with ``classes`` a third value: where a step's time goes (see ``step_classes``)."""
    import torch
    from zinfer_amd.sampling import SamplingParams
    g = torch.Generator().manual_seed(seed)
    sched = llm.new_scheduler()
    sched.max_step_tokens = max(sched.max_step_tokens, min(prompt_len, 8192))
    sched.chunk_size = sched.max_step_tokens
    # requests admitted early decode while later prompts are still being run, so they may be
    # many tokens ahead; none may finish before the timed steps are over
    ahead = decode_lead(batch, prompt_len, sched.chunk_size)
    params = SamplingParams(temperature=0.0, max_new_tokens=warmup + steps + ahead + 8,
                            ignore_eos=True)
    for _ in range(batch):
        sched.add_request(torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist(),
                          params)
    while sched.waiting or any(r.pending > 1 or not r.generated for r in sched.running):
        sched.step()                         # prompts, one or more per step
    assert len(sched.running) == batch
    most = sched.multi_step

    def run_exactly(n):
        """``n`` decode steps of the whole batch; the scheduler may run several in a row on
        the device per call, never more than are still to do."""
        done = 0
        while done < n:
            sched.multi_step = min(most, n - done)
            sched.step()
            assert sched.last_steps >= 1
            done += sched.last_steps
        assert done == n

    run_exactly(warmup)
    torch.cuda.synchronize()
    ctx0 = sum(r.n_computed for r in sched.running) / batch
    if classes:
        llm.engine.step_trace = []
    t0 = time.perf_counter()
    run_exactly(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(r.n_computed for r in sched.running) / batch
    assert len(sched.running) == batch and sched.n_preemptions == 0
    where = None
    if classes:
        trace, llm.engine.step_trace = llm.engine.step_trace, None
        where = step_classes(llm.engine, sched, trace, steps, dt)
    for r in list(sched.running):
        sched._finish(r, "bench")
    return (dt, (ctx0 + ctx1) / 2 + 0.5) + ((where,) if classes else ())


def step_classes(eng, sched, trace, steps: int, seconds: float) -> dict:
    """Where a decode step's time goes, in milliseconds a step.  ``host``: the host's work for
    the timed steps (packing metadata, launching), which runs beside the device's;
    ``device``: between the events around the timed steps' kernels; the classes: a graph of
    the same step with only that class's kernels, replayed (``Engine.class_times``: products =
    the layers' matrix products with what is fused into them (norms, SwiGLU, residual sums),
    attention = attention over the cache, in steps of up to 32 sequences with the per-head
    norm, rotation and cache write; norm_rope_write = those as kernels of their own;
    head_sampling = final norm, head, arg-max)."""
    from zinfer_amd.engine import StepEntry
    host = sum(r[2] + r[3] for r in trace) / steps
    device = sum(r[4].elapsed_time(r[5]) for r in trace) / 1e3 / steps
    entries = [StepEntry(r.id, [r.generated[-1]], [0]) for r in sched.running]
    t = eng.class_times(entries)
    out = {k + "_ms": round(v * 1e3, 4) for k, v in t.items() if k != "step"}
    out["classes_sum_ms"] = round(sum(v for k, v in t.items() if k != "step") * 1e3, 4)
    out["graph_step_ms"] = round(t["step"] * 1e3, 4)
    out["device_ms"] = round(device * 1e3, 4)
    out["host_ms"] = round(host * 1e3, 4)
    out["wall_ms"] = round(seconds / steps * 1e3, 4)
    return out


def decode_roofline(cfg, elem: int, batch: int, mean_ctx: float, seconds_per_step: float,
                    measured_gbs: float = None) -> dict:
    """``measured``: what a kernel that only reads (16-byte non-temporal loads, 8 in flight a
    lane, a workgroup 64 KB in a row, 2 GiB from HBM, the best pass between two events over 256
    to 4096 workgroups) reaches on this card."""
    step_bytes = weight_bytes_per_step(cfg, elem) + batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / seconds_per_step / 1e9
    out = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
           "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)}
    if measured_gbs:
        out["measured_read"] = round(measured_gbs, 1)
        out["frac_of_measured"] = round(achieved / measured_gbs, 4)
    return out


def config_of(cfg, shape: str, **more) -> dict:
    out = {"model": f"{SHAPE_NAMES[shape]} shape, random weights",
           "layers": cfg.num_hidden_layers,
           "layers_of_config": SHAPES[shape]["num_hidden_layers"],
           "hidden_size": cfg.hidden_size, "num_attention_heads": cfg.num_attention_heads,
           "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
           "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
           "page_size": PAGE, "parallelism": "single GPU", "sampling": "greedy"}
    out.update(more)
    return out


# --------------------------------------------------------------------------- continuous batching
def run_continuous(llm, cfg, elem: int, n_requests: int, lo: int, hi: int, new_tokens: int,
                   seed: int) -> dict:
    """All requests arrive together; the scheduler admits them, cuts their prompts into
    portions beside the decode tokens of the others, decodes, finishes and frees.  The
    workload runs three times with the same requests; the third pass is timed (the first
    settles work buffers and captures the decode graph of every batch shape that occurs, the
    second records the runs of decode steps whose shape came a second time: a server that has
    been up for a while)."""
    import torch
    from zinfer_amd.sampling import SamplingParams
    eng = llm.engine
    out = {}
    for timed in (False, False, True):
        g = torch.Generator().manual_seed(seed)
        lens = torch.randint(lo, hi + 1, (n_requests,), generator=g).tolist()
        sched = llm.new_scheduler()
        params = SamplingParams(temperature=0.0, max_new_tokens=new_tokens, ignore_eos=True)
        for n in lens:
            sched.add_request(torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist(), params)
        eng.step_trace = []
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        first_done = None
        prompts_done = None
        while sched.has_work():
            done = sched.step()
            if prompts_done is None and not sched.waiting and \
                    all(r.generated for r in sched.running):
                torch.cuda.synchronize()
                prompts_done = time.perf_counter() - t0
            if done and first_done is None:
                first_done = time.perf_counter() - t0
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        trace, eng.step_trace = eng.step_trace, None
        if not timed:
            continue
        generated = sum(len(r.generated) for r in sched.finished.values())
        assert generated == n_requests * new_tokens
        prompt_tokens = sum(lens)
        mixed = [r for r in trace if r[6]]                  # steps with a prompt portion

        def summary(rows):
            if not rows:
                return None
            dev = sum(r[4].elapsed_time(r[5]) for r in rows) / 1e3
            return {"steps": len(rows), "tokens": sum(r[0] for r in rows),
                    "host_pack_ms": round(sum(r[2] for r in rows) / len(rows) * 1e3, 3),
                    "host_launch_ms": round(sum(r[3] for r in rows) / len(rows) * 1e3, 3),
                    "device_ms": round(dev / len(rows) * 1e3, 3), "device_s": round(dev, 3)}

        mixed_s = summary(mixed)
        # roofline of the mean step with a prompt portion: its matrices' flops and the bytes
        # it must read (every weight once, the cache of the live requests about once)
        if mixed_s:
            t_step = mixed_s["device_ms"] / 1e3
            toks = mixed_s["tokens"] / mixed_s["steps"]
            flops = linear_flops_per_token(cfg) * toks
            mixed_s["tokens_per_step"] = round(toks, 1)
            mixed_s["frac_mfma"] = round(flops / t_step / PEAK_FLOPS["bf16"], 4)
            mixed_s["frac_hbm_weights"] = round(
                weight_bytes_per_step(cfg, elem) / t_step / 1e9 / HBM_PEAK_GBS, 4)
        out = {"seconds": round(dt, 3), "total_tok_s": round((prompt_tokens + generated) / dt, 1),
               "decode_tok_s": round(generated / dt, 1), "prompt_tokens": prompt_tokens,
               "generated_tokens": generated, "engine_steps": sched.n_steps,
               "scheduler_calls": len(trace), "preemptions": sched.n_preemptions,
               "prompts_done_s": round(prompts_done or 0.0, 3),
               "first_finished_s": round(first_done or 0.0, 3),
               "device_busy_frac": round(sum(r[4].elapsed_time(r[5]) for r in trace) / 1e3 / dt, 4),
               "mixed_steps": mixed_s, "decode_calls": summary([r for r in trace if not r[6]])}
    return out


def main_continuous(args) -> int:
    raw = dict(SHAPES[args.shape or "14b"])
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    n, lo, hi, new = args.requests, args.prompt_min, args.prompt_max, args.new_tokens
    t_build = time.perf_counter()
    step_tokens = args.step_tokens or args.chunk
    llm = build_llm(raw, args.dtype, args.seed, n * (hi + new + PAGE), n,
                    max_step_tokens=step_tokens, chunk_size=args.chunk,
                    multi_step=args.multi_step)
    cfg = llm.config
    build_s = time.perf_counter() - t_build
    llm.engine.capture_runs = not args.no_run_graphs
    elem = 2 if args.dtype == "bfloat16" else 4
    res = run_continuous(llm, cfg, elem, n, lo, hi, new, args.seed + 7)
    line = {"metric": f"continuous batching tok/s (prompt + generated), "
                      f"{SHAPE_NAMES[args.shape or '14b']} shape, {n} requests",
            "value": res["total_tok_s"], "unit": "tokens/s", "n_gpus": 1,
            "steps": res["engine_steps"], "warmup": res["engine_steps"],
            "ms_per_step": round(res["seconds"] / max(res["engine_steps"], 1) * 1e3, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": config_of(cfg, args.shape or "14b", requests=n, prompt_min=lo,
                                prompt_max=hi, new_tokens=new, chunk_size=args.chunk,
                                max_step_tokens=step_tokens,
                                steps_in_a_row=args.multi_step),
            "continuous": res, "build_s": round(build_s, 1)}
    print(json.dumps(line))
    return 0


# --------------------------------------------------------------------------- long context
def run_long_context(llm, cfg, elem: int, context: int, batches, steps: int, seed: int) -> dict:
    """Decode with every request's context just below ``context``: prompts of
    ``context - steps - warm-up`` tokens are run through the scheduler, then the timed steps
    end at ``context``."""
    out = {}
    for b in batches:
        warm = 16
        prompt_len = context - steps - warm - b * ((context + 8191) // 8192) - 8
        dt, mean_ctx = run_decode(llm, cfg, b, prompt_len, steps, warm, seed + b)
        out[f"decode_b{b}"] = round(b * steps / dt, 1)
        out[f"decode_b{b}_ms"] = round(dt / steps * 1e3, 3)
        out[f"decode_b{b}_ctx"] = int(round(mean_ctx))
        out[f"decode_b{b}_hbm_frac"] = decode_roofline(cfg, elem, b, mean_ctx, dt / steps)["frac"]
    return out


def main_long_context(args) -> int:
    import torch
    shape = args.shape or "32b"
    raw = dict(SHAPES[shape])
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    context = args.context
    batches = tuple(int(b) for b in args.batches.split(","))
    t_build = time.perf_counter()
    llm = build_llm(raw, args.dtype, args.seed, max(batches) * (context + PAGE), max(batches),
                    max_step_tokens=8192, multi_step=args.multi_step)
    cfg = llm.config
    build_s = time.perf_counter() - t_build
    elem = 2 if args.dtype == "bfloat16" else 4
    free, total = torch.cuda.mem_get_info()
    pre_s = run_prefill(llm, cfg, args.prefill_tokens, args.seed + 1)
    steps = max(16, min(args.steps, 64))
    res = run_long_context(llm, cfg, elem, context, batches, steps, args.seed + 2)
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    hb = 8 if 8 in batches else max(batches)      # the batch of the headline
    line = {"metric": f"decode tok/s at context {context}, {SHAPE_NAMES[shape]} shape, batch {hb}",
            "value": res[f"decode_b{hb}"], "unit": "tokens/s", "n_gpus": 1, "steps": steps,
            "warmup": 16, "ms_per_step": res[f"decode_b{hb}_ms"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": config_of(cfg, shape, global_batch=hb, seq_len=context,
                                pool_tokens=max(batches) * (context + PAGE),
                                steps_in_a_row=args.multi_step),
            "prefill": prefill_record(cfg, args.prefill_tokens, pre_s, peak),
            "roofline": {"bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": res[f"decode_b{hb}_hbm_frac"],
                         "achieved": round(res[f"decode_b{hb}_hbm_frac"] * HBM_PEAK_GBS, 1)},
            "points": res, "weights_gb": round(weight_bytes_per_step(cfg, elem) / 1e9, 1),
            "pool_gb": round(llm.engine.cache.kv_bytes() / 1e9, 1),
            "free_gb_after_build": round(free / 1e9, 1), "build_s": round(build_s, 1)}
    print(json.dumps(line))
    return 0


# --------------------------------------------------------------------------- the default line
def check_fp32(llm, cfg, raw, seed: int, T: int) -> dict:
    """What bfloat16 costs at this shape: the same random weights (bfloat16 values widened)
    through the true 32-bit path (FMA products, 32-bit attention, 32-bit cache) beside the
    serving engine, on one prompt of ``T`` tokens: its first 512 tokens as one step, the rest
    as a second, then one decode token (the 32-bit arg-max) at context ``T``.  For each of the
    three places: the largest difference of the logits relative to their largest magnitude,
    the root-mean-square difference relative to their root-mean-square, and whether the
    arg-max agrees."""
    import torch
    from zinfer_amd.engine import Engine, StepEntry
    from zinfer_amd.models.build import random_model
    g = torch.Generator().manual_seed(seed + 99)
    toks = torch.randint(0, cfg.vocab_size, (T,), generator=g).tolist()
    head = min(512, T)
    # same seed, same draws, rounded to bfloat16 as the serving model's, then widened
    _, model32 = random_model(raw, seed, "float32", "cuda:0", store_dtype="bfloat16")
    eng32 = Engine(model32, page_size=PAGE, num_pages=(T + 1 + PAGE - 1) // PAGE + 1,
                   max_requests=2)
    out = {"tokens": T}
    t0 = time.perf_counter()
    cuts = [("prefill_%d" % head, toks[:head])]
    if T > head:
        cuts.append(("prefill_%d" % T, toks[head:]))
    nxt = None
    for name, part in cuts + [("decode_ctx%d" % T, None)]:
        part = [nxt] if part is None else part
        entry = [StepEntry("chk", part, [len(part) - 1])]
        lb = llm.engine.step(entry).float().clone()
        lf = eng32.step(entry).float()
        nxt = int(lf.argmax())
        out[name] = {
            "rel_max_diff": round(float((lb - lf).abs().max() / lf.abs().max()), 5),
            "rel_rms_diff": round(float((lb - lf).pow(2).mean().sqrt() / lf.pow(2).mean().sqrt()), 5),
            "argmax_equal": bool(int(lb.argmax()) == nxt)}
    torch.cuda.synchronize()
    out["seconds"] = round(time.perf_counter() - t0, 2)
    llm.engine.release("chk")
    eng32.release("chk")
    del eng32, model32
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    return out


def main_decode(args) -> int:
    shape = args.shape or "8b"
    raw = dict(SHAPES[shape])
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    step_tokens = max(2048, args.prompt_len)
    ctx_cap = args.prompt_len + args.warmup + args.steps + 64 \
        + decode_lead(max_batch, args.prompt_len, min(step_tokens, 8192))
    longest_prefill = args.prefill_tokens if args.no_points else max(args.prefill_tokens, 8192)
    tokens = max(max_batch * ctx_cap, longest_prefill + 64)
    t_build = time.perf_counter()
    llm = build_llm(raw, args.dtype, args.seed, tokens, max_batch,
                    max_step_tokens=step_tokens, multi_step=args.multi_step)
    cfg = llm.config
    build_s = time.perf_counter() - t_build
    llm.engine.capture_runs = not args.no_run_graphs
    elem = 2 if args.dtype == "bfloat16" else 4
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]

    import zinfer_amd.ops as ops
    measured_gbs = ops.measure_read_bandwidth("cuda:0") / 1e9
    pre_s = run_prefill(llm, cfg, args.prefill_tokens, args.seed + 1)
    # what the matrix cores sustain on random operands with nothing else to do (the chip's
    # power limit sets it, far under the 2.4 GHz figure): bfloat16 only
    mfma_rate = ops.measure_mfma_rate("cuda:0") if args.dtype == "bfloat16" else None
    dt, mean_ctx, where = run_decode(llm, cfg, args.batch, args.prompt_len, args.steps,
                                     args.warmup, args.seed + 2, classes=True)
    value = args.batch * args.steps / dt
    points = {}
    if not args.no_points:
        for b in (1, 64):
            k = max(16, args.steps // 4)
            d, ctx = run_decode(llm, cfg, b, args.prompt_len, k, args.warmup, args.seed + 3 + b)
            points[f"decode_b{b}"] = round(b * k / d, 1)
            points[f"decode_b{b}_hbm_frac"] = decode_roofline(cfg, elem, b, ctx, d / k)["frac"]
        for T in (512, 1024, 8192):
            s = run_prefill(llm, cfg, T, args.seed + 5)
            points[f"prefill_{T}"] = round(T / s, 1)
            points[f"prefill_{T}_frac"] = round(prefill_flops(cfg, T) / s / peak, 4)
    line = {
        "metric": "decode tok/s, %s shape, batch %d, %d-token prompts"
                  % (SHAPE_NAMES[shape], args.batch, args.prompt_len),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt / args.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": config_of(cfg, shape, global_batch=args.batch, prompt_len=args.prompt_len,
                            seq_len=int(round(mean_ctx)), steps_in_a_row=args.multi_step),
        "prefill": prefill_record(cfg, args.prefill_tokens, pre_s, peak, mfma_rate),
        "roofline": decode_roofline(cfg, elem, args.batch, mean_ctx, dt / args.steps,
                                    measured_gbs),
        "classes": where,
        "points": points,
        "build_s": round(build_s, 1),
    }
    check_tokens = args.check_fp32 if args.check_fp32 is not None else \
        (0 if args.no_points or args.dtype != "bfloat16" else 2048)
    if check_tokens:
        line["fp32_check"] = check_fp32(llm, cfg, raw, args.seed, check_tokens)
    if not args.no_points and args.layers is None and args.dtype == "bfloat16":
        # the other two workloads in short form (their own modes report them in full)
        drop(llm)
        n = 32
        llm = build_llm(SHAPES["14b"], args.dtype, args.seed, n * (4096 + 256 + PAGE), n,
                        max_step_tokens=512, chunk_size=512, multi_step=args.multi_step)
        res = run_continuous(llm, llm.config, elem, n, 128, 4096, 256, args.seed + 7)
        points["continuous_14b_total"] = res["total_tok_s"]
        points["continuous_14b_decode"] = res["decode_tok_s"]
        points["continuous_14b_seconds"] = res["seconds"]
        points["continuous_14b_preemptions"] = res["preemptions"]
        drop(llm)
        if args.long_context_points:
            llm = build_llm(SHAPES["32b"], args.dtype, args.seed, 64 * (8192 + PAGE), 64,
                            max_step_tokens=8192, multi_step=args.multi_step)
            pre32 = run_prefill(llm, llm.config, 2048, args.seed + 1)
            points["prefill_2048_32b"] = round(2048 / pre32, 1)
            points["prefill_2048_32b_frac"] = round(prefill_flops(llm.config, 2048) / pre32 / peak, 4)
            res = run_long_context(llm, llm.config, elem, 8192, (1, 8, 64), 16, args.seed + 2)
            for k, v in res.items():
                if not k.endswith("_ctx"):
                    points[k.replace("decode_", "decode_32b_ctx8192_")] = v
            drop(llm)
    print(json.dumps(line))
    return 0


# --------------------------------------------------------------------------- Fezupel beside Qwen3
# Layer sizes that resemble served mixture-of-experts models; every shape is run beside the dense
# Qwen3 decoder of the same width, heads, head size, depth and vocabulary whose feed-forward is
# as wide as the experts one token uses (top * ff + shared ff): the same matrix work a token.
FEZUPEL_SHAPES = {
    "small": dict(width=2048, heads=16, kv_heads=4, dim=128, window=2048, experts=32, top=4,
                  ff=768, shared_ff=1024, layers=4, vocab=32768),
    "medium": dict(width=4096, heads=32, kv_heads=8, dim=128, window=2048, experts=64, top=8,
                   ff=1024, shared_ff=2048, layers=4, vocab=32768),
    "narrow-heads": dict(width=3072, heads=32, kv_heads=8, dim=96, window=1024, experts=16,
                         top=2, ff=2048, shared_ff=2048, layers=4, vocab=32768),
}


def fezupel_config(sh: dict, max_positions: int) -> dict:
    layer = {"type": "attention",
             "mixer": {"heads": sh["heads"], "kv_heads": sh["kv_heads"], "dim": sh["dim"],
                       "vdim": sh["dim"], "scale": sh["dim"] ** -0.5,
                       "mask": {"size": sh["window"]}},
             "mlp": {"kind": "moe", "router": {"experts": sh["experts"], "top": sh["top"]},
                     "expert": {"ff": sh["ff"], "limit": 7.0},
                     "shared": {"ff": sh["shared_ff"], "limit": 7.0}}}
    return {"architecture": "Fezupel", "vocab": sh["vocab"], "width": sh["width"],
            "max_positions": max_positions, "norm": {"eps": 1e-6},
            "layers": [layer] * sh["layers"]}


def dense_twin(sh: dict, max_positions: int) -> dict:
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3",
                num_hidden_layers=sh["layers"], hidden_size=sh["width"],
                num_attention_heads=sh["heads"], num_key_value_heads=sh["kv_heads"],
                head_dim=sh["dim"], intermediate_size=sh["top"] * sh["ff"] + sh["shared_ff"],
                vocab_size=sh["vocab"], rope_theta=1000000.0, rms_norm_eps=1e-6,
                tie_word_embeddings=False, max_position_embeddings=max_positions,
                torch_dtype="bfloat16")


def _timed(fn, repeats: int = 20) -> float:
    """Seconds of one call of ``fn`` (launches on the current stream), the mean of ``repeats``
    between two events after two calls that warm up."""
    import torch
    fn()
    fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(repeats):
        fn()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) * 1e-3 / repeats


def fezupel_kernels(sh: dict, T: int, ctx: int, mfma_rate: float, read_bw: float) -> dict:
    """The new design's kernels alone beside the like kernels of the dense decoder, at ``T``
    tokens of one sequence that holds ``ctx`` tokens (T = ctx: a prompt; T = 1 x 8 sequences: a
    decode step), each with the fraction of its bound it reaches: matrix work against the MFMA
    loop's rate (prompt) or bytes read against the measured read stream (decode)."""
    import torch
    import zinfer_amd.ops as ops
    dev = "cuda:0"
    W, nH, nKV, hd = sh["width"], sh["heads"], sh["kv_heads"], sh["dim"]
    E, top, ff, sff = sh["experts"], sh["top"], sh["ff"], sh["shared_ff"]
    bf = torch.bfloat16
    decode = T == 1
    n_seqs = 8 if decode else 1
    rows = n_seqs * T
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *shape: (torch.randn(shape, generator=g, device=dev) * 0.05).to(bf)
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)
    pages = (ctx + PAGE - 1) // PAGE
    table = torch.arange(n_seqs * pages, dtype=torch.int32, device=dev).view(n_seqs, pages)
    q_start = i32([i * T for i in range(n_seqs + 1)])
    ctx_len = i32([ctx] * n_seqs)
    seq_index = i32([i for i in range(n_seqs) for _ in range(T)])
    out = {}
    # ---- attention: keys (and values) of ctx tokens per sequence
    q = rnd(rows, nH * hd)
    gate = rnd(rows, nH * hd)
    k_pool = rnd(n_seqs * pages, nKV * PAGE * hd)
    v_pool = rnd(n_seqs * pages, nKV * PAGE * hd)
    o = torch.empty((rows, nH * hd), dtype=bf, device=dev)
    window = sh["window"]
    seen = min(ctx, window)
    pairs = n_seqs * (seen if decode else sum(min(i + 1, window) for i in range(T)))
    att_flops = 4.0 * pairs * hd * nH
    t_new = _timed(lambda: ops.tied_attention(q, gate, k_pool, table, q_start, ctx_len,
                                              seq_index, o, hd ** -0.5, window, True, nH,
                                              nKV, hd, PAGE, T, ctx))
    t_old = _timed(lambda: ops.paged_attention(q, k_pool, v_pool, table, q_start, ctx_len,
                                               seq_index, o, hd ** -0.5, window, nH, nKV, hd,
                                               PAGE, T, ctx))
    if decode:
        kb = n_seqs * seen * nKV * hd * 2
        out["attention"] = {"fezupel_us": round(t_new * 1e6, 1), "qwen3_us": round(t_old * 1e6, 1),
                            "fezupel_frac_of_read": round(kb / t_new / read_bw, 4),
                            "qwen3_frac_of_read": round(2 * kb / t_old / read_bw, 4)}
    else:
        out["attention"] = {"fezupel_us": round(t_new * 1e6, 1), "qwen3_us": round(t_old * 1e6, 1),
                            "fezupel_frac_of_mfma": round(att_flops / t_new / mfma_rate, 4),
                            "qwen3_frac_of_mfma": round(att_flops / t_old / mfma_rate, 4)}
    # ---- feed-forward: the routed experts beside a dense feed-forward of top * ff
    h = rnd(rows, W)
    router = torch.randn((E, W), generator=g, device=dev) * 0.05
    ids = torch.empty((rows, top), dtype=torch.int32, device=dev)
    share = torch.empty((rows, top), dtype=torch.float32, device=dev)
    gate_up = rnd(E, 2 * ff, W)
    down = rnd(E, W, ff)
    res = torch.zeros((rows, W), dtype=torch.float32, device=dev)
    moe = _moe_launcher(ops, h, router, ids, share, gate_up, down, res, top, ff)
    t_moe = _timed(moe)
    inter = top * ff
    wgu = ops.pretile_weight(ops.interleave_gate_up(rnd(inter, W), rnd(inter, W)))
    wd = ops.pretile_weight(rnd(W, inter))
    act = torch.empty((rows, inter), dtype=bf, device=dev)

    def dense():
        ops.gemm_swiglu(h, wgu, act, w_tiled=True)
        ops.gemm(act, wd, res, accumulate=True, w_tiled=True)
    t_dense = _timed(dense)
    ff_flops = 2.0 * rows * 3 * inter * W
    if decode:
        used = min(E, rows * top)        # at most this many experts' matrices are read
        mb, db = used * 3 * ff * W * 2, 3 * inter * W * 2
        out["feed_forward"] = {"fezupel_us": round(t_moe * 1e6, 1), "qwen3_us": round(t_dense * 1e6, 1),
                               "fezupel_frac_of_read": round(mb / t_moe / read_bw, 4),
                               "qwen3_frac_of_read": round(db / t_dense / read_bw, 4)}
    else:
        out["feed_forward"] = {"fezupel_us": round(t_moe * 1e6, 1), "qwen3_us": round(t_dense * 1e6, 1),
                               "fezupel_frac_of_mfma": round(ff_flops / t_moe / mfma_rate, 4),
                               "qwen3_frac_of_mfma": round(ff_flops / t_dense / mfma_rate, 4)}
    # ---- norms: a layer norm that adds into the stream beside an RMS norm that stores
    x = torch.randn((rows, W), generator=g, device=dev)
    gain = torch.ones((W,), device=dev)
    bias = torch.zeros((W,), device=dev)
    normed = torch.empty((rows, W), dtype=bf, device=dev)
    t_ln = _timed(lambda: ops.norm_rows(x, gain, bias, 1e-6, normed, True))
    t_rms = _timed(lambda: ops.rmsnorm(x, gain, 1e-6, normed))
    out["norm"] = {"fezupel_us": round(t_ln * 1e6, 1), "qwen3_us": round(t_rms * 1e6, 1)}
    return out


def _moe_launcher(ops, h, router, ids, share, gate_up, down, res, top, ff):
    import torch
    rows = h.shape[0]
    y = torch.empty((rows, top, ff), dtype=h.dtype, device=h.device)

    def run():
        ops.moe_route(h, router, None, ids, share)
        ops.moe_experts(h, gate_up, down, ids, share, y, res, 7.0, 1.702, 1.0, add=False)
    return run


def main_fezupel(args) -> int:
    """Prefill and decode throughput of Fezupel shapes beside the dense Qwen3 decoder of equal
    size, and the new kernels alone beside the like kernels of that decoder."""
    import torch
    import zinfer_amd.ops as ops
    from zinfer_amd.config import entry_for
    T, batch, prompt = args.prefill_tokens, args.batch, args.prompt_len
    max_positions = max(T, prompt + args.steps + args.warmup + 64) + 64
    read_bw = ops.measure_read_bandwidth("cuda:0")
    mfma_rate = ops.measure_mfma_rate("cuda:0")
    names = [args.fezupel_shape] if args.fezupel_shape else list(FEZUPEL_SHAPES)
    shapes = {}
    for name in names:
        sh = FEZUPEL_SHAPES[name]
        row = {"sizes": sh}
        for label, raw in (("fezupel", fezupel_config(sh, max_positions)),
                           ("qwen3", dense_twin(sh, max_positions))):
            cfg = entry_for(raw).config_type.from_dict(raw)
            pool = batch * (prompt + args.steps + args.warmup + 64) + T + 256
            llm = build_llm(raw, args.dtype, args.seed, pool, max(batch, 8),
                            max_step_tokens=max(T, 2048), multi_step=args.multi_step)
            t_pre = run_prefill(llm, cfg, T, args.seed + 1)
            dt, mean_ctx = run_decode(llm, cfg, batch, prompt, args.steps, args.warmup, args.seed + 2)
            row[label] = {"prefill_tokens_per_s": round(T / t_pre, 1), "prefill_ms": round(t_pre * 1e3, 3),
                          "decode_tokens_per_s": round(batch * args.steps / dt, 1),
                          "decode_ms_per_step": round(dt / args.steps * 1e3, 4),
                          "decode_mean_context": round(mean_ctx, 1)}
            drop(llm)
        row["prefill_vs_qwen3"] = round(row["fezupel"]["prefill_tokens_per_s"]
                                        / row["qwen3"]["prefill_tokens_per_s"], 3)
        row["decode_vs_qwen3"] = round(row["fezupel"]["decode_tokens_per_s"]
                                       / row["qwen3"]["decode_tokens_per_s"], 3)
        if args.dtype == "bfloat16":
            row["kernels_prefill"] = fezupel_kernels(sh, T, T, mfma_rate, read_bw)
            row["kernels_decode"] = fezupel_kernels(sh, 1, prompt, mfma_rate, read_bw)
        ops._workspaces.clear()
        torch.cuda.empty_cache()
        shapes[name] = row
    first = shapes[names[0]]
    print(json.dumps({
        "metric": "fezupel_decode_tokens_per_s", "value": first["fezupel"]["decode_tokens_per_s"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": first["fezupel"]["decode_ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic", "config": {"model": f"Fezupel {names[0]} shape beside the dense Qwen3 "
                                                 "decoder of equal size, random weights",
                                        "batch": batch, "prompt_len": prompt, "prefill_tokens": T,
                                        "parallelism": "single GPU"},
        "measured_read_gbs": round(read_bw / 1e9, 1), "mfma_loop_tflops": round(mfma_rate / 1e12, 1),
        "shapes": shapes}))
    return 0



# --------------------------------------------------------------------------- Lodenex beside Qwen3
# Layer sizes that resemble served models; every shape is run beside the dense Qwen3 decoder of
# the same width, heads, head size, depth and vocabulary whose gated feed-forward does the same
# matrix work a token as the ungated one (three matrices of 2/3 the width instead of two).
LODENEX_SHAPES = {
    # grouped-query attention in chunks, values of their own
    "gqa": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=16384, layers=4, vocab=32768,
                mixers=("attention",) * 4, chunk=8192),
    # attention over a latent row of 128 + 64 numbers a token
    "latent": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=16384, layers=4, vocab=32768,
                   mixers=("latent_attention",) * 4, window=4096, q_rank=1536, kv_rank=128,
                   rot_dim=64),
    # three chunked layers to one latent layer
    "mixed": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=16384, layers=4, vocab=32768,
                  mixers=("attention", "attention", "latent_attention", "attention"), chunk=8192,
                  window=4096, q_rank=1536, kv_rank=128, rot_dim=64),
    # a latent of 512 + 64: wider than the MFMA attention kernels take (the 32-bit kernel runs)
    "latent-512": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=16384, layers=2, vocab=32768,
                       mixers=("latent_attention",) * 2, window=4096, q_rank=1536, kv_rank=512,
                       rot_dim=64),
}


def lodenex_config(sh: dict) -> dict:
    def layer(kind):
        if kind == "attention":
            mixer = {"heads": sh["heads"], "kv_heads": sh["kv_heads"], "dim": sh["dim"],
                     "vdim": sh["dim"], "scale": sh["dim"] ** -0.5, "softcap": 30.0,
                     "mask": {"size": sh["chunk"]},
                     "rot": {"base": 500000.0, "dims": sh["dim"] // 2,
                             "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
        else:
            mixer = {"heads": sh["heads"], "dim": sh["dim"], "rot_dim": sh["rot_dim"],
                     "vdim": sh["dim"], "q_rank": sh["q_rank"], "kv_rank": sh["kv_rank"],
                     "scale": (sh["dim"] + sh["rot_dim"]) ** -0.5, "mask": {"size": sh["window"]},
                     "rot": {"base": 1000000.0, "dims": sh["rot_dim"],
                             "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
        return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": sh["ff"]}}
    return {"architecture": "Lodenex", "vocab": sh["vocab"], "width": sh["width"],
            "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}, "logit_softcap": 30.0,
            "layers": [layer(k) for k in sh["mixers"]]}


def lodenex_twin(sh: dict, max_positions: int) -> dict:
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3",
                num_hidden_layers=sh["layers"], hidden_size=sh["width"],
                num_attention_heads=sh["heads"], num_key_value_heads=sh["kv_heads"],
                head_dim=sh["dim"], intermediate_size=sh["ff"] * 2 // 3 // 64 * 64,
                vocab_size=sh["vocab"], rope_theta=1000000.0, rms_norm_eps=1e-6,
                tie_word_embeddings=False, max_position_embeddings=max_positions,
                torch_dtype="bfloat16")


def _timed_graph(fn, inner: int = 10, repeats: int = 10) -> float:
    """Seconds of one call of ``fn`` on the device: ``inner`` calls are recorded into one graph
    (after two eager calls that settle work buffers) and the graph is replayed ``repeats`` times
    between two events, so that what the host spends on a launch does not count: a decode step's
    kernels run that way in the engine."""
    import torch
    fn()
    fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(inner):
            fn()
    graph.replay()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(repeats):
        graph.replay()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) * 1e-3 / (repeats * inner)


def lodenex_kernels(sh: dict, T: int, ctx: int, mfma_rate: float, read_bw: float) -> dict:
    """The new design's kernels alone beside the like kernels of the dense decoder, at ``T``
    tokens of one sequence that holds ``ctx`` tokens (T = ctx: a prompt; T = 1 x 8 sequences: a
    decode step), each with the fraction of its bound it reaches: matrix work against the MFMA
    loop's rate (prompt) or bytes that must be read against the measured read stream (decode)."""
    import torch
    import zinfer_amd.ops as ops
    dev = "cuda:0"
    W, nH, nKV, hd, ff = sh["width"], sh["heads"], sh["kv_heads"], sh["dim"], sh["ff"]
    bf = torch.bfloat16
    decode = T == 1
    n_seqs = 8 if decode else 1
    rows = n_seqs * T
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *shape: (torch.randn(shape, generator=g, device=dev) * 0.05).to(bf)
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)
    pages = (ctx + PAGE - 1) // PAGE
    table = torch.arange(n_seqs * pages, dtype=torch.int32, device=dev).view(n_seqs, pages)
    q_start = i32([i * T for i in range(n_seqs + 1)])
    ctx_len = i32([ctx] * n_seqs)
    seq_index = i32([i for i in range(n_seqs) for _ in range(T)])
    positions = i32([ctx - T + t for _ in range(n_seqs) for t in range(T)])
    slots = i32([(s * pages) * PAGE + ctx - T + t for s in range(n_seqs) for t in range(T)])
    bound = "frac_of_read" if decode else "frac_of_mfma"
    out = {}

    def row(name, t_new, t_old, work_new, work_old):
        rate = read_bw if decode else mfma_rate
        r = {"lodenex_us": round(t_new * 1e6, 1), "lodenex_" + bound: round(work_new / t_new / rate, 4)}
        if t_old is not None:
            r.update({"qwen3_us": round(t_old * 1e6, 1),
                      "qwen3_" + bound: round(work_old / t_old / rate, 4)})
        out[name] = r

    # ---- the dense decoder's attention at these heads
    q = rnd(rows, nH * hd)
    k_pool = rnd(n_seqs * pages, nKV * PAGE * hd)
    v_pool = rnd(n_seqs * pages, nKV * PAGE * hd)
    o = torch.empty((rows, nH * hd), dtype=bf, device=dev)
    t_old = _timed_graph(lambda: ops.paged_attention(q, k_pool, v_pool, table, q_start, ctx_len,
                                               seq_index, o, hd ** -0.5, 0, nH, nKV, hd, PAGE, T, ctx))
    pairs = n_seqs * (ctx if decode else T * (T + 1) // 2)
    old_work = n_seqs * ctx * nKV * 2 * hd * 2 if decode else 4.0 * pairs * hd * nH
    if "attention" in sh["mixers"]:
        gate = rnd(rows, nH)
        sink = torch.zeros((nH,), device=dev)
        t_new = _timed_graph(lambda: ops.attend_masked(q, gate, "head", k_pool, v_pool, sink, table, q_start,
                                                 ctx_len, seq_index, o, hd ** -0.5, 30.0, 0, sh["chunk"],
                                                 nH, nKV, hd, hd, PAGE, T, ctx))
        row("attention", t_new, t_old, old_work, old_work)
        # the projection's rows normed, rotated and stored, beside the dense decoder's kernel
        width = (nH + 2 * nKV) * hd
        proj = rnd(rows, width + nH)
        gq, gk = torch.ones((nH * hd,), device=dev), torch.ones((nKV * hd,), device=dev)
        freq = torch.rand((hd // 4,), generator=g, device=dev)
        segs = [ops.RowSegment(0, nH * hd, q, gain=gq, eps=1e-6, hd=hd, rot_dims=hd // 2, freq=freq),
                ops.RowSegment(nH * hd, nKV * hd, k_pool, gain=gk, eps=1e-6, hd=hd, rot_dims=hd // 2,
                               freq=freq, pool_heads=nKV),
                ops.RowSegment((nH + nKV) * hd, nKV * hd, v_pool, hd=hd, pool_heads=nKV)]
        t_new = _timed_graph(lambda: ops.project_rows(proj, positions, slots, PAGE, segs))
        qkv = rnd(rows, width)
        cos = torch.rand((ctx + 1, hd // 2), generator=g, device=dev)
        gh = torch.ones((hd,), device=dev)
        t_qk = _timed_graph(lambda: ops.qk_norm_rope_kv_write(qkv, gh, gh, 1e-6, cos, cos, positions, slots,
                                                        k_pool, v_pool, q, nH, nKV, hd, PAGE))
        out["norm_rotate_store"] = {"lodenex_us": round(t_new * 1e6, 1), "qwen3_us": round(t_qk * 1e6, 1)}
    if "latent_attention" in sh["mixers"]:
        rank, dr = sh["kv_rank"], sh["rot_dim"]
        KW = rank + dr
        qa = rnd(rows, nH * KW)
        lat_pool = rnd(n_seqs * pages, PAGE * KW)
        mixed = torch.empty((rows, nH * rank), dtype=bf, device=dev)
        seen = min(ctx, sh["window"])
        t_new = _timed_graph(lambda: ops.attend_masked(qa, None, None, lat_pool, None, None, table, q_start,
                                                 ctx_len, seq_index, mixed, KW ** -0.5, 0.0,
                                                 sh["window"], 0, nH, 1, KW, rank, PAGE, T, ctx))
        new_work = n_seqs * seen * KW * 2 if decode else 2.0 * pairs * (KW + rank) * nH
        row("latent_attention", t_new, t_old, new_work, old_work)
        # the two products a head around it
        qfull = rnd(rows, nH * (hd + dr))
        uk_t, uv = rnd(nH, rank, hd), rnd(nH, hd, rank)
        attn = torch.empty((rows, nH * hd), dtype=bf, device=dev)
        gate_e = rnd(rows, nH * hd)

        def around():
            ops.head_products(qfull, 0, hd + dr, uk_t, None, qa, 0, KW)
            ops.head_products(mixed, 0, rank, uv, gate_e, attn, 0, hd)
        t_hp = _timed_graph(around)
        work = 2 * nH * rank * hd * 2 if decode else 2.0 * rows * 2 * nH * rank * hd
        row("head_products", t_hp, None, work, None)
    # ---- feed-forward: two matrices and an activation beside three of 2/3 the width
    h = rnd(rows, W)
    w_up, w_down = ops.pretile_weight(rnd(ff, W)), ops.pretile_weight(rnd(W, ff))
    act = torch.empty((rows, ff), dtype=bf, device=dev)
    branch = torch.zeros((rows, W), dtype=torch.float32, device=dev)

    def plain_ff():
        ops.gemm(h, w_up, act, w_tiled=True)
        ops.activation(act, act, "gelu")
        ops.gemm(act, w_down, branch, w_tiled=True)
    t_new = _timed_graph(plain_ff)
    inter = ff * 2 // 3 // 64 * 64
    wgu = ops.pretile_weight(ops.interleave_gate_up(rnd(inter, W), rnd(inter, W)))
    wd = ops.pretile_weight(rnd(W, inter))
    act2 = torch.empty((rows, inter), dtype=bf, device=dev)

    def gated_ff():
        ops.gemm_swiglu(h, wgu, act2, w_tiled=True)
        ops.gemm(act2, wd, branch, accumulate=True, w_tiled=True)
    t_old = _timed_graph(gated_ff)
    if decode:
        row("feed_forward", t_new, t_old, 2 * ff * W * 2, 3 * inter * W * 2)
    else:
        row("feed_forward", t_new, t_old, 2.0 * rows * 2 * ff * W, 2.0 * rows * 3 * inter * W)
    # ---- the norm behind a sublayer (adds, leaves the sum for the next product) beside an RMS
    # norm that stores
    x = torch.randn((rows, W), generator=g, device=dev)
    gain = torch.ones((W,), device=dev)
    normed = torch.empty((rows, W), dtype=bf, device=dev)
    t_ln = _timed_graph(lambda: ops.norm_add_store(branch, gain, None, 1e-6, False, x, normed))
    t_rms = _timed_graph(lambda: ops.rmsnorm(x, gain, 1e-6, normed))
    out["norm"] = {"lodenex_us": round(t_ln * 1e6, 1), "qwen3_us": round(t_rms * 1e6, 1)}
    return out


def main_lodenex(args) -> int:
    """Prefill and decode throughput of Lodenex shapes beside the dense Qwen3 decoder of equal
    size, and the new kernels alone beside the like kernels of that decoder."""
    import torch
    import zinfer_amd.ops as ops
    from zinfer_amd.config import entry_for
    T, batch, prompt = args.prefill_tokens, args.batch, args.prompt_len
    max_positions = max(T, prompt + args.steps + args.warmup + 64) + 64
    read_bw = ops.measure_read_bandwidth("cuda:0")
    mfma_rate = ops.measure_mfma_rate("cuda:0")
    names = [args.lodenex_shape] if args.lodenex_shape else ["gqa", "latent", "mixed"]
    shapes = {}
    for name in names:
        sh = LODENEX_SHAPES[name]
        row = {"sizes": {k: (list(v) if isinstance(v, tuple) else v) for k, v in sh.items()}}
        for label, raw in (("lodenex", lodenex_config(sh)), ("qwen3", lodenex_twin(sh, max_positions))):
            cfg = entry_for(raw).config_type.from_dict(raw)
            pool = batch * (prompt + args.steps + args.warmup + 64) + T + 256
            llm = build_llm(raw, args.dtype, args.seed, pool, max(batch, 8),
                            max_step_tokens=max(T, 2048), multi_step=args.multi_step)
            t_pre = run_prefill(llm, cfg, T, args.seed + 1)
            dt, mean_ctx = run_decode(llm, cfg, batch, prompt, args.steps, args.warmup, args.seed + 2)
            row[label] = {"prefill_tokens_per_s": round(T / t_pre, 1), "prefill_ms": round(t_pre * 1e3, 3),
                          "decode_tokens_per_s": round(batch * args.steps / dt, 1),
                          "decode_ms_per_step": round(dt / args.steps * 1e3, 4),
                          "decode_mean_context": round(mean_ctx, 1)}
            drop(llm)
        row["prefill_vs_qwen3"] = round(row["lodenex"]["prefill_tokens_per_s"]
                                        / row["qwen3"]["prefill_tokens_per_s"], 3)
        row["decode_vs_qwen3"] = round(row["lodenex"]["decode_tokens_per_s"]
                                       / row["qwen3"]["decode_tokens_per_s"], 3)
        if args.dtype == "bfloat16":
            row["kernels_prefill"] = lodenex_kernels(sh, T, T, mfma_rate, read_bw)
            row["kernels_decode"] = lodenex_kernels(sh, 1, prompt, mfma_rate, read_bw)
        ops._workspaces.clear()
        torch.cuda.empty_cache()
        shapes[name] = row
    first = shapes[names[0]]
    print(json.dumps({
        "metric": "lodenex_decode_tokens_per_s", "value": first["lodenex"]["decode_tokens_per_s"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": first["lodenex"]["decode_ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic", "config": {"model": f"Lodenex {names[0]} shape beside the dense Qwen3 "
                                                 "decoder of equal size, random weights",
                                        "batch": batch, "prompt_len": prompt, "prefill_tokens": T,
                                        "parallelism": "single GPU"},
        "measured_read_gbs": round(read_bw / 1e9, 1), "mfma_loop_tflops": round(mfma_rate / 1e12, 1),
        "shapes": shapes}))
    return 0


# --------------------------------------------------------------------------- Nupovik beside Qwen3
# Layer sizes that resemble served models with recurrent mixers; every shape is run beside the
# dense Qwen3 decoder of the same width, depth and vocabulary, with heads of 128, whose gated
# feed-forward does the matrix work a token of the new design's feed-forwards (a mixture counts
# the experts a token uses).
def _np_moe(experts, top, ff, groups):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top,
                       "groups": {"count": groups[0], "keep": groups[1]}}}


NUPOVIK_SHAPES = {
    # recurrent layers alone: token-shift layers with heads of 64, gated linear attention with
    # keys half as wide as the values
    "recurrent": dict(width=2048, vocab=32768, loop=None, layers=[
        ("wkv", dict(heads=32, dim=64), {"kind": "dense", "ff": 7168}),
        ("gla", dict(heads=8, dim=128, vdim=256, tau=16.0), {"kind": "dense", "ff": 7168}),
        ("wkv", dict(heads=32, dim=64), {"kind": "dense", "ff": 7168}),
        ("gla", dict(heads=8, dim=128, vdim=256, tau=16.0), {"kind": "dense", "ff": 7168})]),
    # all three mixers, a mixture of 32 experts in 8 groups, the first two layers run twice
    "hybrid": dict(width=4096, vocab=32768, loop=dict(start=0, stop=2, times=2), layers=[
        ("gla", dict(heads=16, dim=128, vdim=256, tau=16.0), {"kind": "dense", "ff": 12288}),
        ("latent_attention", dict(heads=32, dim=128, vdim=128, kv_rank=128, scale=128 ** -0.5),
         _np_moe(32, 4, 2048, (8, 4))),
        ("wkv", dict(heads=64, dim=64), _np_moe(32, 4, 2048, (8, 4))),
        ("latent_attention", dict(heads=32, dim=128, vdim=128, kv_rank=128, scale=128 ** -0.5),
         {"kind": "dense", "ff": 12288})]),
}


def nupovik_config(sh: dict) -> dict:
    return {"architecture": "Nupovik", "vocab": sh["vocab"], "width": sh["width"],
            "norm": {"eps": 1e-6}, "logit_scale": 1.0, "loop": sh["loop"],
            "layers": [{"type": kind, "mixer": dict(mixer), "mlp": mlp}
                       for kind, mixer, mlp in sh["layers"]]}


def nupovik_runs(sh: dict) -> list:
    """The layers in the order they run, a repeated one once a pass."""
    n = len(sh["layers"])
    if sh["loop"] is None:
        return list(range(n))
    a, b, times = sh["loop"]["start"], sh["loop"]["stop"], sh["loop"]["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def nupovik_twin(sh: dict, max_positions: int) -> dict:
    runs = nupovik_runs(sh)
    used = [m["ff"] if m["kind"] == "dense" else m["router"]["top"] * m["expert"]["ff"]
            for m in (sh["layers"][i][2] for i in runs)]
    inter = int(sum(used) / len(used)) * 2 // 3 // 64 * 64
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3",
                num_hidden_layers=len(runs), hidden_size=sh["width"],
                num_attention_heads=sh["width"] // 128, num_key_value_heads=8, head_dim=128,
                intermediate_size=inter, vocab_size=sh["vocab"], rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=False,
                max_position_embeddings=max_positions, torch_dtype="bfloat16")


def nupovik_kernels(sh: dict, T: int, ctx: int, mfma_rate: float, read_bw: float) -> dict:
    """The new design's kernels alone beside the like kernels of the dense decoder, at ``T``
    tokens of one sequence that holds ``ctx`` tokens (T = ctx: a prompt; T = 1 x 8 sequences: a
    decode step).  Each has the fraction of its bound it reaches.  Matrix work: the MFMA loop's
    rate (prompt) or the bytes that must be read against the measured read stream (decode).
    The recurrence is 32-bit vector work, five operations a state element a token (prompt:
    against the published 32-bit vector rate), or its state read and written once (decode)."""
    import torch
    import zinfer_amd.ops as ops
    dev = "cuda:0"
    W = sh["width"]
    nH, nKV, hd = W // 128, 8, 128
    bf = torch.bfloat16
    decode = T == 1
    n_seqs = 8 if decode else 1
    rows = n_seqs * T
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *shape: (torch.randn(shape, generator=g, device=dev) * 0.05).to(bf)
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)
    pages = (ctx + PAGE - 1) // PAGE
    table = torch.arange(n_seqs * pages, dtype=torch.int32, device=dev).view(n_seqs, pages)
    q_start = i32([i * T for i in range(n_seqs + 1)])
    ctx_len = i32([ctx] * n_seqs)
    seq_index = i32([i for i in range(n_seqs) for _ in range(T)])
    state_slots = i32(list(range(n_seqs)))
    out = {}

    def row(name, t_new, work_new, rate_new, bound_new, t_old=None, work_old=None, rate_old=None,
            bound_old=None):
        r = {"nupovik_us": round(t_new * 1e6, 1),
             "nupovik_frac_of_" + bound_new: round(work_new / t_new / rate_new, 4)}
        if t_old is not None:
            r.update({"qwen3_us": round(t_old * 1e6, 1),
                      "qwen3_frac_of_" + bound_old: round(work_old / t_old / rate_old, 4)})
        out[name] = r

    mat_bound, mat_rate = ("read", read_bw) if decode else ("mfma", mfma_rate)
    # ---- the dense decoder's attention at the twin's heads
    q = rnd(rows, nH * hd)
    k_pool = rnd(n_seqs * pages, nKV * PAGE * hd)
    v_pool = rnd(n_seqs * pages, nKV * PAGE * hd)
    o = torch.empty((rows, nH * hd), dtype=bf, device=dev)
    t_att = _timed_graph(lambda: ops.paged_attention(q, k_pool, v_pool, table, q_start, ctx_len,
                                                     seq_index, o, hd ** -0.5, 0, nH, nKV, hd,
                                                     PAGE, T, ctx))
    pairs = n_seqs * (ctx if decode else T * (T + 1) // 2)
    att_work = n_seqs * ctx * nKV * 2 * hd * 2 if decode else 4.0 * pairs * hd * nH
    seen = set()
    for kind, m, _ in sh["layers"]:
        if kind in seen:
            continue
        seen.add(kind)
        if kind == "latent_attention":
            H, rank, vdim = m["heads"], m["kv_rank"], m["vdim"]
            qa = rnd(rows, H * rank)
            gate = rnd(rows, H)
            lat_pool = rnd(n_seqs * pages, PAGE * rank)
            mixed = torch.empty((rows, H * rank), dtype=bf, device=dev)
            t_new = _timed_graph(lambda: ops.attend_masked(
                qa, gate, "head", lat_pool, None, None, table, q_start, ctx_len, seq_index, mixed,
                m["scale"], 0.0, 0, 0, H, 1, rank, rank, PAGE, T, ctx))
            new_work = n_seqs * ctx * rank * 2 if decode else 4.0 * pairs * rank * H
            row("latent_attention", t_new, new_work, mat_rate, mat_bound, t_att, att_work,
                mat_rate, mat_bound)
            qfull = rnd(rows, H * m["dim"])
            uk_t, uv = rnd(H, rank, m["dim"]), rnd(H, vdim, rank)
            attn = torch.empty((rows, H * vdim), dtype=bf, device=dev)

            def around():
                ops.head_products(qfull, 0, m["dim"], uk_t, None, qa, 0, rank)
                ops.head_products(mixed, 0, rank, uv, None, attn, 0, vdim)
            t_hp = _timed_graph(around)
            work = H * rank * (m["dim"] + vdim) * 2 if decode \
                else 2.0 * rows * H * rank * (m["dim"] + vdim)
            row("head_products", t_hp, work, mat_rate, mat_bound)
            continue
        H, d = m["heads"], m["dim"]
        dv = m.get("vdim", d)
        size = ops.recurrence_state_size(H, d, dv)
        state = torch.zeros((n_seqs, size + W), dtype=torch.float32, device=dev)
        qk = rnd(2, rows, H * d)
        v = rnd(rows, H * dv)
        z = torch.randn((rows, H * d), generator=g, device=dev)
        zb = torch.zeros((H * d,), device=dev)
        bonus = torch.rand((H * d,), generator=g, device=dev) if kind == "wkv" else None
        ro = torch.empty((rows, H * dv), dtype=torch.float32, device=dev)
        rule = "double_exp" if kind == "wkv" else "sigmoid_root"
        t_new = _timed_graph(lambda: ops.decay_recurrence(
            qk[0], qk[1], v, z, zb, bonus, state, state_slots, q_start, ro, H, d, dv, rule,
            tau=float(m.get("tau", 1.0)), q_scale=d ** -0.5, max_q_len=T))
        if decode:
            row(kind + "_recurrence", t_new, 2.0 * n_seqs * H * d * dv * 4, read_bw, "read",
                t_att, att_work, read_bw, "read")
        else:
            row(kind + "_recurrence", t_new, 5.0 * rows * H * d * dv, PEAK_FLOPS["fp32"],
                "fp32_vector", t_att, att_work, mfma_rate, "mfma")
        gate = rnd(rows, H * dv)
        gain = torch.ones((dv if kind == "gla" else H * dv,), device=dev)
        mixed = torch.empty((rows, H * dv), dtype=bf, device=dev)
        t_norm = _timed_graph(lambda: ops.head_norm_gate(ro, gain, gate, mixed, H, 1e-6))
        row(kind + "_head_norm_gate", t_norm, rows * H * dv * (4 + 2 + 2), read_bw, "read")
        if kind == "wkv":
            h = rnd(rows, W)
            mu = torch.rand((5, W), generator=g, device=dev)
            mixes = torch.empty((5, rows, W), dtype=bf, device=dev)
            t_mix = _timed_graph(lambda: ops.token_shift_mix(h, mu, state, size, state_slots,
                                                             seq_index, q_start, mixes))
            row("token_shift_mix", t_mix, rows * W * 2 * (1 + 5), read_bw, "read")
    # ---- feed-forwards: two matrices around a squared relu beside three of 2/3 the width
    h = rnd(rows, W)
    branch = torch.zeros((rows, W), dtype=torch.float32, device=dev)
    dense = next((f for _, _, f in sh["layers"] if f["kind"] == "dense"), None)
    moe = next((f for _, _, f in sh["layers"] if f["kind"] == "moe"), None)

    def gated_twin(inter):
        wgu = ops.pretile_weight(ops.interleave_gate_up(rnd(inter, W), rnd(inter, W)))
        wd = ops.pretile_weight(rnd(W, inter))
        act2 = torch.empty((rows, inter), dtype=bf, device=dev)

        def run():
            ops.gemm_swiglu(h, wgu, act2, w_tiled=True)
            ops.gemm(act2, wd, branch, accumulate=True, w_tiled=True)
        return _timed_graph(run)
    if dense is not None:
        ff = dense["ff"]
        w_up, w_down = ops.pretile_weight(rnd(ff, W)), ops.pretile_weight(rnd(W, ff))
        act = torch.empty((rows, ff), dtype=bf, device=dev)

        def plain_ff():
            ops.gemm(h, w_up, act, w_tiled=True)
            ops.activation(act, act, "relu2")
            ops.gemm(act, w_down, branch, accumulate=True, w_tiled=True)
        t_new = _timed_graph(plain_ff)
        inter = ff * 2 // 3 // 64 * 64
        t_old = gated_twin(inter)
        if decode:
            row("feed_forward", t_new, 2 * ff * W * 2, read_bw, "read", t_old, 3 * inter * W * 2,
                read_bw, "read")
        else:
            row("feed_forward", t_new, 2.0 * rows * 2 * ff * W, mfma_rate, "mfma", t_old,
                2.0 * rows * 3 * inter * W, mfma_rate, "mfma")
    if moe is not None:
        E, top, ff = moe["router"]["experts"], moe["router"]["top"], moe["expert"]["ff"]
        groups = (moe["router"]["groups"]["count"], moe["router"]["groups"]["keep"])
        router = torch.randn((E, W), generator=g, device=dev) * 0.05
        correction = torch.randn((E,), generator=g, device=dev) * 0.1
        ids = torch.empty((rows, top), dtype=torch.int32, device=dev)
        share = torch.empty((rows, top), dtype=torch.float32, device=dev)
        up, down = rnd(E, ff, W), rnd(E, W, ff)
        y = torch.empty((rows, top, ff), dtype=bf, device=dev)

        def mixture():
            ops.moe_route(h, router, None, ids, share, scoring="sigmoid", correction=correction,
                          groups=groups)
            ops.moe_experts(h, up, down, ids, share, y, branch, 0.0, 1.0, 0.0, add=True,
                            act="relu2")
        t_new = _timed_graph(mixture)
        inter = top * ff * 2 // 3 // 64 * 64
        t_old = gated_twin(inter)
        if decode:
            used = min(E, rows * top)        # at most this many experts' matrices are read
            row("mixture", t_new, used * 2 * ff * W * 2, read_bw, "read", t_old,
                3 * inter * W * 2, read_bw, "read")
        else:
            row("mixture", t_new, 2.0 * rows * 2 * top * ff * W, mfma_rate, "mfma", t_old,
                2.0 * rows * 3 * inter * W, mfma_rate, "mfma")
    return out


def main_nupovik(args) -> int:
    """Prefill and decode throughput of Nupovik shapes beside the dense Qwen3 decoder of equal
    size, and the new kernels alone beside the like kernels of that decoder."""
    import torch
    import zinfer_amd.ops as ops
    from zinfer_amd.config import entry_for
    T, batch, prompt = args.prefill_tokens, args.batch, args.prompt_len
    max_positions = max(T, prompt + args.steps + args.warmup + 64) + 64
    read_bw = ops.measure_read_bandwidth("cuda:0")
    mfma_rate = ops.measure_mfma_rate("cuda:0")
    names = [args.nupovik_shape] if args.nupovik_shape else list(NUPOVIK_SHAPES)
    shapes = {}
    for name in names:
        sh = NUPOVIK_SHAPES[name]
        row = {"sizes": {"width": sh["width"], "vocab": sh["vocab"], "loop": sh["loop"],
                         "layers": [[k, m, f] for k, m, f in sh["layers"]]}}
        for label, raw in (("nupovik", nupovik_config(sh)), ("qwen3", nupovik_twin(sh, max_positions))):
            cfg = entry_for(raw).config_type.from_dict(raw)
            pool = batch * (prompt + args.steps + args.warmup + 64) + T + 256
            llm = build_llm(raw, args.dtype, args.seed, pool, max(batch, 8),
                            max_step_tokens=max(T, 2048), multi_step=args.multi_step)
            t_pre = run_prefill(llm, cfg, T, args.seed + 1)
            dt, mean_ctx = run_decode(llm, cfg, batch, prompt, args.steps, args.warmup, args.seed + 2)
            row[label] = {"prefill_tokens_per_s": round(T / t_pre, 1), "prefill_ms": round(t_pre * 1e3, 3),
                          "decode_tokens_per_s": round(batch * args.steps / dt, 1),
                          "decode_ms_per_step": round(dt / args.steps * 1e3, 4),
                          "decode_mean_context": round(mean_ctx, 1)}
            drop(llm)
        row["prefill_vs_qwen3"] = round(row["nupovik"]["prefill_tokens_per_s"]
                                        / row["qwen3"]["prefill_tokens_per_s"], 3)
        row["decode_vs_qwen3"] = round(row["nupovik"]["decode_tokens_per_s"]
                                       / row["qwen3"]["decode_tokens_per_s"], 3)
        if args.dtype == "bfloat16":
            row["kernels_prefill"] = nupovik_kernels(sh, T, T, mfma_rate, read_bw)
            row["kernels_decode"] = nupovik_kernels(sh, 1, prompt, mfma_rate, read_bw)
        ops._workspaces.clear()
        torch.cuda.empty_cache()
        shapes[name] = row
    first = shapes[names[0]]
    print(json.dumps({
        "metric": "nupovik_decode_tokens_per_s", "value": first["nupovik"]["decode_tokens_per_s"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": first["nupovik"]["decode_ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic", "config": {"model": f"Nupovik {names[0]} shape beside the dense Qwen3 "
                                                 "decoder of equal size, random weights",
                                        "batch": batch, "prompt_len": prompt, "prefill_tokens": T,
                                        "parallelism": "single GPU"},
        "measured_read_gbs": round(read_bw / 1e9, 1), "mfma_loop_tflops": round(mfma_rate / 1e12, 1),
        "shapes": shapes}))
    return 0

# --------------------------------------------------------------------------- Kugisun beside Qwen3
# Layer sizes that resemble served models of this kind: a stream in four copies, attention heads
# of 128 beside delta-rule heads of 128 x 128, a gated feed-forward or a mixture with outputs
# that hand their input on and a shared expert.  Every shape is run beside the dense Qwen3
# decoder of the same width, depth and vocabulary whose attention has the left mixer's heads and
# whose gated feed-forward does the matrix work a token of the new design's feed-forwards; the
# new kernels alone stand beside the like kernels of that decoder and of Nupovik, the closest
# design with a recurrence (its gated linear attention at the same heads).
def _kg_moe(experts, identity, top, ff, groups, shared):
    return {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": shared},
            "router": {"experts": experts, "identity": identity, "top": top, "scale": 2.5,
                       "groups": {"count": groups[0], "keep": groups[1]}}}


def _kg_mixer(heads, kv, r_heads, r_kv):
    return {"left": {"heads": heads, "kv_heads": kv, "dim": 128, "vdim": 128,
                     "scale": 128 ** -0.5, "rot": {"dims": 64, "base": 1000000.0}},
            "right": {"heads": r_heads, "kv_heads": r_kv, "dim": 128, "vdim": 128, "conv": 4},
            "left_scale": 0.75, "right_scale": 1.25}


KUGISUN_SHAPES = {
    "medium": dict(width=2048, vocab=32768, streams=4, mixer=_kg_mixer(16, 4, 16, 8),
                   mlps=[{"kind": "dense", "ff": 5632}, _kg_moe(30, 2, 4, 1024, (8, 4), 1536)],
                   order=[0, 1, 1, 1]),
    "wide": dict(width=4096, vocab=32768, streams=4, mixer=_kg_mixer(32, 8, 32, 16),
                 mlps=[{"kind": "dense", "ff": 11264}, _kg_moe(62, 2, 6, 1536, (8, 4), 2048)],
                 order=[0, 1, 0, 1]),
}


def kugisun_config(sh: dict, max_positions: int) -> dict:
    layers, first = [], {}
    for i, j in enumerate(sh["order"]):
        L = {"type": "parallel", "mixer": sh["mixer"], "mlp": sh["mlps"][j]}
        if j in first:
            L["weights_of"] = first[j]
        first.setdefault(j, i)
        layers.append(L)
    return {"architecture": "Kugisun", "vocab": sh["vocab"], "width": sh["width"],
            "max_positions": max_positions, "streams": sh["streams"], "norm": {"eps": 1e-6},
            "layers": layers}


def _kg_used(mlp: dict) -> int:
    return mlp["ff"] if mlp["kind"] == "dense" \
        else mlp["router"]["top"] * mlp["expert"]["ff"] + mlp["shared"]["ff"]


def kugisun_twin(sh: dict, max_positions: int) -> dict:
    used = [_kg_used(sh["mlps"][j]) for j in sh["order"]]
    left = sh["mixer"]["left"]
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3",
                num_hidden_layers=len(sh["order"]), hidden_size=sh["width"],
                num_attention_heads=left["heads"], num_key_value_heads=left["kv_heads"],
                head_dim=128, intermediate_size=int(sum(used) / len(used)) // 64 * 64,
                vocab_size=sh["vocab"], rope_theta=1000000.0, rms_norm_eps=1e-6,
                tie_word_embeddings=True, max_position_embeddings=max_positions,
                torch_dtype="bfloat16")


def kugisun_kernels(sh: dict, T: int, ctx: int, mfma_rate: float, read_bw: float) -> dict:
    """The new design's kernels alone beside the like kernels of the dense decoder and of
    Nupovik, at ``T`` tokens of one sequence that holds ``ctx`` tokens (T = ctx: a prompt;
    T = 1 x 8 sequences: a decode step), each with the fraction of its bound it reaches: matrix
    work against the MFMA loop's rate (prompt) or the bytes that must be read against the
    measured read stream (decode); the recurrences are 32-bit vector work (the delta rule six
    operations a state element a token, the decayed sum five) against the published 32-bit
    vector rate, or their state read and written once (decode)."""
    import torch
    import zinfer_amd.ops as ops
    dev = "cuda:0"
    W, S = sh["width"], sh["streams"]
    left, right = sh["mixer"]["left"], sh["mixer"]["right"]
    bf = torch.bfloat16
    decode = T == 1
    n_seqs = 8 if decode else 1
    rows = n_seqs * T
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *shape: (torch.randn(shape, generator=g, device=dev) * 0.05).to(bf)
    rnd32 = lambda *shape: torch.randn(shape, generator=g, device=dev) * 0.05
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)
    pages = (ctx + PAGE - 1) // PAGE
    table = torch.arange(n_seqs * pages, dtype=torch.int32, device=dev).view(n_seqs, pages)
    q_start = i32([i * T for i in range(n_seqs + 1)])
    ctx_len = i32([ctx] * n_seqs)
    seq_index = i32([i for i in range(n_seqs) for _ in range(T)])
    positions = i32([ctx - T + i for _ in range(n_seqs) for i in range(T)])
    slot_mapping = i32([s * pages * PAGE + ctx - T + i for s in range(n_seqs) for i in range(T)])
    state_slots = i32(list(range(n_seqs)))
    out = {}

    def row(name, t_new, work_new, rate_new, bound_new, like=None, t_old=None, work_old=None,
            rate_old=None, bound_old=None):
        r = {"kugisun_us": round(t_new * 1e6, 1),
             "kugisun_frac_of_" + bound_new: round(work_new / t_new / rate_new, 4)}
        if t_old is not None:
            r.update({"like": like, "like_us": round(t_old * 1e6, 1),
                      "like_frac_of_" + bound_old: round(work_old / t_old / rate_old, 4)})
        out[name] = r

    mat_bound, mat_rate = ("read", read_bw) if decode else ("mfma", mfma_rate)
    # ---- attention: the masked kernels at the left mixer's heads beside the dense decoder's
    nH, nKV, hd = left["heads"], left["kv_heads"], 128
    q = rnd(rows, nH * hd)
    k_pool = rnd(n_seqs * pages, nKV * PAGE * hd)
    v_pool = rnd(n_seqs * pages, nKV * PAGE * hd)
    o = torch.empty((rows, nH * hd), dtype=bf, device=dev)
    t_old = _timed_graph(lambda: ops.paged_attention(q, k_pool, v_pool, table, q_start, ctx_len,
                                                     seq_index, o, hd ** -0.5, 0, nH, nKV, hd,
                                                     PAGE, T, ctx))
    t_new = _timed_graph(lambda: ops.attend_masked(q, None, None, k_pool, v_pool, None, table,
                                                   q_start, ctx_len, seq_index, o, hd ** -0.5, 0.0,
                                                   0, 0, nH, nKV, hd, hd, PAGE, T, ctx))
    pairs = n_seqs * (ctx if decode else T * (T + 1) // 2)
    att_work = n_seqs * ctx * nKV * 2 * hd * 2 if decode else 4.0 * pairs * hd * nH
    row("attention", t_new, att_work, mat_rate, mat_bound, "qwen3 attention", t_old, att_work,
        mat_rate, mat_bound)
    # ---- bias, norm a head, rotation, cache write beside the dense decoder's kernel
    qkv = rnd(rows, (nH + 2 * nKV) * hd)
    bias = rnd32((nH + 2 * nKV) * hd)
    gq, gk = torch.ones(hd, device=dev), torch.ones(hd, device=dev)
    freq = torch.tensor([1000000.0 ** (-2.0 * i / 64) for i in range(32)], device=dev)
    qw, kw = nH * hd, nKV * hd
    segs = [ops.RowSegment(0, qw, o, gain=gq, eps=1e-6, hd=hd, bias=bias[:qw].contiguous(),
                           per_head=True, rot_dims=64, freq=freq, interleaved=True),
            ops.RowSegment(qw, kw, k_pool, gain=gk, eps=1e-6, hd=hd, pool_heads=nKV,
                           bias=bias[qw:qw + kw].contiguous(), per_head=True, rot_dims=64,
                           freq=freq, interleaved=True),
            ops.RowSegment(qw + kw, kw, v_pool, hd=hd, pool_heads=nKV,
                           bias=bias[qw + kw:].contiguous())]
    t_new = _timed_graph(lambda: ops.project_rows(qkv, positions, slot_mapping, PAGE, segs))
    cos = torch.ones((ctx + 1, hd // 2), device=dev)
    sin = torch.zeros((ctx + 1, hd // 2), device=dev)
    kp2 = torch.empty_like(k_pool)
    vp2 = torch.empty_like(v_pool)
    t_old = _timed_graph(lambda: ops.qk_norm_rope_kv_write(qkv, gq, gk, 1e-6, cos, sin, positions,
                                                           slot_mapping, kp2, vp2, o, nH, nKV, hd,
                                                           PAGE))
    rw = rows * (nH + 2 * nKV) * hd * 2 * 2
    row("norm_rotate_write", t_new, rw, read_bw, "read", "qwen3 norm, rotation, cache write",
        t_old, rw, read_bw, "read")
    # ---- the delta rule beside Nupovik's decayed sum at the same heads
    H, KH, d, dv, taps = right["heads"], right["kv_heads"], right["dim"], right["vdim"], right["conv"]
    C = 2 * KH * d + H * dv
    msize = (ops.delta_state_size(H, d, dv) + 3) // 4 * 4
    state = torch.zeros((n_seqs, msize + (taps - 1) * C), dtype=torch.float32, device=dev)
    f32qkv = rnd32(rows, C)
    f32qkv[:, :2 * KH * d] = torch.nn.functional.normalize(
        f32qkv[:, :2 * KH * d].view(rows, 2 * KH, d), dim=-1).view(rows, -1)
    ab = torch.randn((rows, 2 * H), generator=g, device=dev)
    a_log, dtb = torch.zeros(H, device=dev) - 3.0, torch.zeros(H, device=dev)
    ro = torch.empty((rows, H * dv), dtype=torch.float32, device=dev)
    t_new = _timed_graph(lambda: ops.delta_recurrence(f32qkv, 0, KH * d, 2 * KH * d, ab, a_log,
                                                      dtb, state, state_slots, q_start, ro, H, KH,
                                                      d, dv))
    size = ops.recurrence_state_size(H, d, dv)
    st2 = torch.zeros((n_seqs, size), dtype=torch.float32, device=dev)
    qk = rnd(2, rows, H * d)
    v = rnd(rows, H * dv)
    z = torch.randn((rows, H * d), generator=g, device=dev)
    zb = torch.zeros((H * d,), device=dev)
    t_old = _timed_graph(lambda: ops.decay_recurrence(qk[0], qk[1], v, z, zb, None, st2,
                                                      state_slots, q_start, ro, H, d, dv,
                                                      "sigmoid_root", tau=16.0, q_scale=d ** -0.5,
                                                      max_q_len=T))
    if decode:
        sb = 2.0 * n_seqs * H * d * dv * 4
        row("delta_recurrence", t_new, sb, read_bw, "read", "nupovik decayed sum", t_old, sb,
            read_bw, "read")
    else:
        row("delta_recurrence", t_new, 6.0 * rows * H * d * dv, PEAK_FLOPS["fp32"], "fp32_vector",
            "nupovik decayed sum", t_old, 5.0 * rows * H * d * dv, PEAK_FLOPS["fp32"],
            "fp32_vector")
    # ---- short convolutions beside Nupovik's token shift (both read rows and a kept row)
    proj = rnd(rows, C + H * dv)
    tapw = torch.randn((C, taps), generator=g, device=dev)
    cout = torch.empty((rows, C), dtype=torch.float32, device=dev)
    t_new = _timed_graph(lambda: ops.short_conv(proj, tapw, state, msize, state_slots, seq_index,
                                                q_start, cout, unit_heads=2 * KH, head_dim=d,
                                                scaled_heads=KH, scale=d ** -0.5, unit_eps=1e-6,
                                                single_tokens=decode))
    hrow = rnd(rows, W)
    mu = torch.rand((5, W), generator=g, device=dev)
    mixes = torch.empty((5, rows, W), dtype=bf, device=dev)
    st3 = torch.zeros((n_seqs, W), dtype=torch.float32, device=dev)
    t_old = _timed_graph(lambda: ops.token_shift_mix(hrow, mu, st3, 0, state_slots, seq_index,
                                                     q_start, mixes))
    row("short_conv", t_new, rows * C * (2 + 4), read_bw, "read", "nupovik token shift", t_old,
        rows * W * 2 * (1 + 5), read_bw, "read")
    gate = rnd(rows, H * dv)
    gain = torch.ones((dv,), device=dev)
    mixed = torch.empty((rows, H * dv), dtype=bf, device=dev)
    t_norm = _timed_graph(lambda: ops.head_norm_gate(ro, gain, gate, mixed, H, 1e-6))
    row("head_norm_gate", t_norm, rows * H * dv * (4 + 2 + 2), read_bw, "read")
    # ---- the copies: write and read in one launch beside the dense decoder's norm
    x = torch.randn((S, rows, W), generator=g, device=dev)
    y0, y1 = rnd32(rows, W), rnd32(rows, W)
    M = torch.eye(S, device=dev) + 0.1 * torch.randn((S, S), generator=g, device=dev)
    bco, aco = torch.ones(S, device=dev), torch.ones(S, device=dev) / S
    gw = torch.ones(W, device=dev)
    hout = torch.empty((rows, W), dtype=bf, device=dev)
    t_new = _timed_graph(lambda: ops.streams_step(x, [(y0, 0.75), (y1, 1.0)], M, bco, read=True,
                                                  in_coef=aco, gain=gw, eps=1e-6, out=hout))
    x1 = torch.randn((rows, W), generator=g, device=dev)
    t_old = _timed_graph(lambda: ops.rmsnorm(x1, gw, 1e-6, hout))
    row("streams_step", t_new, rows * W * (4 * (2 * S + 2) + 2), read_bw, "read", "qwen3 norm",
        t_old, rows * W * (4 + 2), read_bw, "read")
    # ---- feed-forwards
    h = rnd(rows, W)
    branch = torch.zeros((rows, W), dtype=torch.float32, device=dev)

    def gated(inter):
        wgu = ops.pretile_weight(ops.interleave_gate_up(rnd(inter, W), rnd(inter, W)))
        wd = ops.pretile_weight(rnd(W, inter))
        act2 = torch.empty((rows, inter), dtype=bf, device=dev)

        def run():
            ops.gemm_swiglu(h, wgu, act2, w_tiled=True)
            ops.gemm(act2, wd, branch, accumulate=True, w_tiled=True)
        return _timed_graph(run)
    moe = next(f for f in sh["mlps"] if f["kind"] == "moe")
    r = moe["router"]
    E, I, top, ff, shared = r["experts"], r["identity"], r["top"], moe["expert"]["ff"], moe["shared"]["ff"]
    groups = (r["groups"]["count"], r["groups"]["keep"])
    router = torch.randn((E + I + 1, W), generator=g, device=dev) * 0.05
    correction = torch.randn((E + I,), generator=g, device=dev) * 0.01
    ids = torch.empty((rows, top), dtype=torch.int32, device=dev)
    share = torch.empty((rows, top), dtype=torch.float32, device=dev)
    sgate = torch.empty((rows, 1), dtype=torch.float32, device=dev)
    gu, down = rnd(E, 2 * ff, W), rnd(E, W, ff)
    y = torch.empty((rows, top, ff), dtype=bf, device=dev)
    wsgu = ops.pretile_weight(rnd(2 * shared, W))
    wsd = ops.pretile_weight(rnd(W, shared))
    sgu = torch.empty((rows, 2 * shared), dtype=bf, device=dev)
    sy = torch.empty((rows, shared), dtype=bf, device=dev)

    def mixture():
        ops.moe_route(h, router, None, ids, share, scoring="softmax_all", correction=correction,
                      groups=groups, group_mark=1, normalize=False, weight_scale=2.5, extra=sgate)
        ops.moe_experts(h, gu, down, ids, share, y, branch, 0.0, 1.0, 0.0, add=False, n_identity=I)
        ops.gemm(h, wsgu, sgu, w_tiled=True)
        ops.gated_act(sgu, sy, 0.0, 1.0, 0.0, row_factor=sgate[:, 0])
        ops.gemm(sy, wsd, branch, accumulate=True, w_tiled=True)
    t_new = _timed_graph(mixture)
    inter = (top * ff + shared) // 64 * 64
    t_old = gated(inter)
    if decode:
        used = min(E, rows * top)
        row("mixture", t_new, (used * ff + shared) * 3 * W * 2, read_bw, "read",
            "qwen3 feed-forward of the width a token uses", t_old, 3 * inter * W * 2, read_bw,
            "read")
    else:
        row("mixture", t_new, 2.0 * rows * 3 * (top * ff + shared) * W, mfma_rate, "mfma",
            "qwen3 feed-forward of the width a token uses", t_old, 2.0 * rows * 3 * inter * W,
            mfma_rate, "mfma")
    return out


def main_kugisun(args) -> int:
    """Prefill and decode throughput of Kugisun shapes beside the dense Qwen3 decoder of equal
    size, and the new kernels alone beside the like kernels of that decoder and of Nupovik."""
    import torch
    import zinfer_amd.ops as ops
    from zinfer_amd.config import entry_for
    T, batch, prompt = args.prefill_tokens, args.batch, args.prompt_len
    max_positions = max(T, prompt + args.steps + args.warmup + 64) + 64
    read_bw = ops.measure_read_bandwidth("cuda:0")
    mfma_rate = ops.measure_mfma_rate("cuda:0")
    names = [args.kugisun_shape] if args.kugisun_shape else list(KUGISUN_SHAPES)
    shapes = {}
    for name in names:
        sh = KUGISUN_SHAPES[name]
        row = {"sizes": {k: sh[k] for k in ("width", "vocab", "streams", "mixer", "mlps", "order")}}
        for label, raw in (("kugisun", kugisun_config(sh, max_positions)),
                           ("qwen3", kugisun_twin(sh, max_positions))):
            cfg = entry_for(raw).config_type.from_dict(raw)
            pool = batch * (prompt + args.steps + args.warmup + 64) + T + 256
            llm = build_llm(raw, args.dtype, args.seed, pool, max(batch, 8),
                            max_step_tokens=max(T, 2048), multi_step=args.multi_step)
            t_pre = run_prefill(llm, cfg, T, args.seed + 1)
            dt, mean_ctx = run_decode(llm, cfg, batch, prompt, args.steps, args.warmup, args.seed + 2)
            row[label] = {"prefill_tokens_per_s": round(T / t_pre, 1), "prefill_ms": round(t_pre * 1e3, 3),
                          "decode_tokens_per_s": round(batch * args.steps / dt, 1),
                          "decode_ms_per_step": round(dt / args.steps * 1e3, 4),
                          "decode_mean_context": round(mean_ctx, 1)}
            drop(llm)
        row["prefill_vs_qwen3"] = round(row["kugisun"]["prefill_tokens_per_s"]
                                        / row["qwen3"]["prefill_tokens_per_s"], 3)
        row["decode_vs_qwen3"] = round(row["kugisun"]["decode_tokens_per_s"]
                                       / row["qwen3"]["decode_tokens_per_s"], 3)
        if args.dtype == "bfloat16":
            row["kernels_prefill"] = kugisun_kernels(sh, T, T, mfma_rate, read_bw)
            row["kernels_decode"] = kugisun_kernels(sh, 1, prompt, mfma_rate, read_bw)
        ops._workspaces.clear()
        torch.cuda.empty_cache()
        shapes[name] = row
    first = shapes[names[0]]
    print(json.dumps({
        "metric": "kugisun_decode_tokens_per_s", "value": first["kugisun"]["decode_tokens_per_s"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": first["kugisun"]["decode_ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic", "config": {"model": f"Kugisun {names[0]} shape beside the dense Qwen3 "
                                                 "decoder of equal size, random weights",
                                        "batch": batch, "prompt_len": prompt, "prefill_tokens": T,
                                        "parallelism": "single GPU"},
        "measured_read_gbs": round(read_bw / 1e9, 1), "mfma_loop_tflops": round(mfma_rate / 1e12, 1),
        "shapes": shapes}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--workload", default="decode", choices=["decode", "continuous", "long-context", "fezupel", "lodenex", "nupovik",
                             "kugisun"])
    ap.add_argument("--shape", default=None, choices=sorted(SHAPES),
                    help="layer sizes (default: 8b for decode, 14b for continuous, 32b for "
                         "long-context)")
    ap.add_argument("--multi-step", type=int, default=8,
                    help="most decode steps in a row on the device without the host between")
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the "
                    "configuration has (both numbers are reported)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true",
                    help="only the headline: no other batches, prompt lengths or workloads")
    ap.add_argument("--no-long-context-points", dest="long_context_points", action="store_false",
                    help="leave the 32B-shape points out of the default line")
    ap.add_argument("--check-fp32", type=int, default=None, metavar="TOKENS",
                    help="also run a prompt of TOKENS tokens and one decode token through a true "
                         "32-bit engine with the same weights and report how far the logits "
                         "are apart (default: 2048, with --no-points 0 = not at all)")
    ap.add_argument("--requests", type=int, default=32, help="continuous: requests")
    ap.add_argument("--prompt-min", type=int, default=128)
    ap.add_argument("--prompt-max", type=int, default=4096)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--chunk", type=int, default=512, help="continuous: tokens of a prompt per step")
    ap.add_argument("--step-tokens", type=int, default=None,
                    help="continuous: token budget of a step (default: the chunk, so that a "
                         "prompt's portion and the decode tokens beside it fill whole tiles)")
    ap.add_argument("--context", type=int, default=8192, help="long-context: context decoded at")
    ap.add_argument("--batches", default="1,8,64",
                    help="long-context: the batch sizes decoded at (the pool holds the largest)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--fezupel-shape", default=None, choices=sorted(FEZUPEL_SHAPES),
                    help="fezupel: only this shape (default: all of them)")
    ap.add_argument("--lodenex-shape", default=None, choices=sorted(LODENEX_SHAPES),
                    help="lodenex: only this shape (default: gqa, latent and mixed)")
    ap.add_argument("--nupovik-shape", default=None, choices=sorted(NUPOVIK_SHAPES),
                    help="nupovik: only this shape (default: all of them)")
    ap.add_argument("--kugisun-shape", default=None, choices=sorted(KUGISUN_SHAPES),
                    help="kugisun: only this shape (default: all of them)")
    ap.add_argument("--no-run-graphs", action="store_true",
                    help="decode steps in a row replay one graph per step instead of one for the run")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py runs on one GPU only (asked for {args.gpus}): this engine has no "
              "multi-GPU path")
        return 2
    return {"decode": main_decode, "continuous": main_continuous,
            "long-context": main_long_context, "fezupel": main_fezupel,
            "lodenex": main_lodenex, "nupovik": main_nupovik,
            "kugisun": main_kugisun}[args.workload](args)


if __name__ == "__main__":
    sys.exit(main())
