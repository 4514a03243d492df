"""Kugisun models through the engine against ``plain_kugisun``, in 32-bit and in bfloat16:
whole prompts; most of a prompt and then its last tokens one by one; portions of changing
size down to two tokens; token by token from the first token on (long decoding); mixed
batches of four live requests in a pool so small that pages are used again (what was given
back is overwritten with NaN first) with four state slots that are used again; the same bits
however a prompt is cut in 32-bit; a slot used again starts from zero; every run of a layer
alone; a token far back that only the attention or only the delta rule can still see; greedy
generation through the entry point and the scheduler; decode steps replayed as graphs; the
replay program and the command line on a model folder."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import kugisun_tiny as kt
import plain_kugisun as P
import traces
from gpu_util import DEV

pytestmark = pytest.mark.gpu

# float32: what is left is the order of sums and the 32-bit angles, decays and exponentials.
# bfloat16: activations are rounded to 8 bits of mantissa some ten times a layer.  A router
# whose two best choice scores lie closer than that rounding may choose another expert than the
# plain implementation, and the delta rule then carries the difference on to the tokens behind.
# So under bfloat16 the median is held to half the tolerance and a third of the positions may
# lie beyond it; 32-bit holds every one.
TOL = {"float32": 4e-5}
LENGTHS = {"A": (1, 5, 23, 60, 150), "B": (2, 9, 47, 130), "C": (3, 17, 64), "D": (4, 33, 100, 260)}
_ref = {}


def _runs(name):
    return len(kt.config_of(name).order)


def _tol(name, dtype):
    if dtype == "float32":
        return TOL[dtype]
    return 0.01 + 0.008 * _runs(name)


def _requests(name, twice=False):
    vocab = kt.CONFIGS[name]["vocab"]
    req = {f"r{i}": kt.tokens(n, vocab, 100 + i) for i, n in enumerate(LENGTHS[name])}
    if twice:
        req.update({f"s{i}": kt.tokens(n, vocab, 200 + i)
                    for i, n in enumerate(reversed(LENGTHS[name]))})
    return req


def _reference(name, requests):
    w = None
    out = {}
    for rid, toks in requests.items():
        key = (name, tuple(toks))
        if key not in _ref:
            w = w or kt.weights_of(name)
            _ref[key] = P.forward(kt.CONFIGS[name], w, toks).numpy()
        out[rid] = _ref[key]
    return out


def _engine(name, dtype, num_pages, poison=True, max_requests=4, use_graphs=True, weights=None):
    from zinfer_amd.engine import Engine
    from zinfer_amd.models.build import build_model
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    w = weights if weights is not None else kt.weights_of(name, dtype=store)
    model = build_model(kt.config_of(name).model_spec(), w, dtype, DEV)
    return Engine(model, page_size=kt.PAGE_SIZE[name], num_pages=num_pages,
                  max_requests=max_requests, poison_freed=poison, use_graphs=use_graphs)


def _replay(eng, steps):
    from zinfer_amd.engine import StepEntry
    outputs = {}
    for st in steps:
        for e in st["entries"]:
            held = eng.length(e["id"]) if eng.has_request(e["id"]) else 0
            assert e["start"] == held
        logits = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]],
                          end=st["end"])
        if logits.shape[0]:
            outputs[st["step"]] = logits.cpu().numpy().copy()
    eng.cache.check()
    assert not eng.cache.requests
    return outputs


def _compare(steps, outputs, ref, vocab, dtype, name):
    tolerance = _tol(name, dtype)
    got = traces.collect(steps, outputs, vocab)
    assert set(got) == set(ref)
    worst, errs = 0.0, []
    for rid in ref:
        assert got[rid].shape == ref[rid].shape
        assert np.isfinite(got[rid]).all(), f"{rid}: logits are not finite"
        err = np.abs(got[rid].astype(np.float64) - ref[rid]).max(axis=1) / np.abs(ref[rid]).max()
        if dtype == "float32":
            bad = np.nonzero(err > tolerance)[0]
            assert bad.size == 0, \
                (f"request {rid}: {bad.size} of {len(err)} positions wrong, the first {bad[0]} "
                 f"(error {err[bad[0]]:.3g} > {tolerance})")
        errs.append(err)
        worst = max(worst, float(err.max()))
    errs = np.concatenate(errs)
    if dtype == "bfloat16":
        assert (errs > tolerance).sum() <= len(errs) / 3 + 1, \
            f"{(errs > tolerance).sum()} of {len(errs)} positions beyond {tolerance}"
        assert float(np.median(errs)) <= tolerance / 2, float(np.median(errs))
    return worst


MODES = {"whole": traces.whole,
         "prefill_then_single": lambda r: traces.prefill_then_single(r, tail=20),
         "portions": traces.changing_portions, "token_by_token": traces.token_by_token,
         "mixed": lambda r: traces.mixed(r, decode_tail=9)}


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(kt.CONFIGS))
def test_replay_modes(name, dtype, mode):
    requests = _requests(name, twice=mode == "mixed")
    steps = MODES[mode](requests)
    page = kt.PAGE_SIZE[name]
    # the pool holds what is live at the fullest step and no more; four state slots
    pages = (traces.peak_tokens(steps, page) + page - 1) // page
    eng = _engine(name, dtype, pages)
    outputs = _replay(eng, steps)
    worst = _compare(steps, outputs, _reference(name, requests), kt.CONFIGS[name]["vocab"], dtype,
                     name)
    if mode == "mixed":
        assert max(len(st["entries"]) for st in steps) == 4
        assert len(requests) > 4                     # so every slot served several requests
        for grp in eng.cache.groups:
            assert grp.pages.handed_out > grp.pages.num_pages, "no page was used again"
    print(f"{name} {dtype} {mode}: error {worst:.3g}")


@pytest.mark.parametrize("name", sorted(kt.CONFIGS))
def test_cut_and_batch_leave_the_bits(name):
    """32-bit: a position's logits are the same bits whole, in portions, token by token and
    beside other requests, whichever slot and pages the request got."""
    requests = _requests(name)
    vocab = kt.CONFIGS[name]["vocab"]
    rows = []
    for mode in ("whole", "portions", "token_by_token", "mixed"):
        steps = MODES[mode](requests)
        eng = _engine(name, "float32", 64, poison=False)
        rows.append(traces.collect(steps, _replay(eng, steps), vocab))
    for other in rows[1:]:
        for rid in rows[0]:
            assert np.array_equal(rows[0][rid], other[rid]), rid


def test_a_slot_that_is_used_again_starts_from_zero():
    """Two requests one after the other in an engine with a single state slot: the second one's
    logits are those it has alone in a fresh engine (32-bit, the same bits): neither the
    matrices nor the convolutions' last rows of the first request are left."""
    name = "A"
    vocab = kt.CONFIGS[name]["vocab"]
    a, b = kt.tokens(40, vocab, 11), kt.tokens(33, vocab, 12)
    eng = _engine(name, "float32", 8, max_requests=1)
    first = _replay(eng, traces.changing_portions({"a": a}, sizes=(9, 2, 11)))
    again = _replay(eng, traces.changing_portions({"b": b}, sizes=(5, 28)))
    fresh = _replay(_engine(name, "float32", 8, max_requests=1),
                    traces.changing_portions({"b": b}, sizes=(5, 28)))
    assert first and set(again) == set(fresh)
    for k in fresh:
        assert np.array_equal(again[k], fresh[k])


def test_every_run_of_a_layer_alone():
    """Every run of a layer alone (``Engine.probe_block``) on the plain implementation's copies
    of the stream before it gives the plain implementation's copies after it, in 32-bit; and
    the whole model's stream behind every run (the decoder's probe: the copies added up) is
    the plain one."""
    from zinfer_amd.engine import StepEntry
    for name in ("A", "C"):
        raw = kt.CONFIGS[name]
        eps = float(raw["norm"]["eps"])
        toks = kt.tokens(50, raw["vocab"], 3)
        w = kt.weights_of(name)
        sums = []
        P.forward(raw, w, toks, sums)
        cfg = kt.config_of(name)
        eng = _engine(name, "float32", 64, poison=False)
        e = w["embed"].double()[torch.tensor(toks)] + w["pos"].double()[:len(toks)]
        X = [e.clone() for _ in range(int(raw.get("streams", 1)))]
        for run, index in enumerate(cfg.order):
            j = cfg.layer_numbers[index]
            L = raw["layers"][j]
            lw = P.below(w, f"l{j}.")
            X = P.stream_step(X, lw, 1, lambda u: P.parallel_mixer(
                P.norm_one_plus(u, lw["norm1"], eps), P.below(lw, "mix."), L["mixer"], eps))
            if L.get("mlp") is not None:
                X = P.stream_step(X, lw, 2, lambda u: P.feed_forward(
                    P.norm_one_plus(u, lw["norm2"], eps), P.below(lw, "mlp."), L["mlp"]))
        # (the plain model's own walk gives the same sums)
        assert float((sum(X) - sums[-1]).abs().max()) < 1e-9
        # block by block from the plain copies before it
        X = [e.clone() for _ in range(int(raw.get("streams", 1)))]
        for run, index in enumerate(cfg.order):
            j = cfg.layer_numbers[index]
            L = raw["layers"][j]
            lw = P.below(w, f"l{j}.")
            before = torch.stack(X).to(torch.float32).to(DEV)
            if raw.get("streams") is None:
                before = before[0]
            got, held = eng.probe_block(index, before)
            assert held == len(toks)
            X = P.stream_step(X, lw, 1, lambda u: P.parallel_mixer(
                P.norm_one_plus(u, lw["norm1"], eps), P.below(lw, "mix."), L["mixer"], eps))
            if L.get("mlp") is not None:
                X = P.stream_step(X, lw, 2, lambda u: P.feed_forward(
                    P.norm_one_plus(u, lw["norm2"], eps), P.below(lw, "mlp."), L["mlp"]))
            want = torch.stack(X) if raw.get("streams") is not None else X[0]
            err = float((got.cpu().double() - want).abs().max() / want.abs().max())
            assert err < 2e-5, f"{name} run {run}: {err:.3g}"
        seen = []
        eng.model.layer_probe = lambda pos, x: seen.append(x.detach().cpu().double())
        eng.step([StepEntry("r", toks, [])], end=["r"])
        eng.model.layer_probe = None
        assert len(seen) == len(sums)
        for pos, (got, want) in enumerate(zip(seen, sums)):
            # (the sums behind five runs of loud weights: the runs' 32-bit errors add up and the
            # copies' mixing carries them on)
            err = float((got - want).abs().max() / want.abs().max())
            assert err < 1e-4, f"{name} run {pos}: {err:.3g}"


def _loud(name, which):
    """Weights of ``name`` in which one side of every mixer is silent (its output matrix is
    zero), so that what the logits know of a far token they know through the other side."""
    w = kt.weights_of(name)
    for n in w:
        if n.endswith(f".mix.{which}.o"):
            w[n] = torch.zeros_like(w[n])
    return w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("silent", ["left", "right"])
def test_a_token_far_back_shows_through_either_side(silent, dtype):
    """Two prompts of 300 tokens that differ in token 2 alone.  With the delta rule silent only
    the attention reaches that far (its keys lie 19 pages back); with the attention silent only
    the heads whose decay is slow remember.  The last position's logits differ between the
    prompts, and the engine's difference is the plain implementation's: in one step, and with
    the last 40 tokens decoded one by one."""
    name = "A"
    raw = kt.CONFIGS[name]
    w = _loud(name, silent)
    a = kt.tokens(300, raw["vocab"], 77)
    b = list(a)
    b[2] = (a[2] + 1) % raw["vocab"]
    ref = {k: P.forward(raw, w, t)[-1].numpy() for k, t in (("a", a), ("b", b))}
    gap = np.abs(ref["a"] - ref["b"]).max()
    assert gap > 1e-3 * np.abs(ref["a"]).max()          # the far token matters
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    wd = {n: t.to(store) for n, t in w.items()}
    for mode in (traces.whole, lambda r: traces.prefill_then_single(r, tail=40)):
        got = {}
        for k, t in (("a", a), ("b", b)):
            steps = mode({k: t})
            eng = _engine(name, dtype, 32, weights=wd)
            got[k] = traces.collect(steps, _replay(eng, steps), raw["vocab"])[k][-1]
        if dtype == "float32":
            assert np.abs((got["a"] - got["b"]) - (ref["a"] - ref["b"])).max() < 0.02 * gap
        else:
            assert np.abs(got["a"] - got["b"]).max() > 0.3 * gap


def _write_folder(name, path, store):
    from zinfer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(kt.CONFIGS[name], f)
    write_safetensors(os.path.join(path, "model.safetensors"), kt.weights_of(name, dtype=store))
    return path


def _check_greedy(name, prompt, got, w):
    logits = P.forward(kt.CONFIGS[name], w, list(prompt) + list(got))
    for i, tok in enumerate(got):
        row = logits[len(prompt) - 1 + i]
        top2 = torch.topk(row, 2).values
        if float(top2[0] - top2[1]) > 1e-3 * float(row.abs().max()):
            assert int(row.argmax()) == tok, f"token {i} of a prompt of {len(prompt)}"


@pytest.mark.parametrize("name", ["B", "D"])
def test_greedy_generation_through_entry_point_and_scheduler(name, tmp_path):
    """Prompts of unequal length generate together (more prompts than state slots, so slots
    are used again); every request's tokens are the plain implementation's arg-max wherever
    that one is clear."""
    from zinfer_amd.entrypoints import LLM, SamplingParams
    path = _write_folder(name, str(tmp_path / name), torch.float32)
    vocab = kt.CONFIGS[name]["vocab"]
    prompts = [kt.tokens(n, vocab, 300 + n) for n in (3, 41, 18, 7, 29, 12)]
    llm = LLM(path, dtype="float32", device=DEV, page_size=kt.PAGE_SIZE[name], max_tokens=512,
              max_step_tokens=48, chunk_size=16, max_seqs=4)
    n_new = 14
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=n_new,
                                                ignore_eos=True))
    w = kt.weights_of(name)
    for prompt, got in zip(prompts, outs):
        assert len(got) == n_new
        _check_greedy(name, prompt, got, w)


def test_decode_steps_replayed_as_graphs_keep_the_state_right():
    """32-bit: prompt, then forty single tokens through captured graphs (the first step of a
    shape runs once eagerly before it is captured and replayed: matrices and last rows must
    not move twice), against the same without graphs: the same bits."""
    name = "A"
    toks = kt.tokens(70, kt.CONFIGS[name]["vocab"], 21)
    steps = traces.prefill_then_single({"r": toks}, tail=40)
    with_graphs = _engine(name, "float32", 16, poison=False, use_graphs=True)
    a = _replay(with_graphs, steps)
    b = _replay(_engine(name, "float32", 16, poison=False, use_graphs=False), steps)
    assert with_graphs.graph_replays > 30
    for k in b:
        assert np.array_equal(a[k], b[k]), k


def test_long_generation_in_bfloat16_stays_finite_and_uses_graphs(tmp_path):
    """Sixty tokens decoded behind a prompt through the scheduler's runs of decode steps: the
    steps replay as graphs and the tokens are ids."""
    from zinfer_amd.entrypoints import LLM, SamplingParams
    name = "D"
    path = _write_folder(name, str(tmp_path / name), torch.bfloat16)
    prompts = [kt.tokens(n, 512, 400 + n) for n in (5, 70)]
    params = SamplingParams(temperature=0.0, max_new_tokens=60, ignore_eos=True)
    llm = LLM(path, dtype="bfloat16", device=DEV, page_size=16, max_tokens=512, max_seqs=4)
    outs = llm.generate(prompts, params)
    assert all(len(o) == 60 and all(0 <= t < 512 for t in o) for o in outs)
    assert llm.engine.graph_replays > 0


def test_replay_program_on_a_model_folder(tmp_path):
    """``bin/trace_run`` chooses the model class by config.json and writes the logits of a
    mixed trace; both dtypes."""
    name = "C"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    requests = _requests(name, twice=True)
    steps = traces.mixed(requests, decode_tail=5)
    text = "".join(json.dumps({k: v for k, v in st.items()}) + "\n" for st in steps)
    ref = _reference(name, requests)
    for dtype in ("float32", "bfloat16"):
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        path = _write_folder(name, str(tmp_path / dtype), store)
        out = str(tmp_path / ("out_" + dtype))
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path,
                            "--dtype", dtype, "--out", out, "--max-tokens",
                            str(traces.peak_tokens(steps, 64))],
                           input=text, capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        done = [l for l in r.stdout.splitlines() if l.startswith("done ")]
        assert done == [f"done {st['step']}" for st in steps]
        outputs = {st["step"]: np.fromfile(os.path.join(out, f"{st['step']}.f32"), dtype="<f4")
                   for st in steps if any(e["want"] for e in st["entries"])}
        _compare(steps, outputs, ref, kt.CONFIGS[name]["vocab"], dtype, name)


def test_generation_through_the_command_line(tmp_path):
    """``bin/zinfer generate-token-ids`` on a Kugisun folder: the oracle's greedy tokens."""
    name = "A"
    path = _write_folder(name, str(tmp_path / name), torch.float32)
    prompt = kt.tokens(11, kt.CONFIGS[name]["vocab"], 9)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "zinfer"), "generate-token-ids",
                        path, ",".join(map(str, prompt)), "6", "--dtype", "float32"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("tokens: ")][0]
    got = json.loads(line[len("tokens: "):])
    assert got[:len(prompt)] == prompt and len(got) == len(prompt) + 6
    _check_greedy(name, prompt, got[len(prompt):], kt.weights_of(name))
