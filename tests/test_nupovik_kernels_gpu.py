"""Each mechanism of the Nupovik design alone against the plain functions of ``plain_nupovik``,
in 32-bit and in bfloat16: the position vectors, the two streams side by side, the blends of
a row with the row before it (the row kept in a state slot), the recurrence with both decay
rules and both output rules (states in slots, portions against the whole, key sizes off the
kernel's groups of channels, a token far back kept by a channel that does not decay and lost
by one that does), the norm a head with gain and gate, the sigmoid router (corrections that
make every choice score negative, groups marked by two scores, groups of one), experts
without a gate in both forms, and the attention over a latent with a gate a head (a loud key
far back, at a page's border and at position 0)."""
import math

import pytest
import torch

import plain_nupovik as P
from gpu_util import DEV, rel_err, tol
from test_lodenex_kernels_gpu import Paged
from zinfer_amd import ops

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _rand(shape, seed, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def _starts(lens):
    out = [0]
    for n in lens:
        out.append(out[-1] + n)
    return out


# ------------------------------------------------------------------------------ embedding
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W", [6, 50, 51, 320])
def test_embed_sinusoid(dt, W):
    V = 23
    table = _rand((V, W), 1, 1.0, dt)
    ids = [5, 0, 22, 7, 7, 13, 1]
    near = [0, 1, 2, 63, 64, 65, 99]
    far = [500, 1023, 1024, 2047, 2048, 2999, 3000]
    freq = torch.tensor([P.POSITION_BASE ** (-2.0 * i / W) for i in range((W + 1) // 2)],
                        dtype=torch.float64).to(torch.float32).to(DEV)
    for positions, limit in ((near, 2e-5), (far, 1e-3)):
        out = torch.empty((len(ids), W), dtype=torch.float32, device=DEV)
        ops.embed_sinusoid(table.to(DEV), _i32(ids), _i32(positions), freq, out)
        want = table[ids].double()
        for row, p in enumerate(positions):
            want[row] += P.position_vectors(1, W, start=p)[0]
        # (an angle is the 32-bit product position * frequency: its error grows with the position)
        assert float((out.double().cpu() - want).abs().max()) < limit
    # sine at even entries, cosine at odd ones: at position 0 they are 0 and 1
    out = torch.empty((1, W), dtype=torch.float32, device=DEV)
    ops.embed_sinusoid(torch.zeros((V, W), dtype=dt, device=DEV), _i32([3]), _i32([0]), freq, out)
    assert torch.equal(out[0, 0::2].cpu(), torch.zeros((W + 1) // 2))
    assert torch.equal(out[0, 1::2].cpu(), torch.ones(W // 2))


@pytest.mark.parametrize("dt", DTYPES)
def test_concat_rows(dt):
    a, b = _rand((5, 37), 2), _rand((5, 37), 3)
    out = torch.empty((5, 74), dtype=dt, device=DEV)
    ops.concat_rows(a.to(DEV), b.to(DEV), out)
    assert torch.equal(out.cpu(), torch.cat([a, b], dim=1).to(dt))


# ------------------------------------------------------------------------------ token shift
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W", [10, 48, 321])
def test_token_shift_mix(dt, W):
    """Three requests over two steps: whole rows first, then one token, two tokens and none;
    slots out of order, a state row that holds other numbers in front of the kept row."""
    n_mix, offset, slots = 5, 7, [4, 0, 2]
    mu = torch.rand((n_mix, W), generator=torch.Generator().manual_seed(4))
    seqs = [_rand((n, W), 10 + i, 1.0, dt) for i, n in enumerate([6, 1, 9])]
    state = torch.zeros((5, offset + W), dtype=torch.float32, device=DEV)
    state[:, :offset] = 3.0

    def step(parts, which):
        lens = [p.shape[0] for p in parts]
        T = sum(lens)
        out = torch.empty((n_mix, T, W), dtype=dt, device=DEV)
        seq_index = [i for i, n in enumerate(lens) for _ in range(n)]
        ops.token_shift_mix(torch.cat(parts).to(DEV), mu.to(DEV), state, offset,
                            _i32([slots[i] for i in which]), _i32(seq_index), _i32(_starts(lens)),
                            out)
        return out, _starts(lens)

    first = [seqs[0][:4], seqs[1][:1], seqs[2][:7]]
    out, at = step(first, [0, 1, 2])
    for i, part in enumerate(first):
        for m in range(n_mix):
            want = P.token_shift(part, mu[m])
            assert rel_err(out[m, at[i]:at[i + 1]], want) < tol(dt)
        assert torch.equal(state[slots[i], offset:].cpu(), part[-1].float())
    second = [seqs[2][7:], seqs[0][4:]]            # one request left out, the others swapped
    out, at = step(second, [2, 0])
    for j, (i, part, before) in enumerate([(2, seqs[2][7:], seqs[2][6]), (0, seqs[0][4:], seqs[0][3])]):
        for m in range(n_mix):
            want = P.token_shift(part, mu[m], before=before)
            assert rel_err(out[m, at[j]:at[j + 1]], want) < tol(dt)
        assert torch.equal(state[slots[i], offset:].cpu(), part[-1].float())
    # the request that was left out keeps its row; nothing in front of the rows was touched
    assert torch.equal(state[slots[1], offset:].cpu(), seqs[1][0].float())
    assert float((state[:, :offset] - 3.0).abs().max()) == 0.0


# ------------------------------------------------------------------------------ the recurrence
def _decays(z, bias, rule, tau):
    x = z.double() + bias.double()
    return torch.sigmoid(x).pow(1.0 / tau) if rule == "sigmoid_root" else torch.exp(-torch.exp(x))


def _plain_recurrence(q, k, v, z, bias, bonus, H, d, dv, rule, tau, q_scale, state=None):
    """(o [T, H dv], S [H, d, dv]) of one sequence."""
    T = q.shape[0]
    a = _decays(z, bias, rule, tau).view(T, H, d)
    qq, kk, vv = (q.double() * q_scale).view(T, H, d), k.double().view(T, H, d), v.double().view(T, H, dv)
    o = torch.zeros((T, H, dv), dtype=torch.float64)
    S = torch.zeros((H, d, dv), dtype=torch.float64)
    for h in range(H):
        o[:, h], S[h] = P.decayed_outer_recurrence(
            qq[:, h], kk[:, h], vv[:, h], a[:, h],
            bonus=None if bonus is None else bonus.double().view(H, d)[h],
            state=None if state is None else state[h])
    return o.reshape(T, H * dv), S


def _run_recurrence(parts, state, slots, bias, bonus, H, d, dv, rule, tau, q_scale, dt, columns=None,
                    span=0):
    """``parts``: (q, k, v, z) a sequence for this step.  ``span`` 0: token by token from end to
    end; None: the spans the product chooses; else spans of that many tokens."""
    lens = [p[0].shape[0] for p in parts]
    cat = [torch.cat([p[i] for p in parts]) for i in range(4)]
    T = sum(lens)
    out = torch.full((T, H * dv), float("nan"), dtype=torch.float32, device=DEV)
    ops.decay_recurrence(cat[0].to(dt).to(DEV), cat[1].to(dt).to(DEV), cat[2].to(dt).to(DEV),
                         cat[3].to(DEV), bias.to(DEV), None if bonus is None else bonus.to(DEV),
                         state, _i32(slots), _i32(_starts(lens)), out, H, d, dv, rule, tau=tau,
                         q_scale=q_scale, columns=columns, max_q_len=max(lens), span=span)
    return out.cpu(), _starts(lens)


RECURRENCES = [  # H, d, dv, rule, bonus, tau, lens
    (3, 12, 12, "double_exp", True, 1.0, [21, 1, 40]),
    (2, 20, 12, "sigmoid_root", False, 4.0, [17, 2, 33]),
    (1, 1, 1, "sigmoid_root", False, 1.0, [9, 5]),
    (4, 8, 16, "sigmoid_root", False, 16.0, [50]),
    (1, 24, 24, "double_exp", True, 1.0, [3, 64]),
    (2, 64, 100, "sigmoid_root", False, 8.0, [19, 30]),
    (1, 256, 8, "double_exp", True, 1.0, [11]),
    (5, 7, 3, "sigmoid_root", True, 2.5, [26, 26, 1, 4]),
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", RECURRENCES)
def test_decay_recurrence_against_plain(dt, case):
    """Sequences of unequal length in one launch, whole; then the same sequences in two steps
    (cut at every sequence's own place, down to one token on a side) from the states the first
    step left, in other slots' company; the states themselves."""
    H, d, dv, rule, with_bonus, tau, lens = case
    q_scale = d ** -0.5
    seqs = []
    for i, n in enumerate(lens):
        q, k = _rand((n, H * d), 100 + i, 1.0, dt), _rand((n, H * d), 200 + i, 1.0, dt)
        v = _rand((n, H * dv), 300 + i, 1.0, dt)
        z = _rand((n, H * d), 400 + i, 2.0)
        seqs.append((q, k, v, z))
    bias = _rand((H * d,), 5, 1.0) + (1.0 if rule == "sigmoid_root" else -1.5)
    bonus = _rand((H * d,), 6, 0.5) if with_bonus else None
    size = ops.recurrence_state_size(H, d, dv)
    state = torch.zeros((len(lens) + 2, size + 5), dtype=torch.float32, device=DEV)
    slots = list(range(len(lens), 0, -1))
    out, at = _run_recurrence(seqs, state, slots, bias, bonus, H, d, dv, rule, tau, q_scale, dt)
    limit = 2e-5 if dt == torch.float32 else 2.0 ** -7
    for i, s in enumerate(seqs):
        want, S = _plain_recurrence(*s, bias, bonus, H, d, dv, rule, tau, q_scale)
        assert rel_err(out[at[i]:at[i + 1]], want) < limit, i
        got = ops.recurrence_state_matrix(state[slots[i]], H, d, dv)
        assert rel_err(got, S) < 2e-5, i
    assert float(state[0].abs().max()) == 0.0 and float(state[:, size:].abs().max()) == 0.0
    # in two steps, with other columns a workgroup: the same bits in 32-bit
    again = torch.zeros_like(state)
    cuts = [max(1, n - 1 - i) if n > 1 else 1 for i, n in enumerate(lens)]
    heads = [tuple(t[:c] for t in s) for s, c in zip(seqs, cuts)]
    tails = [(i, tuple(t[c:] for t in s)) for i, (s, c) in enumerate(zip(seqs, cuts)) if c < lens[i]]
    o1, a1 = _run_recurrence(heads, again, slots, bias, bonus, H, d, dv, rule, tau, q_scale, dt,
                             columns=1 if dv < 4 else None)
    o2, a2 = _run_recurrence([t for _, t in tails], again, [slots[i] for i, _ in tails], bias,
                             bonus, H, d, dv, rule, tau, q_scale, dt,
                             columns=min(dv, 256 // ((d + 7) // 8)))
    for i in range(len(lens)):
        pieces = [o1[a1[i]:a1[i + 1]]]
        for j, (which, _) in enumerate(tails):
            if which == i:
                pieces.append(o2[a2[j]:a2[j + 1]])
        assert torch.equal(torch.cat(pieces), out[at[i]:at[i + 1]]), i
    assert torch.equal(again, state)


SPANNED = [  # H, d, dv, rule, bonus, tau, span, lens of the first step, lens of the second
    (2, 12, 12, "double_exp", True, 1.0, 16, [33, 1, 80, 16, 49], [40, 2, 1, 33, 64]),
    (3, 20, 9, "sigmoid_root", False, 4.0, 16, [100, 32, 17], [1, 97, 48]),
    (1, 64, 40, "sigmoid_root", False, 16.0, 32, [200, 65], [129, 3]),
    (2, 136, 8, "double_exp", True, 1.0, 16, [48, 50], [35, 1]),
    (4, 8, 16, "double_exp", True, 1.0, None, [300, 129, 5], [130, 1, 260]),
    (1, 7, 3, "sigmoid_root", True, 2.5, 48, [150], [97]),
    # more tokens than the most spans of the usual length hold: the spans grow
    (1, 8, 4, "sigmoid_root", False, 8.0, None, [4200, 70], [3, 1]),
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", SPANNED)
def test_decay_recurrence_in_spans(dt, case):
    """Portions of several spans beside portions of one span and single tokens, in one launch:
    lengths that end at a span's edge, one token behind it and one before it.  Two steps: the
    second starts from the states the first left and leaves its own."""
    H, d, dv, rule, with_bonus, tau, span, first, second = case
    q_scale = d ** -0.5
    seqs = []
    for i, n in enumerate(a + b for a, b in zip(first, second)):
        q, k = _rand((n, H * d), 100 + i, 1.0, dt), _rand((n, H * d), 200 + i, 1.0, dt)
        seqs.append((q, k, _rand((n, H * dv), 300 + i, 1.0, dt), _rand((n, H * d), 400 + i, 2.0)))
    bias = _rand((H * d,), 5, 1.0) + (2.0 if rule == "sigmoid_root" else -2.0)
    bonus = _rand((H * d,), 6, 0.5) if with_bonus else None
    size = ops.recurrence_state_size(H, d, dv)
    state = torch.zeros((len(seqs) + 1, size + 3), dtype=torch.float32, device=DEV)
    slots = list(range(len(seqs), 0, -1))
    heads = [tuple(t[:c] for t in s) for s, c in zip(seqs, first)]
    tails = [tuple(t[c:] for t in s) for s, c in zip(seqs, first)]
    o1, a1 = _run_recurrence(heads, state, slots, bias, bonus, H, d, dv, rule, tau, q_scale, dt,
                             span=span)
    limit = 2e-5 if dt == torch.float32 else 2.0 ** -7
    for i, (s, c) in enumerate(zip(seqs, first)):
        want, S = _plain_recurrence(*(t[:c] for t in s), bias, bonus, H, d, dv, rule, tau, q_scale)
        assert rel_err(o1[a1[i]:a1[i + 1]], want) < limit, i
        assert rel_err(ops.recurrence_state_matrix(state[slots[i]], H, d, dv), S) < 2e-5, i
    order = list(reversed(range(len(seqs))))        # the second step lists the requests backwards
    o2, a2 = _run_recurrence([tails[i] for i in order], state, [slots[i] for i in order], bias,
                             bonus, H, d, dv, rule, tau, q_scale, dt, span=span)
    for j, i in enumerate(order):
        want, S = _plain_recurrence(*seqs[i], bias, bonus, H, d, dv, rule, tau, q_scale)
        assert rel_err(o2[a2[j]:a2[j + 1]], want[first[i]:]) < limit, i
        assert rel_err(ops.recurrence_state_matrix(state[slots[i]], H, d, dv), S) < 2e-5, i
    assert float(state[0].abs().max()) == 0.0 and float(state[:, size:].abs().max()) == 0.0
    # against the walk from end to end: rounding apart, the same
    again = torch.zeros_like(state)
    w1, _ = _run_recurrence(heads, again, slots, bias, bonus, H, d, dv, rule, tau, q_scale, dt)
    assert rel_err(o1, w1) < 1e-5


@pytest.mark.parametrize("rule", ["sigmoid_root", "double_exp"])
def test_a_token_far_back_is_kept_or_lost_by_its_channel(rule):
    """Channel 0 does not decay, channel 1 decays fast.  A key on channel 0 at position 2 with
    a value of its own is read back 600 tokens later, in a prompt and by a token alone; the
    same key on channel 1 is gone after a few tokens; the token's own outer product is in the
    output of the rule that reads the new state and enters the other rule's only through the
    bonus."""
    H, d, dv, n = 1, 10, 4, 603
    keep, lose = (30.0, -30.0) if rule == "sigmoid_root" else (-30.0, 3.0)
    bias = torch.full((d,), lose)
    bias[0] = keep
    for channel, seen in ((0, True), (1, False)):
        q, k = torch.zeros((n, d)), torch.zeros((n, d))
        v = _rand((n, dv), 7, 0.01)
        k[:, 2:] = _rand((n, d - 2), 8, 0.1)
        k[2, :] = 0.0
        k[2, channel] = 4.0
        v[2] = torch.tensor([1.0, -2.0, 3.0, 0.5])
        q[-1, channel] = 1.0
        z = torch.zeros((n, d))
        bonus = torch.zeros((d,)) if rule == "double_exp" else None
        want, _ = _plain_recurrence(q, k, v, z, bias, bonus, H, d, dv, rule, 1.0, 1.0)
        # whole; the last token alone; cut right behind the key; each token by token and in spans
        for cut, span in ((n, 0), (n, None), (n, 16), (n - 1, None), (3, 0), (3, None), (2, 0)):
            state = torch.zeros((1, ops.recurrence_state_size(H, d, dv)), device=DEV)
            outs = []
            for a, b in ((0, cut), (cut, n)):
                if a < b:
                    o, _ = _run_recurrence([(q[a:b], k[a:b], v[a:b], z[a:b])], state, [0], bias,
                                           bonus, H, d, dv, rule, 1.0, 1.0, torch.float32,
                                           span=span)
                    outs.append(o)
            got = torch.cat(outs)
            assert rel_err(got, want) < 2e-5
            if seen:
                assert float((got[-1] - 4.0 * v[2]).abs().max()) < 1e-3
            else:
                assert float(got[-1].abs().max()) < 1e-3
    # the token's own product: S_t holds it, S_(t-1) does not unless the bonus brings it in
    q, k, v = torch.ones((1, d)), torch.ones((1, d)), torch.ones((1, dv))
    for bonus, want in ((None, float(d)), (torch.zeros((d,)), 0.0), (torch.full((d,), 0.5), 0.5 * d)):
        if (bonus is None) != (rule == "sigmoid_root"):
            continue
        state = torch.zeros((1, ops.recurrence_state_size(H, d, dv)), device=DEV)
        o, _ = _run_recurrence([(q, k, v, torch.zeros((1, d)))], state, [0], bias, bonus, H, d, dv,
                               rule, 1.0, 1.0, torch.float32)
        assert float((o - want).abs().max()) < 1e-5


def test_the_root_of_the_sigmoid_is_taken():
    """tau > 1 brings a decay nearer to 1: after 8 tokens a key's weight is sigmoid(b)^(8 / tau),
    which differs from sigmoid(b)^8 by orders of magnitude."""
    H, d, dv, n, tau, b = 1, 8, 2, 9, 16.0, -1.0
    q, k, v = torch.zeros((n, d)), torch.zeros((n, d)), torch.zeros((n, dv))
    k[0, 0], v[0, 0], q[-1, 0] = 1.0, 1.0, 1.0
    state = torch.zeros((1, ops.recurrence_state_size(H, d, dv)), device=DEV)
    o, _ = _run_recurrence([(q, k, v, torch.zeros((n, d)))], state, [0], torch.full((d,), b), None,
                           H, d, dv, "sigmoid_root", tau, 1.0, torch.float32)
    want = (1.0 / (1.0 + math.exp(-b))) ** ((n - 1) / tau)
    assert abs(float(o[-1, 0]) - want) < 1e-5 and want > 0.5


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H, dv, whole", [(3, 12, False), (1, 40, True), (6, 4, True), (4, 64, False),
                                          (2, 128, True)])
def test_head_norm_gate(dt, H, dv, whole):
    T, eps = 5, 1e-3
    o = _rand((T, H * dv), 20, 3.0)
    o[1] *= 1e-3                                   # eps matters where a head is small
    gain = 1.0 + _rand((H * dv,) if whole else (dv,), 21, 0.3)
    gate = _rand((T, H * dv + 9), 22, 1.5, dt)[:, 4:4 + H * dv]     # rows inside wider rows
    out = torch.empty((T, H * dv), dtype=dt, device=DEV)
    ops.head_norm_gate(o.to(DEV), gain.to(DEV), gate.to(DEV), out, H, eps)
    normed = P.rms_norm(o.view(T, H, dv), None, eps)
    normed = normed * (gain.double().view(H, dv) if whole else gain.double())
    want = normed.reshape(T, H * dv) * P.silu(gate.double())
    assert rel_err(out, want) < tol(dt)


# ------------------------------------------------------------------------------ router, experts
def _route(h, router, correction, experts, top, groups):
    T = h.shape[0]
    ids = torch.empty((T, top), dtype=torch.int32, device=DEV)
    weights = torch.empty((T, top), dtype=torch.float32, device=DEV)
    ops.moe_route(h.to(DEV), router.to(DEV), None, ids, weights, scoring="sigmoid",
                  correction=correction.to(DEV), groups=groups)
    return ids.cpu(), weights.cpu()


ROUTERS = [  # experts, top, groups, the correction's mean and spread
    (8, 2, (4, 3), 0.0, 0.3), (8, 2, (4, 3), -5.0, 0.5), (6, 2, (3, 2), 0.0, 0.3),
    (16, 3, (4, 2), -2.0, 1.0), (5, 3, (5, 4), 0.0, 0.5), (9, 2, (3, 1), -1.0, 0.4),
    (4, 1, None, 0.0, 0.5), (3, 3, None, -3.0, 1.0), (64, 8, (8, 4), 0.0, 0.2),
    (12, 4, (2, 1), 0.5, 0.5), (7, 7, (1, 1), 0.0, 1.0),
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", ROUTERS)
def test_sigmoid_router_against_plain(dt, case):
    """Also with corrections that make every choice score negative (an expert outside the kept
    groups must lose against them, so its score counts as minus infinity and not as 0), with
    groups of one expert (marked by that one score) and with a single group."""
    experts, top, groups, mean, spread = case
    T, W = 64, 40
    h = _rand((T, W), 30, 1.0, dt)
    router = _rand((experts, W), 31, 3.0 / math.sqrt(W))
    correction = mean + _rand((experts,), 32, spread)
    ids, weights = _route(h, router, correction, experts, top, groups)
    r = {"experts": experts, "top": top,
         "groups": None if groups is None else {"count": groups[0], "keep": groups[1]}}
    chosen, want = P.route(h.double(), router, correction, r)
    assert torch.equal(ids.long(), chosen)
    assert rel_err(weights, want) < 1e-5
    assert float((weights.sum(dim=1) - 1.0).abs().max()) < 1e-5


def test_router_by_hand():
    """Scores made so that each rule decides: the correction changes the choice and not the
    weights; a group is marked by the sum of its two largest choice scores, not by its
    largest; an expert outside the kept groups is not chosen although its score is the
    largest left, also where every kept score is negative."""
    W = 8
    router = torch.zeros((8, W))
    logits = torch.tensor([2.0, -1.0, 0.5, 0.4, 0.9, 0.8, -2.0, -3.0])
    router[:, 0] = logits
    h = torch.zeros((1, W))
    h[0, 0] = 1.0
    s = torch.sigmoid(logits.double())
    zero = torch.zeros((8,))
    # no groups, no correction: experts 0 and 4
    ids, w = _route(h, router, zero, 8, 2, None)
    assert ids.tolist() == [[0, 4]]
    assert rel_err(w, (s[[0, 4]] / s[[0, 4]].sum())[None]) < 1e-6
    # a correction lifts expert 7 to the top: it is chosen first, its weight is its plain score
    lift = zero.clone()
    lift[7] = 5.0
    ids, w = _route(h, router, lift, 8, 2, None)
    assert ids.tolist() == [[7, 0]]
    assert rel_err(w, (s[[7, 0]] / s[[7, 0]].sum())[None]) < 1e-6
    # four groups of two, one kept: group 0 has the largest expert (0.88 + 0.27 = 1.15) but
    # group 2's two add up to more (0.71 + 0.69 = 1.40)
    ids, w = _route(h, router, zero, 8, 2, (4, 1))
    assert ids.tolist() == [[4, 5]]
    # two kept: groups 2 and 1 (0.62 + 0.60 = 1.22); expert 0 stays out
    ids, w = _route(h, router, zero, 8, 3, (4, 2))
    assert ids.tolist() == [[4, 5, 2]]
    # every choice score negative: still groups 2 and 1, and never expert 0 (whose -9.12 would
    # lose against a 0 but wins against nothing that is left once it is shut out)
    ids, w = _route(h, router, torch.full((8,), -10.0), 8, 4, (4, 2))
    assert ids.tolist() == [[4, 5, 2, 3]]
    assert rel_err(w, (s[[4, 5, 2, 3]] / s[[4, 5, 2, 3]].sum())[None]) < 1e-6


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("T, W, ff, experts, top", [(3, 48, 24, 6, 2), (1, 50, 14, 3, 3), (40, 64, 40, 5, 1),
                                                     (200, 128, 64, 16, 3), (70, 320, 96, 8, 2)])
def test_experts_without_a_gate(dt, T, W, ff, experts, top):
    """W_down relu(W_up h)^2, weighted and summed in the order chosen; a few tokens and many
    (the many-token form in bfloat16 sorts tokens by expert)."""
    h = _rand((T, W), 40, 1.0, dt)
    w = {"router": _rand((experts, W), 41, 3.0 / math.sqrt(W)), "correction": _rand((experts,), 42, 0.3)}
    for e in range(experts):
        w[f"e{e}.up"] = _rand((ff, W), 50 + e, 1.5 / math.sqrt(W), dt)
        w[f"e{e}.down"] = _rand((W, ff), 80 + e, 1.5 / math.sqrt(ff), dt)
    f = {"router": {"experts": experts, "top": top, "groups": None}}
    want = P.moe_ff(h, w, f)
    ids, weights = _route(h, w["router"], w["correction"], experts, top, None)
    up = torch.stack([w[f"e{e}.up"] for e in range(experts)]).to(DEV)
    down = torch.stack([w[f"e{e}.down"] for e in range(experts)]).to(DEV)
    y = torch.empty((T, top, ff), dtype=dt, device=DEV)
    base = _rand((T, W), 43)
    out = base.to(DEV)
    ops.moe_experts(h.to(DEV), up, down, ids.to(DEV), weights.to(DEV), y, out, 0.0, 0.0, 0.0,
                    add=True, act="relu2")
    limit = 2e-5 if dt == torch.float32 else 2.0 ** -6       # y is rounded to bfloat16 on its way
    assert rel_err(out.cpu().double() - base.double(), want) < limit
    out2 = torch.empty((T, W), dtype=torch.float32, device=DEV)
    ops.moe_experts(h.to(DEV), up, down, ids.to(DEV), weights.to(DEV), y, out2, 0.0, 0.0, 0.0,
                    add=False, act="relu2")
    assert rel_err(out2, want) < limit


# ------------------------------------------------------------------------------ latent attention
def _softmax_attention(q, c, H, scale, gate):
    """q [T, H, R] on the latent's side, the last T positions of the latents c [n, R]; every
    position sees itself and all before it; values are the latents; sigmoid gate a head."""
    n, T = c.shape[0], q.shape[0]
    s = torch.einsum("thr,nr->htn", q.double(), c.double()) * scale
    rows = torch.arange(n - T, n)[:, None]
    s = s.masked_fill(torch.arange(n)[None, :] > rows, -math.inf)
    out = torch.einsum("htn,nr->thr", torch.softmax(s, dim=-1), c.double())
    return out if gate is None else out * torch.sigmoid(gate.double())[:, :, None]


def _attend(pg, q, q_lens, dt, H, R, scale, gate):
    T = sum(q_lens)
    out = torch.zeros((T, H * R), dtype=dt, device=DEV)
    seq_index = [s for s, n in enumerate(q_lens) for _ in range(n)]
    ops.attend_masked(q.reshape(T, -1).to(DEV), None if gate is None else gate.to(DEV),
                      None if gate is None else "head", pg.k_pool, None, None, pg.table,
                      _i32(_starts(q_lens)), _i32(pg.lens), _i32(seq_index), out, scale, 0.0, 0, 0,
                      H, 1, R, R, pg.ps, max(q_lens), max(pg.lens))
    return out.view(T, H, R)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H, R, ps, lens, q_lens", [(3, 24, 16, [70, 9], [70, 9]), (6, 96, 16, [300, 120], [40, 1]),
                                                     (4, 64, 8, [150, 33, 64], [1, 1, 1]), (7, 11, 4, [41], [41]),
                                                     (8, 128, 16, [260], [260]), (2, 40, 16, [500, 2], [3, 2])])
def test_attention_over_the_latent_with_a_gate_a_head(dt, H, R, ps, lens, q_lens):
    pg = Paged(lens, 1, R, 0, ps, dt, 60)
    scale = 0.9 / math.sqrt(R)
    T = sum(q_lens)
    qs = [_rand((n, H, R), 61 + i, 1.0, dt) for i, n in enumerate(q_lens)]
    gate = _rand((T, H), 70, 1.5, dt)
    got = _attend(pg, torch.cat(qs), q_lens, dt, H, R, scale, gate)
    at = _starts(q_lens)
    want = torch.cat([_softmax_attention(q, pg.k[s][:, 0], H, scale, gate[at[s]:at[s + 1]])
                      for s, q in enumerate(qs)])
    assert rel_err(got, want) < 2 * tol(dt)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("R", [16, 64, 128])
def test_a_loud_latent_far_back(dt, decode, R):
    """One latent among 700 quiet ones takes nearly all the weight wherever it lies: at
    position 0, a few tokens in, on either side of a page's border, in the middle, right
    before the query and at the query's own place."""
    H, ps, n = 2, 16, 700
    T = 1 if decode else 45
    q = torch.zeros((T, H, R))
    q[:, :, 0] = 1.0
    for at in (0, 3, 15, 16, 351, n - 2, n - 1):
        c = _rand((n, 1, R), 90, 0.3, dt)
        c[at] = 0.0
        c[at, 0, 0] = 30.0
        c[at, 0, 1] = 5.0
        pg = Paged([n], 1, R, 0, ps, dt, 91, k=[c])
        got = _attend(pg, q.to(dt), [T], dt, H, R, 1.0, None)
        last = got[-1].float().cpu()
        assert float((last[:, 1] - 5.0).abs().max()) < 0.05, at
        assert rel_err(got, _softmax_attention(q.to(dt), c[:, 0], H, 1.0, None)) < 2 * tol(dt), at
    # a loud latent behind the query is not seen
    c = _rand((n, 1, R), 92, 0.3, dt)
    c[n - 1] = 0.0
    c[n - 1, 0, 0], c[n - 1, 0, 1] = 30.0, 5.0
    pg = Paged([n], 1, R, 0, ps, dt, 93, k=[c])
    q2 = torch.zeros((2, H, R))
    q2[:, :, 0] = 1.0
    got = _attend(pg, q2.to(dt), [2], dt, H, R, 1.0, None)
    assert float(got[0, :, 1].float().abs().max()) < 1.0
    assert float((got[1, :, 1].float() - 5.0).abs().max()) < 0.05
