"""Each mechanism of the Kugisun design alone against the plain functions of ``plain_kugisun``,
in 32-bit and in bfloat16: the stream in several copies (read, write, both in one launch, one
branch and two); a projection's rows with a bias, a norm a head and neighbouring pairs rotated
(both forms of the kernel, into rows and into pages); the short convolutions (unequal
sequences, two steps with a request left out, single tokens, one to four taps); the delta rule
(every padded key size, grouped heads, portions against the whole, a token far back kept by a
head that does not decay and lost by one that does, by hand); the router over all outputs (a
correction that changes the choice and not the weights, a group shut out although it holds the
best output, negative choice scores, the gate beside it); experts with outputs that hand their
input on, streamed and sorted."""
import math

import pytest
import torch

import plain_kugisun as P
from gpu_util import DEV, rel_err, tol
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


# ------------------------------------------------------------------------------ the copies
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("S,W", [(1, 48), (2, 50), (3, 384), (4, 128), (8, 7)])
def test_streams_step(dt, S, W):
    T, eps = 9, 1e-5
    x = _rand((S, T, W), 1)
    a, b, M = _rand((S,), 2), _rand((S,), 3), _rand((S, S), 4)
    w = _rand((W,), 5, 0.3)
    y0, y1 = _rand((T, W), 6), _rand((T, W), 7)
    gain = (1.0 + w).to(DEV)
    xs = [x[s].double() for s in range(S)]
    # the read alone, with the norm and without
    out = torch.empty((T, W), dtype=dt, device=DEV)
    ops.streams_step(x.to(DEV), read=True, in_coef=a.to(DEV), gain=gain, eps=eps, out=out)
    u = sum(float(a[s]) * xs[s] for s in range(S))
    assert rel_err(out, P.norm_one_plus(u, w, eps)) < tol(dt)
    total = torch.empty((T, W), dtype=torch.float32, device=DEV)
    ops.streams_step(x.to(DEV), read=True, out=total)
    assert rel_err(total, sum(xs)) < tol(torch.float32)
    # the write alone: one branch, and two with factors; all copies from the old ones
    for branches, y in (([(y0, 1.0)], y0.double()),
                        ([(y0, 0.6), (y1, -1.1)], 0.6 * y0.double() - 1.1 * y1.double())):
        new = [sum(float(M[s, t]) * xs[s] for s in range(S)) + float(b[t]) * y for t in range(S)]
        xd = x.to(DEV).clone()
        ops.streams_step(xd, [(t.to(DEV), c) for t, c in branches], M.to(DEV), b.to(DEV))
        assert rel_err(xd, torch.stack(new)) < tol(torch.float32)
        # both in one launch: the same copies, and the read sees the new ones
        xe = x.to(DEV).clone()
        ops.streams_step(xe, [(t.to(DEV), c) for t, c in branches], M.to(DEV), b.to(DEV),
                         read=True, in_coef=a.to(DEV), gain=gain, eps=eps, out=out)
        assert torch.equal(xe, xd)
        u = sum(float(a[s]) * new[s] for s in range(S))
        assert rel_err(out, P.norm_one_plus(u, w, eps)) < tol(dt)
    # a view of one copy among several is a stream of one copy
    if S > 1:
        big = x.to(DEV).clone()
        ops.streams_step(big[1:2], read=True, out=total)
        assert torch.equal(total.cpu(), x[1])


# ------------------------------------------------------------------------------ rows of a projection
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,rot", [(4, 2, 12, 20, 6), (3, 3, 16, 8, 16), (2, 1, 96, 160, 40),
                                          (5, 5, 10, 6, 0), (4, 2, 64, 64, 32)])
def test_rows_with_bias_head_norm_and_neighbouring_pairs(dt, H, G, d, dv, rot):
    """q to plain rows, k and v into pages, against the plain norm and rotation; positions up to
    3000; sizes the 16-byte form of the kernel takes (in bfloat16) and sizes it does not."""
    T, ps, eps, base = 7, 4, 1e-5, 1000.0
    qw, kw, vw = H * d, G * d, G * dv
    src = _rand((T, qw + kw + vw), 11, 1.0, dt)
    bias = _rand((qw + kw + vw,), 12, 0.5)
    gq, gk = 1.0 + _rand((d,), 13, 0.3), 1.0 + _rand((d,), 14, 0.3)
    positions = [0, 1, 2, 63, 64, 1500, 3000]
    freq = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)],
                        dtype=torch.float64).to(torch.float32).to(DEV) if rot else None
    slots = [9, 2, 3, 12, 0, 5, 6]
    n_pages = 4
    q = torch.empty((T, qw), dtype=dt, device=DEV)
    k_pool = torch.zeros((n_pages, G * ps * d), dtype=dt, device=DEV)
    v_pool = torch.zeros((n_pages, G * ps * dv), dtype=dt, device=DEV)
    kw_args = dict(rot_dims=rot, freq=freq, interleaved=True) if rot else {}
    b = bias.to(DEV)
    ops.project_rows(src.to(DEV), _i32(positions), _i32(slots), ps, [
        ops.RowSegment(0, qw, q, gain=gq.to(DEV), eps=eps, hd=d, bias=b[:qw].contiguous(),
                       per_head=True, **kw_args),
        ops.RowSegment(qw, kw, k_pool, gain=gk.to(DEV), eps=eps, hd=d, pool_heads=G,
                       bias=b[qw:qw + kw].contiguous(), per_head=True, **kw_args),
        ops.RowSegment(qw + kw, vw, v_pool, hd=dv, pool_heads=G,
                       bias=b[qw + kw:].contiguous())])
    x = src.double() + bias.double()
    pos = torch.tensor(positions)
    want_q = P.norm_plain(x[:, :qw].view(T, H, d), gq, eps)
    want_k = P.norm_plain(x[:, qw:qw + kw].view(T, G, d), gk, eps)
    if rot:
        want_q, want_k = P.rotate_pairs(want_q, pos, rot, base), P.rotate_pairs(want_k, pos, rot, base)
    # (an angle is the 32-bit product position * frequency: its error grows with the position)
    limit = max(tol(dt), 2e-4)
    assert rel_err(q, want_q.reshape(T, qw)) < limit
    k_rows = ops.masked_pool_rows(k_pool, G, ps, d)
    v_rows = ops.masked_pool_rows(v_pool, G, ps, dv)
    for t, slot in enumerate(slots):
        assert rel_err(k_rows[slot // ps, :, slot % ps], want_k[t]) < limit
        assert rel_err(v_rows[slot // ps, :, slot % ps], x[t, qw + kw:].view(G, dv)) < tol(dt)
    # position 0 turns nothing; elements beyond the rotated ones only pass the norm
    first = P.norm_plain(x[0, :qw].view(H, d), gq, eps)
    assert rel_err(q[0], first.reshape(qw)) < tol(dt)


# ------------------------------------------------------------------------------ short convolutions
def _conv_reference(rows, taps, unit_heads, hd, scaled, scale, before=None):
    """silu(conv) of one sequence's rows [n, C] (``before``: the rows in front of them), heads
    made unit vectors."""
    n = rows.shape[0]
    hist = taps.shape[1] - 1
    full = rows.double() if before is None else torch.cat([before.double(), rows.double()])
    y = P.silu(P.short_convolution(full, taps))[-n:]
    out = y.clone()
    for h in range(unit_heads):
        seg = P.unit(y[:, h * hd:(h + 1) * hd])
        out[:, h * hd:(h + 1) * hd] = seg * (scale if h < scaled else 1.0)
    return out


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("taps,heads,hd,plain", [(4, 4, 12, 20), (2, 2, 24, 9), (1, 3, 8, 5),
                                                 (3, 6, 32, 64), (4, 2, 70, 3)])
def test_short_convolutions_over_two_steps(dt, taps, heads, hd, plain):
    """Three requests: whole portions first (one of a single token, one shorter than the taps),
    then one left out and the others swapped with one and many tokens; slots out of order; the
    state row holds other numbers in front of the kept rows."""
    C = heads * hd + plain
    K = _rand((C, taps), 21, 0.7)
    offset, slots = 8, [3, 0, 2]
    lens = [5, 1, 2]
    more = [3, 0, 1]
    seqs = [_rand((lens[i] + more[i], C + 5), 30 + i, 1.0, dt) for i in range(3)]
    width = offset + (taps - 1) * C + 3
    state = torch.zeros((4, width), dtype=torch.float32, device=DEV)
    state[:, :offset] = 3.0
    scaled, scale = heads // 2, hd ** -0.5

    def step(parts, which, single=False):
        n = [p.shape[0] for p in parts]
        T = sum(n)
        out = torch.empty((T, C), dtype=torch.float32, device=DEV)
        ops.short_conv(torch.cat(parts).to(DEV), K.to(DEV), state, offset,
                       _i32([slots[i] for i in which]), _i32([i for i, m in enumerate(n) for _ in range(m)]),
                       _i32(_starts(n)), out, unit_heads=heads, head_dim=hd, scaled_heads=scaled,
                       scale=scale, unit_eps=1e-6, single_tokens=single)
        return out, _starts(n)

    first = [seqs[i][:lens[i]] for i in range(3)]
    out, at = step(first, [0, 1, 2])
    for i, part in enumerate(first):
        want = _conv_reference(part[:, :C], K, heads, hd, scaled, scale)
        assert rel_err(out[at[i]:at[i + 1]], want) < 2e-5
    second = [seqs[2][lens[2]:], seqs[0][lens[0]:]]
    out, at = step(second, [2, 0])
    for j, i in enumerate([2, 0]):
        want = _conv_reference(seqs[i][lens[i]:, :C], K, heads, hd, scaled, scale,
                               before=seqs[i][:lens[i], :C])
        assert rel_err(out[at[j]:at[j + 1]], want) < 2e-5
    # the kept rows: the last taps - 1 rows each request has brought (zeros before its start)
    for i in range(3):
        seen = seqs[i][:lens[i] + (more[i] if i != 1 else 0), :C].float()
        padded = torch.cat([torch.zeros((taps - 1, C)), seen])[-(taps - 1):] if taps > 1 \
            else torch.zeros((0, C))
        kept = state[slots[i], offset:offset + (taps - 1) * C].cpu().view(taps - 1, C)
        assert torch.equal(kept, padded), i
    assert float((state[:, :offset] - 3.0).abs().max()) == 0.0
    # single tokens, the state moved on by the same launch: the same numbers as in one portion
    state.zero_()
    rows = seqs[0][:, :C]
    got = []
    for t in range(rows.shape[0]):
        out, _ = step([seqs[0][t:t + 1]], [0], single=True)
        got.append(out[0].cpu())
    state.zero_()
    whole, _ = step([seqs[0]], [0])
    assert torch.equal(torch.stack(got), whole.cpu())


# ------------------------------------------------------------------------------ the delta rule
def _delta_inputs(T, H, KH, d, dv, seed):
    C = 2 * KH * d + H * dv
    qkv = _rand((T, C), seed)
    qkv[:, :2 * KH * d] = P.unit(qkv[:, :2 * KH * d].view(T, 2 * KH, d)).view(T, -1).float()
    ab = _rand((T, 2 * H), seed + 1)
    a_log = torch.linspace(-5.0, 0.5, H)
    dt_bias = _rand((H,), seed + 2)
    return qkv, ab, a_log, dt_bias


def _delta_reference(qkv, ab, a_log, dt_bias, H, KH, d, dv, state=None):
    T = qkv.shape[0]
    q = qkv[:, :KH * d].double().view(T, KH, d)
    k = qkv[:, KH * d:2 * KH * d].double().view(T, KH, d)
    v = qkv[:, 2 * KH * d:].double().view(T, H, dv)
    g = torch.exp(-torch.exp(a_log.double()) * P.softplus(ab[:, :H].double() + dt_bias.double()))
    beta = torch.sigmoid(ab[:, H:].double())
    out, last = [], []
    for n in range(H):
        c = n // (H // KH)
        o, S = P.delta_rule(q[:, c], k[:, c], v[:, n], beta[:, n], g[:, n],
                            None if state is None else state[n])
        out.append(o)
        last.append(S)
    return torch.cat(out, dim=-1), torch.stack(last)


@pytest.mark.parametrize("H,KH,d,dv", [(4, 2, 12, 10), (2, 1, 24, 14), (5, 5, 10, 6), (2, 2, 40, 12),
                                       (4, 2, 64, 64), (2, 1, 128, 32), (6, 2, 32, 48), (1, 1, 256, 5)])
def test_delta_rule_in_one_step_and_in_portions(H, KH, d, dv):
    """Three sequences of unequal length in one launch against the plain walk; then the same
    cut in two steps, in other slots' company, and token by token: the same bits, and the
    matrices left in the slots are the plain ones."""
    lens = [37, 1, 70]
    size = (ops.delta_state_size(H, d, dv) + 3) // 4 * 4 + 8
    data = [_delta_inputs(n, H, KH, d, dv, 40 + 3 * i) for i, n in enumerate(lens)]
    a_log, dt_bias = data[0][2], data[0][3]

    def run(state, parts, slots):
        n = [p[0].shape[0] for p in parts]
        qkv = torch.cat([p[0] for p in parts]).to(DEV)
        ab = torch.cat([p[1] for p in parts]).to(DEV)
        out = torch.empty((sum(n), H * dv), dtype=torch.float32, device=DEV)
        ops.delta_recurrence(qkv, 0, KH * d, 2 * KH * d, ab, a_log.to(DEV), dt_bias.to(DEV), state,
                             _i32(slots), _i32(_starts(n)), out, H, KH, d, dv)
        return out.cpu(), _starts(n)

    state = torch.zeros((5, size), dtype=torch.float32, device=DEV)
    slots = [4, 1, 2]
    whole, at = run(state, [(q, ab) for q, ab, _, _ in data], slots)
    for i, (qkv, ab, _, _) in enumerate(data):
        want, S = _delta_reference(qkv, ab, a_log, dt_bias, H, KH, d, dv)
        assert rel_err(whole[at[i]:at[i + 1]], want) < 2e-5
        got_S = ops.delta_state_matrix(state, H, d, dv)[slots[i]]
        assert rel_err(got_S, S) < 2e-5
    assert float(state[[0, 3]].abs().max()) == 0.0
    # two steps: other cuts, another order, one request left out of the second
    state2 = torch.zeros_like(state)
    cut = [20, 1, 3]
    first, at1 = run(state2, [(q[:c], ab[:c]) for (q, ab, _, _), c in zip(data, cut)], slots)
    second, at2 = run(state2, [(data[2][0][3:], data[2][1][3:]), (data[0][0][20:], data[0][1][20:])],
                      [slots[2], slots[0]])
    assert torch.equal(torch.cat([first[at1[0]:at1[1]], second[at2[1]:at2[2]]]), whole[at[0]:at[1]])
    assert torch.equal(first[at1[1]:at1[2]], whole[at[1]:at[2]])
    assert torch.equal(torch.cat([first[at1[2]:at1[3]], second[at2[0]:at2[1]]]), whole[at[2]:at[3]])
    assert torch.equal(state2, state)
    # token by token
    state3 = torch.zeros_like(state)
    qkv, ab = data[0][0], data[0][1]
    rows = [run(state3, [(qkv[t:t + 1], ab[t:t + 1])], [slots[0]])[0][0] for t in range(lens[0])]
    assert torch.equal(torch.stack(rows), whole[at[0]:at[1]])


def test_a_token_far_back_is_kept_without_decay_and_lost_with_it():
    """Two heads, 600 tokens.  Token 3 alone writes the key e_0 with a value that stands out;
    the last token asks for e_0.  The head whose decay is 1 to rounding (a rate of exp(-30))
    returns the value; the head that loses a tenth a token returns nothing of it; in one
    portion, and with the last 50 tokens alone."""
    H, KH, d, dv, T = 2, 2, 16, 8, 600
    C = 2 * KH * d + H * dv
    qkv = torch.zeros((T, C))
    e1 = torch.zeros(d)
    e1[1] = 1.0
    e0 = torch.zeros(d)
    e0[0] = 1.0
    for h in range(KH):
        qkv[:, KH * d + h * d:KH * d + (h + 1) * d] = e1        # keys elsewhere
        qkv[3, KH * d + h * d:KH * d + (h + 1) * d] = e0        # the far key
        qkv[T - 1, h * d:(h + 1) * d] = e0                      # the last query asks for it
    value = torch.arange(1.0, dv + 1.0)
    qkv[3, 2 * KH * d:2 * KH * d + dv] = value
    qkv[3, 2 * KH * d + dv:] = value
    ab = torch.zeros((T, 2 * H))
    ab[:, H:] = 30.0                                            # step size 1
    a_log = torch.tensor([-30.0, math.log(-math.log(0.9) / math.log(2.0))])
    dt_bias = torch.zeros(H)                                    # softplus(0) = log 2
    size = (ops.delta_state_size(H, d, dv) + 3) // 4 * 4
    for cuts in ([T], [T - 50] + [1] * 50):
        state = torch.zeros((1, size), dtype=torch.float32, device=DEV)
        at = 0
        for n in cuts:
            out = torch.empty((n, H * dv), dtype=torch.float32, device=DEV)
            ops.delta_recurrence(qkv[at:at + n].to(DEV), 0, KH * d, 2 * KH * d,
                                 ab[at:at + n].to(DEV), a_log.to(DEV), dt_bias.to(DEV), state,
                                 _i32([0]), _i32([0, n]), out, H, KH, d, dv)
            at += n
        last = out[-1].cpu()
        assert torch.allclose(last[:dv], value, rtol=1e-4)
        assert float(last[dv:].abs().max()) < 1e-20
    want, _ = _delta_reference(qkv, ab, a_log, dt_bias, H, KH, d, dv)
    assert rel_err(last, want[-1]) < 2e-5


# ------------------------------------------------------------------------------ the router
def _route(h, R, corr, top, groups=None, scale=1.0, gate_row=None):
    T = h.shape[0]
    ids = torch.empty((T, top), dtype=torch.int32, device=DEV)
    wts = torch.empty((T, top), dtype=torch.float32, device=DEV)
    router = R if gate_row is None else torch.cat([R, gate_row[None]])
    extra = torch.empty((T, 1), dtype=torch.float32, device=DEV) if gate_row is not None else None
    ops.moe_route(h.to(DEV), router.float().contiguous().to(DEV), None, ids, wts,
                  scoring="softmax_all", correction=corr.float().to(DEV), groups=groups,
                  group_mark=1, normalize=False, weight_scale=scale, extra=extra)
    return ids.cpu(), wts.cpu(), None if extra is None else extra.cpu()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("E,top,groups,W", [(12, 3, (3, 1), 256), (6, 2, (3, 2), 48), (4, 1, None, 72),
                                            (3, 3, (1, 1), 50), (70, 8, (7, 3), 128)])
def test_router_over_all_outputs(dt, E, top, groups, W):
    T = 41
    h = _rand((T, W), 51, 1.0, dt)
    R = _rand((E, W), 52, 3.0 / W ** 0.5)
    corr = _rand((E,), 53, 0.05)
    gate_row = _rand((W,), 54, 0.2)
    ids, wts, gate = _route(h, R, corr, top, groups, 1.7, gate_row)
    r = {"top": top, "scale": 1.7,
         "groups": None if groups is None else {"count": groups[0], "keep": groups[1]}}
    want_ids, want_w = P.route(h.double(), R, corr, r)
    same = (ids.long() == want_ids).all(dim=1)
    assert same.float().mean() > 0.9                  # (scores closer than rounding may swap)
    assert rel_err(wts[same], want_w[same]) < 2e-5
    assert rel_err(gate[:, 0], torch.sigmoid(h.double() @ gate_row.double())) < 2e-5


def test_router_by_hand():
    h = torch.eye(4)[:1]
    R = torch.tensor([[2.0, 0, 0, 0], [1.0, 0, 0, 0], [3.0, 0, 0, 0], [-4.0, 0, 0, 0]])
    s = torch.softmax(R[:, 0].double(), dim=0)
    # a correction changes the choice and not the weights
    ids, wts, _ = _route(h, R, torch.zeros(4), 2, None, 2.0)
    assert ids[0].tolist() == [2, 0] and rel_err(wts[0], 2.0 * s[[2, 0]]) < 1e-6
    ids, wts, _ = _route(h, R, torch.tensor([0.0, 1.0, 0.0, 0.0]), 2, None, 2.0)
    assert ids[0].tolist() == [1, 2] and rel_err(wts[0], 2.0 * s[[1, 2]]) < 1e-6
    # a group is marked by its largest choice score alone, and shut out although it holds the
    # best score; the weights are scores and do not add up to one
    ids, wts, _ = _route(h, R, torch.tensor([0.0, 0.0, -5.0, 0.5]), 2, (2, 1))
    assert ids[0].tolist() == [3, 2] and rel_err(wts[0], s[[3, 2]]) < 1e-6
    # with two scores a group the other group would win: 0.24 + 0.09 against 0.5
    # every choice score negative: the largest still chooses
    ids, wts, _ = _route(h, R, torch.full((4,), -9.0), 2, (2, 1))
    assert ids[0].tolist() == [2, 3] and rel_err(wts[0], s[[2, 3]]) < 1e-6
    ids, _, _ = _route(h, R, torch.full((4,), -9.0), 3, None)
    assert ids[0].tolist() == [2, 0, 1]


# ------------------------------------------------------------------------------ experts
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("T", [1, 5, 16, 300])
def test_experts_with_outputs_that_hand_their_input_on(dt, T):
    """Five experts and three router outputs without one; a token's slots name experts, such
    outputs, or both; few tokens stream their experts, many are sorted by expert (bfloat16)."""
    E, I, top, W, ff = 5, 3, 4, 64, 24
    h = _rand((T, W), 61, 1.0, dt)
    gate_up = _rand((E, 2 * ff, W), 62, 2.0 / W ** 0.5, dt)
    down = _rand((E, W, ff), 63, 2.0 / ff ** 0.5, dt)
    g = torch.Generator().manual_seed(64)
    ids = torch.stack([torch.randperm(E + I, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    ids[0] = torch.tensor([E, E + 1, E + 2, 0])          # nearly all without an expert
    if T > 1:
        ids[1] = torch.tensor([3, 1, 4, 2])              # none
    wts = torch.rand((T, top), generator=g)
    y = torch.empty((T, top, ff), dtype=dt, device=DEV)
    out = torch.full((T, W), 7.0, dtype=torch.float32, device=DEV)
    ops.moe_experts(h.to(DEV), gate_up.to(DEV), down.to(DEV), ids.to(DEV), wts.to(DEV), y, out,
                    0.0, 1.0, 0.0, add=False, n_identity=I)
    want = torch.zeros((T, W), dtype=torch.float64)
    for t in range(T):
        for e, a in zip(ids[t].tolist(), wts[t].double()):
            if e >= E:
                want[t] += a * h[t].double()
            else:
                want[t] += a * P.gated_ff(h[t:t + 1], gate_up[e, :ff], gate_up[e, ff:], down[e])[0]
    limit = 2e-5 if dt == torch.float32 else 2e-2        # (y is rounded to bfloat16 on its way)
    assert rel_err(out, want) < limit
    # added to what is there, the same numbers
    again = torch.full((T, W), 7.0, dtype=torch.float32, device=DEV)
    ops.moe_experts(h.to(DEV), gate_up.to(DEV), down.to(DEV), ids.to(DEV), wts.to(DEV), y, again,
                    0.0, 1.0, 0.0, add=True, n_identity=I)
    assert rel_err(again - 7.0, out) < 1e-5
    # a token's result does not depend on the tokens beside it
    if T == 300 and dt == torch.bfloat16:
        alone = torch.empty((20, W), dtype=torch.float32, device=DEV)
        y2 = torch.empty((20, top, ff), dtype=dt, device=DEV)
        ops.moe_grouped(h[:20].to(DEV).contiguous(), gate_up.to(DEV), down.to(DEV),
                        ids[:20].to(DEV).contiguous(), wts[:20].to(DEV).contiguous(), y2, alone,
                        0.0, 1.0, 0.0, n_identity=I)
        assert torch.equal(alone, out[:20])


@pytest.mark.parametrize("dt", DTYPES)
def test_shared_expert_gate_is_a_factor_a_row(dt):
    T, ff = 9, 20
    gu = _rand((T, 2 * ff), 71, 1.0, dt)
    factor = torch.rand((T, 3), generator=torch.Generator().manual_seed(72))
    out = torch.empty((T, ff), dtype=dt, device=DEV)
    ops.gated_act(gu.to(DEV), out, 0.0, 1.0, 0.0, row_factor=factor.to(DEV)[:, 1])
    want = P.silu(gu[:, :ff].double()) * gu[:, ff:].double() * factor[:, 1:2].double()
    assert rel_err(out, want) < tol(dt)
