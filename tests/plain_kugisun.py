"""Plain, slow implementation of the Kugisun decoder: whole sequences, no cache, one function
for each mechanism, float64 arithmetic on the CPU.  It shares no code with the engine under
``zinfer_amd/``: it is the oracle the engine is compared with.

The design in this file's own notation (p: a token's position, counted from 0; h: what a
sublayer reads; X_1 .. X_S: the S copies of the residual stream, each [T, W]):

  embedding:   e_p = E[token_p] + P[p];  X_s = e for every s
  order:       the layers as listed; a layer that names another's weights runs with those
               (mixer, feed-forward, norms, stream coefficients) and a cache and state of its own
  sublayer c:  u = sum_s a_c[s] X_s;  y = f_c(N_c(u));  X_t <- sum_s M_c[s, t] X_s + b_c[t] y
               (all t from the old X; c = 1: the mixer, c = 2: the feed-forward, if there is one)
  N(v)       = v / sqrt(mean v^2 + eps) * (1 + w)
  mixer:       c_l * attention(h) + c_r * delta(h)
  attention:   q = Wq h + bq, k = Wk h + bk, v = Wv h + bv;  q, k <- n(q), n(k) a head with
               n(v) = v / sqrt(mean v^2 + eps) * w;  the pairs (2i, 2i + 1), i < r / 2, of every
               q and k head turn by the angle p * base^(-2i / r);  a = softmax_j<=i(scale q_i . k_j);
               out = Wo [heads of sum_j a_ij v_j];  query head n reads kv head floor(n / (H / G))
  delta:       q, k, v = silu(conv(W h)): conv(x)_t[c] = sum_j K[c, j] x_(t - taps + 1 + j)[c],
               zeros before the start;  q, k <- unit(q), unit(k) a head with
               unit(v) = v / sqrt(sum v^2 + 1e-6);  q <- q / sqrt(d)
               beta = sigmoid(Wb h), g = exp(-exp(A) softplus(Wa h + dt))    one a head and token
               S <- g S;  w = beta (v - S^T k);  S <- S + k w^T;  o = S^T q   (S is [d, dv], from 0)
               out = Wo [heads of o / sqrt(mean o^2 + eps) * w_n * silu(Wg h)]
               value head n reads q/k head floor(n / (heads / kv_heads))
  ff dense:    Wd (silu(Wg h) * (Wu h))
  ff moe:      s = softmax(R h) over the E experts and the I identity experts behind them;
               c = s + correction;  groups of neighbours, a group's mark = its largest c, outside
               the best ``keep`` groups c = -inf;  the ``top`` largest c choose;  weight s_e * scale;
               an identity expert's output is h;  + sigmoid(w_sg . h) * shared(h)
  logits     = E N_final(sum_s X_s)
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64
UNIT_EPS = 1e-6


# ----------------------------------------------------------------------------- small pieces
def linear(w: torch.Tensor, h: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """W stored [out, in], applied to every row of h."""
    y = h.to(F64) @ w.to(F64).T
    return y if b is None else y + b.to(F64)


def rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    v = v.to(F64)
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The layers' norm: the weight is stored around zero."""
    return rms(v, eps) * (1.0 + w.to(F64))


def norm_plain(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(v, eps) * w.to(F64)


def unit(v: torch.Tensor) -> torch.Tensor:
    v = v.to(F64)
    return v / torch.sqrt((v * v).sum(dim=-1, keepdim=True) + UNIT_EPS)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, d]: of every head the pairs (2i, 2i + 1), i < dims / 2, turn by
    positions * base^(-2i / dims); the elements from ``dims`` on pass unchanged."""
    out = x.to(F64).clone()
    p = positions.to(F64)
    for i in range(dims // 2):
        a = p * base ** (-2.0 * i / dims)
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., 2 * i].to(F64), x[..., 2 * i + 1].to(F64)
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def short_convolution(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: y_t = sum_j taps[:, j] * x_(t - n + 1 + j), zeros before t = 0."""
    T, C = x.shape
    n = taps.shape[1]
    padded = torch.cat([torch.zeros((n - 1, C), dtype=F64), x.to(F64)], dim=0)
    y = torch.zeros((T, C), dtype=F64)
    for j in range(n):
        y += padded[j:j + T] * taps[:, j].to(F64)
    return y


# ----------------------------------------------------------------------------- the two mixers
def attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float,
              start: int = 0) -> torch.Tensor:
    """``w``: the tensors below '<layer>.mix.left.'; ``m``: the config's 'left'."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(start, start + T)
    q = linear(w["q"], h, w["q.b"]).view(T, H, d)
    k = linear(w["k"], h, w["k.b"]).view(T, G, d)
    v = linear(w["v"], h, w["v.b"]).view(T, G, dv)
    q = norm_plain(q, w["q.norm"], eps)
    k = norm_plain(k, w["k.norm"], eps)
    rot = m.get("rot")
    if rot is not None and rot["dims"] > 0:
        q = rotate_pairs(q, pos, rot["dims"], float(rot["base"]))
        k = rotate_pairs(k, pos, rot["dims"], float(rot["base"]))
    seen = torch.tril(torch.ones((T, T), dtype=torch.bool))
    heads = []
    for n in range(H):
        g = n // (H // G)
        s = (q[:, n] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(~seen, -math.inf)
        heads.append(torch.softmax(s, dim=-1) @ v[:, g])
    return linear(w["o"], torch.cat(heads, dim=-1))


def delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor,
               g: torch.Tensor, state: Optional[torch.Tensor] = None):
    """One head.  q, k [T, d], v [T, dv], beta, g [T].  Returns o [T, dv] and the last S."""
    T, d = q.shape
    S = torch.zeros((d, v.shape[1]), dtype=F64) if state is None else state.clone()
    out = []
    for t in range(T):
        S = g[t] * S
        w = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], w)
        out.append(S.T @ q[t])
    return torch.stack(out), S


def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """``w``: the tensors below '<layer>.mix.right.'; ``m``: the config's 'right'."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(linear(w["q"], h), w["q.conv"])).view(T, G, d)
    k = silu(short_convolution(linear(w["k"], h), w["k.conv"])).view(T, G, d)
    v = silu(short_convolution(linear(w["v"], h), w["v.conv"])).view(T, H, dv)
    q = unit(q) * d ** -0.5
    k = unit(k)
    beta = torch.sigmoid(linear(w["b"], h))
    g = torch.exp(-torch.exp(w["A_log"].to(F64)) * softplus(linear(w["a"], h) + w["dt_bias"].to(F64)))
    gate = silu(linear(w["g"], h)).view(T, H, dv)
    heads = []
    for n in range(H):
        c = n // (H // G)
        o, _ = delta_rule(q[:, c], k[:, c], v[:, n], beta[:, n], g[:, n])
        heads.append(norm_plain(o, w["norm"], eps) * gate[:, n])
    return linear(w["o"], torch.cat(heads, dim=-1))


def parallel_mixer(h, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """``w``: the tensors below '<layer>.mix.'."""
    left = {n[5:]: t for n, t in w.items() if n.startswith("left.")}
    right = {n[6:]: t for n, t in w.items() if n.startswith("right.")}
    return float(m["left_scale"]) * attention(h, left, m["left"], eps) \
        + float(m["right_scale"]) * delta_mixer(h, right, m["right"], eps)


# ----------------------------------------------------------------------------- feed-forwards
def gated_ff(h, gate, up, down) -> torch.Tensor:
    return linear(down, silu(linear(gate, h)) * linear(up, h))


def route(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, r: dict):
    """Per token the chosen outputs of the router (ids [T, top]) and their weights."""
    s = torch.softmax(linear(router, h), dim=-1)
    c = s + correction.to(F64)
    n = c.shape[1]
    groups = r.get("groups")
    if groups is not None:
        count, keep = groups["count"], groups["keep"]
        size = n // count
        marks = c.view(-1, count, size).max(dim=-1).values
        best = torch.topk(marks, keep, dim=-1).indices
        kept = torch.zeros_like(marks, dtype=torch.bool).scatter_(1, best, True)
        c = c.masked_fill(~kept.repeat_interleave(size, dim=1), -math.inf)
    ids = torch.topk(c, r["top"], dim=-1).indices
    return ids, torch.gather(s, 1, ids) * float(r.get("scale", 1.0))


def mixture(h: torch.Tensor, w: Dict[str, torch.Tensor], f: dict) -> torch.Tensor:
    """``w``: the tensors below '<layer>.mlp.'; ``f``: the config's 'mlp'."""
    r = f["router"]
    E = r["experts"]
    h = h.to(F64)
    ids, weights = route(h, w["router"], w["correction"], r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), weights[t]):
            if e >= E:                       # an identity expert
                out[t] += a * h[t]
            else:
                out[t] += a * gated_ff(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"],
                                       w[f"e{e}.down"])[0]
    if f.get("shared") is not None:
        sg = torch.sigmoid(linear(w["shared.sg"], h))
        out = out + sg * gated_ff(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out


def feed_forward(h, w: Dict[str, torch.Tensor], f: dict) -> torch.Tensor:
    if f["kind"] == "dense":
        return gated_ff(h, w["gate"], w["up"], w["down"])
    return mixture(h, w, f)


# ----------------------------------------------------------------------------- the model
def below(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}


def weights_layer(config: dict, i: int) -> int:
    """The layer whose tensors layer i runs with."""
    while config["layers"][i].get("weights_of") is not None:
        i = config["layers"][i]["weights_of"]
    return i


def stream_step(X: List[torch.Tensor], w: Dict[str, torch.Tensor], c: int, sublayer):
    """One sublayer over the streams X; ``w``: a layer's tensors; returns the new streams."""
    S = len(X)
    a, M, b = w.get(f"hc{c}.in"), w.get(f"hc{c}.mix"), w.get(f"hc{c}.out")
    if a is None:                            # one stream and no coefficients: the plain sum
        return [X[0] + sublayer(X[0])]
    u = sum(float(a[s]) * X[s] for s in range(S))
    y = sublayer(u)
    return [sum(float(M[s, t]) * X[s] for s in range(S)) + float(b[t]) * y for t in range(S)]


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens, layers_out=None):
    """Logits [T, vocab] (float64) of one whole sequence; ``layers_out``: a list that takes the
    sum of the streams after every run of a layer."""
    eps = float(config["norm"]["eps"])
    T = len(tokens)
    e = tensors["embed"].to(F64)[torch.tensor(list(tokens))] + tensors["pos"].to(F64)[:T]
    X = [e.clone() for _ in range(int(config.get("streams", 1)))]
    for i, L in enumerate(config["layers"]):
        j = weights_layer(config, i)
        L = config["layers"][j]
        w = below(tensors, f"l{j}.")
        mix = below(w, "mix.")
        X = stream_step(X, w, 1, lambda u: parallel_mixer(norm_one_plus(u, w["norm1"], eps), mix,
                                                          L["mixer"], eps))
        if L.get("mlp") is not None:
            mlp = below(w, "mlp.")
            X = stream_step(X, w, 2, lambda u: feed_forward(norm_one_plus(u, w["norm2"], eps), mlp,
                                                            L["mlp"]))
        if layers_out is not None:
            layers_out.append(sum(X))
    x = norm_one_plus(sum(X), tensors["final.norm"], eps)
    return linear(tensors["embed"], x)
