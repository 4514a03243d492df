"""Plain, slow implementation of the Nupovik decoder: whole sequences, no cache, one function
for each mechanism, float64 arithmetic on the CPU.  It shares no code with the engine under
``zinfer_amd/``: it is the oracle the engine is compared with.

The design in this file's own notation (x: the residual stream of one sequence, [T, W];
p: a token's position, counted from 0; h: what a sublayer reads):

  x_p        = E[token_p] + pe(p);  pe(p)[2i] = sin(p b^(-2i/W)), pe(p)[2i+1] = cos(same), b = 10^4
  order:       layers before ``start`` once, layers start..stop-1 ``times`` times, the rest once;
               a pass begins with x = W_in [x ; x_0]  (x_0: the stream as the embedding left it)
  layer:       x += mix(N_1(x)) + ff(N_2(x))            both sublayers read the same x
  N(v)       = v / sqrt(mean v^2 + eps) * w
  'gla':       q = Wq h / sqrt(d), k = Wk h, v = Wv h, a = sigmoid(Wa2 Wa1 h + b)^(1/tau)
               S_t = diag(a_t) S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t      (a head: S is [d, dv])
               mix = Wo (N_head(o) * silu(Wg h))         N_head over dv, one gain for all heads
  'latent_attention':
               q = Wq h;  c = N_c(Wdkv h);  k_h = Wuk c, v_h = Wuv c
               a = softmax_j<=i(scale q_i . k_j);  mix = Wo ((sum_j a_ij v_j) * sigmoid(Wg h)_h)
  'wkv':       m_s = h + (h_prev - h) * mu_s  for s in r, k, v, g, w   (h_prev = 0 at p = 0)
               r, k, v = W_s m_s;  g = silu(Wg m_g);  w = exp(-exp(Ww2 tanh(Ww1 m_w) + w0))
               o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t;  S_t = diag(w_t) S_(t-1) + k_t v_t^T
               mix = Wo (o / rms_head(o) * gain * g)
  ff dense:    Wdown relu(Wup h)^2
  ff moe:      s = sigmoid(R h);  c = s + correction;  experts in G equal groups of neighbours,
               a group's mark = its two largest c added; outside the best ``keep`` groups c = -inf;
               the ``top`` largest c choose; weights s_e / (sum of chosen s + 1e-20)
  logits     = H N_final(x) * logit_scale
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64
POSITION_BASE = 10000.0


# ----------------------------------------------------------------------------- small pieces
def rms_norm(v: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    v = v.to(F64)
    out = v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return out if w is None else out * w.to(F64)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def relu_squared(z: torch.Tensor) -> torch.Tensor:
    return torch.clamp(z, min=0.0) ** 2


def linear(w: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
    """W stored [out, in], applied to every row of h."""
    return h.to(F64) @ w.to(F64).T


def position_vectors(T: int, width: int, start: int = 0) -> torch.Tensor:
    """[T, width]: entry 2i is sin(p f_i), entry 2i + 1 cos(p f_i), f_i = base^(-2i / width)."""
    out = torch.zeros((T, width), dtype=F64)
    p = torch.arange(start, start + T, dtype=F64)[:, None]
    for i in range((width + 1) // 2):
        f = POSITION_BASE ** (-2.0 * i / width)
        out[:, 2 * i] = torch.sin(p[:, 0] * f)
        if 2 * i + 1 < width:
            out[:, 2 * i + 1] = torch.cos(p[:, 0] * f)
    return out


def layer_order(n_layers: int, loop: Optional[dict]) -> List[tuple]:
    """(layer, whether a pass begins before it) for every run, in order."""
    if loop is None:
        return [(i, False) for i in range(n_layers)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n_layers)]


# ----------------------------------------------------------------------------- recurrences
def decayed_outer_recurrence(q, k, v, decay, bonus=None, state=None):
    """One head.  q, k, decay [T, d]; v [T, dv]; S [d, dv] starts at ``state`` or zero.
    Without ``bonus``: S_t = diag(decay_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.
    With ``bonus`` u [d]: o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t, then S_t as above.
    Returns (o [T, dv], S after the last token)."""
    T, d = q.shape
    dv = v.shape[1]
    S = torch.zeros((d, dv), dtype=F64) if state is None else state.to(F64).clone()
    o = torch.zeros((T, dv), dtype=F64)
    for t in range(T):
        kv = torch.outer(k[t], v[t])
        if bonus is None:
            S = decay[t][:, None] * S + kv
            o[t] = S.T @ q[t]
        else:
            o[t] = (S + bonus[:, None] * kv).T @ q[t]
            S = decay[t][:, None] * S + kv
    return o, S


def gla_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    heads, d = int(m["heads"]), int(m["dim"])
    dv, tau = int(m["vdim"]), float(m["tau"])
    h = h.to(F64)
    T = h.shape[0]
    q = (linear(w["q"], h) * d ** -0.5).view(T, heads, d)
    k = linear(w["k"], h).view(T, heads, d)
    v = linear(w["v"], h).view(T, heads, dv)
    z = linear(w["a2"], linear(w["a1"], h)) + w["a2.b"].to(F64)
    alpha = torch.sigmoid(z).pow(1.0 / tau).view(T, heads, d)
    o = torch.zeros((T, heads, dv), dtype=F64)
    for i in range(heads):
        o[:, i], _ = decayed_outer_recurrence(q[:, i], k[:, i], v[:, i], alpha[:, i])
    o = rms_norm(o, w["norm"], eps).reshape(T, heads * dv)
    return linear(w["o"], o * silu(linear(w["g"], h)))


def token_shift(h: torch.Tensor, mu: torch.Tensor, before: Optional[torch.Tensor] = None):
    """h + (h_prev - h) * mu; the row before the first is ``before`` or zero."""
    h = h.to(F64)
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    if before is not None:
        prev[0] = before.to(F64)
    return h + (prev - h) * mu.to(F64)


def wkv_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    heads, d = int(m["heads"]), int(m["dim"])
    h = h.to(F64)
    T = h.shape[0]
    mix = {s: token_shift(h, w["mu." + s]) for s in "rkvgw"}
    r = linear(w["r"], mix["r"]).view(T, heads, d)
    k = linear(w["k"], mix["k"]).view(T, heads, d)
    v = linear(w["v"], mix["v"]).view(T, heads, d)
    gate = silu(linear(w["g"], mix["g"]))
    z = linear(w["w2"], torch.tanh(linear(w["w1"], mix["w"]))) + w["w0"].to(F64)
    decay = torch.exp(-torch.exp(z)).view(T, heads, d)
    u = w["u"].to(F64).view(heads, d)
    o = torch.zeros((T, heads, d), dtype=F64)
    for i in range(heads):
        o[:, i], _ = decayed_outer_recurrence(r[:, i], k[:, i], v[:, i], decay[:, i], bonus=u[i])
    o = rms_norm(o, None, eps).reshape(T, heads * d) * w["norm"].to(F64)
    return linear(w["o"], o * gate)


# ----------------------------------------------------------------------------- attention
def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict,
                           eps: float) -> torch.Tensor:
    heads, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    scale = float(m["scale"])
    h = h.to(F64)
    T = h.shape[0]
    q = linear(w["q"], h).view(T, heads, d)
    c = rms_norm(linear(w["dkv"], h), w["dkv.norm"], eps)
    k = linear(w["uk"], c).view(T, heads, d)
    v = linear(w["uv"], c).view(T, heads, dv)
    gate = torch.sigmoid(linear(w["g"], h))                    # [T, heads]
    seen = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    out = torch.zeros((T, heads, dv), dtype=F64)
    for i in range(heads):
        s = (q[:, i] @ k[:, i].T) * scale
        s = s.masked_fill(~seen, -math.inf)
        a = torch.softmax(s, dim=-1)
        out[:, i] = (a @ v[:, i]) * gate[:, i:i + 1]
    return linear(w["o"], out.reshape(T, heads * dv))


# ----------------------------------------------------------------------------- feed-forward
def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return linear(w["down"], relu_squared(linear(w["up"], h)))


def route(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, r: dict):
    """(chosen experts [T, top], their weights [T, top], in the order they were chosen)."""
    experts, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(linear(router, h))                        # [T, E]
    c = s + correction.to(F64)
    groups = r.get("groups")
    if groups is not None:
        count, keep = int(groups["count"]), int(groups["keep"])
        size = experts // count
        per = c.view(-1, count, size)
        mark = per.topk(min(2, size), dim=-1).values.sum(dim=-1)       # [T, count]
        kept = torch.zeros_like(mark, dtype=torch.bool)
        kept.scatter_(1, mark.topk(keep, dim=-1).indices, True)
        c = c.masked_fill(~kept[:, :, None].expand(-1, -1, size).reshape(-1, experts), -math.inf)
    chosen = c.topk(top, dim=-1).indices
    picked = s.gather(1, chosen)
    return chosen, picked / (picked.sum(dim=-1, keepdim=True) + 1e-20)


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], f: dict) -> torch.Tensor:
    h = h.to(F64)
    chosen, weights = route(h, w["router"], w["correction"], f["router"])
    out = torch.zeros((h.shape[0], w["e0.down"].shape[0]), dtype=F64)
    for t in range(h.shape[0]):
        for e, c in zip(chosen[t].tolist(), weights[t].tolist()):
            y = relu_squared(linear(w[f"e{e}.up"], h[t:t + 1]))
            out[t] += c * linear(w[f"e{e}.down"], y)[0]
    return out


# ----------------------------------------------------------------------------- the model
def _under(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


MIXERS = {"gla": gla_mixer, "latent_attention": latent_attention_mixer, "wkv": wkv_mixer}


def layer(x: torch.Tensor, tensors: Dict[str, torch.Tensor], i: int, L: dict, eps: float):
    p = f"l{i}."
    out = MIXERS[L["type"]](rms_norm(x, tensors[p + "norm1"], eps), _under(tensors, p + "mix."),
                            L["mixer"], eps)
    f = L.get("mlp")
    if f is not None:
        h = rms_norm(x, tensors[p + "norm2"], eps)
        w = _under(tensors, p + "mlp.")
        out = out + (dense_ff(h, w) if f["kind"] == "dense" else moe_ff(h, w, f))
    return x + out


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens: Sequence[int],
            streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0.  ``streams`` (a list) receives the
    residual stream after every run of a layer."""
    eps = float(config["norm"]["eps"])
    width = int(config["width"])
    ids = torch.tensor(list(tokens), dtype=torch.long)
    x = tensors["embed"].to(F64)[ids] + position_vectors(len(ids), width)
    x0 = x.clone()
    for i, begins in layer_order(len(config["layers"]), config.get("loop")):
        if begins:
            x = linear(tensors["loop.in"], torch.cat([x, x0], dim=-1))
        x = layer(x, tensors, i, config["layers"][i], eps)
        if streams is not None:
            streams.append(x.clone())
    x = rms_norm(x, tensors["final.norm"], eps)
    return linear(tensors["head"], x) * float(config.get("logit_scale", 1.0))
