"""Small Kugisun configurations for the tests, and weights made for them.  The shapes differ
from each other in every size and option: three, one, four copies of the stream and none named;
layers that run with another layer's tensors (also through a second one that does so itself);
layers without a feed-forward; dense layers and mixtures with and without groups, with outputs
that hand their input on and without, with a shared expert and without, one group, every output
chosen; attention heads of 12, 16, 40 and 64 with values narrower and wider, all or some or none
of a head rotated, one kv head, kv heads = heads; delta-rule heads of 12, 24, 40 and 64 (every
padded size and lane count of the kernel) with one to four taps; widths that the vector kernels
do not take and widths the bfloat16 matrix and MFMA attention kernels take."""
from __future__ import annotations

from typing import Dict

import torch

from zinfer_amd.config import KugisunConfig
from zinfer_amd.models.build import declare_tensors


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, identity=None, groups=None, scale=None, shared=None):
    r = {"experts": experts, "top": top,
         "groups": None if groups is None else {"count": groups[0], "keep": groups[1]}}
    if identity is not None:
        r["identity"] = identity
    if scale is not None:
        r["scale"] = scale
    return {"kind": "moe", "expert": {"ff": ff}, "router": r,
            "shared": None if shared is None else {"ff": shared}}


def _left(heads, kv, dim, vdim, scale, rot=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return m


def _right(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def _layer(left, right, cl, cr, mlp, weights_of=None):
    L = {"type": "parallel",
         "mixer": {"left": left, "right": right, "left_scale": cl, "right_scale": cr}, "mlp": mlp}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


_A1 = _layer(_left(6, 3, 16, 8, 0.3, (16, 100.0)), _right(2, 1, 24, 14, 2), 1.0, 0.6,
             _moe(5, 2, 24, identity=1, groups=(3, 2), scale=1.5, shared=20))
# three copies; a mixture with one output that hands its input on; the last two layers run with
# layer 1's tensors, the last one through layer 2; a layer without a feed-forward
KG_A = {"architecture": "Kugisun", "vocab": 211, "width": 48, "max_positions": 512, "streams": 3,
        "norm": {"eps": 1e-5},
        "layers": [_layer(_left(4, 2, 12, 20, 0.25, (6, 1000.0)), _right(4, 2, 12, 10, 3), 0.7,
                          1.1, _dense(40)),
                   _A1,
                   _layer(_left(2, 1, 8, 8, 0.4, (8, 50.0)), _right(3, 3, 8, 6, 4), 1.2, 0.9,
                          None),
                   dict(_A1, weights_of=1),
                   dict(_A1, weights_of=3)]}

# one copy with coefficients of its own; kv heads = heads; the whole head rotated; no groups, no
# identity outputs, no shared expert; one q/k head for all value heads
KG_B = {"architecture": "Kugisun", "vocab": 300, "width": 72, "max_positions": 300, "streams": 1,
        "norm": {"eps": 1e-6},
        "layers": [_layer(_left(3, 3, 12, 12, 0.3, (12, 10000.0)), _right(4, 1, 24, 9, 2), 0.5,
                          0.5, _moe(4, 1, 32)),
                   _layer(_left(5, 1, 8, 24, 0.35, (4, 7.0)), _right(1, 1, 16, 40, 4), 1.0, 1.0,
                          _dense(24))]}

# no copies named: the plain layer; a width no vector kernel takes; one tap (no history); every
# output chosen; one group; no rotation; key sizes of 40 (padded to 48) and 10
KG_C = {"architecture": "Kugisun", "vocab": 97, "width": 50, "max_positions": 256,
        "norm": {"eps": 1e-3},
        "layers": [_layer(_left(5, 5, 10, 6, 0.3), _right(5, 5, 10, 6, 1), 0.9, 1.3,
                          _moe(2, 3, 14, identity=1, groups=(1, 1), shared=10)),
                   _layer(_left(2, 1, 40, 18, 0.15, (0, 100.0)), _right(2, 2, 40, 12, 3), 1.1,
                          0.4, _dense(30))]}

# widths the bfloat16 matrix kernels take, heads the MFMA attention kernels take; key sizes of 64
# and 128 for the delta rule; four copies; two outputs that hand their input on
_D1 = _layer(_left(4, 2, 64, 64, 0.12, (32, 250000.0)), _right(4, 2, 64, 64, 4), 1.1, 0.7,
             _moe(6, 3, 64, identity=2, groups=(4, 2), scale=1.5, shared=192))
KG_D = {"architecture": "Kugisun", "vocab": 512, "width": 128, "max_positions": 1024, "streams": 4,
        "norm": {"eps": 1e-6},
        "layers": [_layer(_left(2, 2, 128, 128, 0.09, (128, 10000.0)), _right(2, 1, 128, 32, 4),
                          1.0, 1.0, _dense(256)),
                   _D1, dict(_D1, weights_of=1),
                   _layer(_left(4, 1, 96, 96, 0.1, (48, 1000.0)), _right(8, 8, 32, 16, 2), 0.6,
                          1.2, _dense(192))]}

CONFIGS = {"A": KG_A, "B": KG_B, "C": KG_C, "D": KG_D}
PAGE_SIZE = {"A": 16, "B": 8, "C": 4, "D": 16}


def config_of(name: str) -> KugisunConfig:
    return KugisunConfig.from_dict(CONFIGS[name])


def weights_of(name: str, seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Weights large enough that every mechanism shows: norm weights around zero of a size
    that matters, biases of the size of the projections, stream coefficients that mix the
    copies, decays between a memory of a few tokens and one of hundreds, taps of order one,
    corrections of the size of the gaps between scores.  Values are rounded to bfloat16 (and
    stored as ``dtype``), so that both compute dtypes see the same."""
    cfg = config_of(name)
    decls = declare_tensors(cfg.model_spec())
    g = torch.Generator().manual_seed(7000 + seed)
    out = {}
    for n, d in decls.items():
        if d.optional:                       # (a head of its own: the design's is the embedding)
            continue
        shape = d.drawn_shape()
        last = n.split(".")[-1]
        if last in ("norm1", "norm2") or n == "final.norm":
            t = 0.3 * torch.randn(shape, generator=g)
        elif last == "norm":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif ".hc" in n and last == "mix":
            t = torch.eye(shape[0]) + 0.2 * torch.randn(shape, generator=g)
        elif ".hc" in n:
            t = (1.0 if last == "out" else 1.0 / shape[0] ** 0.5) + 0.3 * torch.randn(shape, generator=g)
        elif last == "A_log":
            # from a memory of a few tokens to one of hundreds
            t = torch.linspace(-6.0, 0.5, shape[0]) + 0.2 * torch.randn(shape, generator=g)
        elif last == "dt_bias":
            t = torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.7 * torch.randn(shape, generator=g)
        elif last == "correction":
            t = 0.05 * torch.randn(shape, generator=g)
        elif last == "router":
            t = torch.randn(shape, generator=g) * (3.0 / shape[-1] ** 0.5)
        elif n.endswith(".b") and ".left." in n:
            t = 0.5 * torch.randn(shape, generator=g)
        elif n in ("embed", "pos"):
            t = torch.randn(shape, generator=g) * (1.0 if n == "embed" else 0.5)
        else:
            t = torch.randn(shape, generator=g) * (2.0 / shape[-1] ** 0.5)
        out[n] = t.to(torch.bfloat16).to(dtype)
    return out


def tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
