"""Small Nupovik configurations for the tests, and weights made for them.  The shapes differ
from each other in every size and option: loops over several layers, over one layer, from the
first layer and from a later one, and no loop; layers without a feed-forward; dense layers
and mixtures with and without groups, with groups of one expert, with one expert chosen and
with all of them; key sizes that are no multiple of the recurrence kernel's 8 channels, one
head, value sizes below and above the key size; two latent layers in a row; widths that the
vector kernels do not take and widths the bfloat16 matrix and MFMA attention kernels take."""
from __future__ import annotations

from typing import Dict

import torch

from zinfer_amd.config import NupovikConfig
from zinfer_amd.models.build import declare_tensors


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, groups=None):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top,
                       "groups": None if groups is None else {"count": groups[0], "keep": groups[1]}}}


def _gla(heads, dim, vdim, tau, mlp, rank=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}
    if rank is not None:
        m["decay_rank"] = rank
    return {"type": "gla", "mixer": m, "mlp": mlp}


def _wkv(heads, dim, mlp, rank=None):
    m = {"heads": heads, "dim": dim}
    if rank is not None:
        m["decay_rank"] = rank
    return {"type": "wkv", "mixer": m, "mlp": mlp}


def _latent(heads, dim, vdim, kv_rank, scale, mlp):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale},
            "mlp": mlp}


# a loop over the two middle layers, three times; a mixture with groups; a latent layer
# without a feed-forward; key sizes of 12 and 20 (not multiples of 8)
NP_A = {"architecture": "Nupovik", "vocab": 211, "width": 48, "norm": {"eps": 1e-5},
        "logit_scale": 0.7, "loop": {"start": 1, "stop": 3, "times": 3},
        "layers": [_wkv(3, 12, _dense(40), rank=5),
                   _gla(2, 20, 12, 4.0, _moe(6, 2, 24, groups=(3, 2)), rank=7),
                   _latent(3, 8, 10, 24, 0.3, None),
                   _gla(4, 8, 16, 9.0, _dense(36))]}

# no loop; two latent layers in a row; one head; a mixture without groups that chooses one
# expert, one with groups of a single expert; values wider than keys
NP_B = {"architecture": "Nupovik", "vocab": 300, "width": 72, "norm": {"eps": 1e-6},
        "logit_scale": 1.0, "loop": None,
        "layers": [_latent(2, 16, 12, 40, 0.2, _moe(4, 1, 32)),
                   _latent(5, 4, 6, 20, 0.45, _dense(24)),
                   _wkv(1, 24, _moe(5, 3, 16, groups=(5, 4)), rank=3),
                   _gla(1, 16, 40, 1.0, None, rank=2),
                   _wkv(6, 4, None)]}

# a width no vector kernel takes, sizes that are no multiple of 4; a loop over the first
# layer alone; every expert chosen; no "logit_scale"
NP_C = {"architecture": "Nupovik", "vocab": 97, "width": 50, "norm": {"eps": 1e-3},
        "loop": {"start": 0, "stop": 1, "times": 2},
        "layers": [_gla(5, 10, 6, 2.5, _moe(3, 3, 14), rank=4),
                   _wkv(2, 18, _dense(30), rank=9),
                   _latent(7, 6, 5, 11, 0.6, _moe(9, 2, 10, groups=(3, 1)))]}

# widths the bfloat16 matrix kernels take, latents the MFMA attention kernels take, key sizes
# of 64 and 128; a loop up to the last layer
NP_D = {"architecture": "Nupovik", "vocab": 512, "width": 128, "norm": {"eps": 1e-6},
        "logit_scale": 1.5, "loop": {"start": 1, "stop": 5, "times": 2},
        "layers": [_latent(4, 32, 32, 64, 0.15, _dense(192)),
                   _gla(2, 64, 64, 8.0, _moe(16, 3, 64, groups=(4, 2))),
                   _wkv(2, 64, _dense(128)),
                   _latent(2, 48, 80, 128, 0.11, _moe(8, 2, 128)),
                   _gla(1, 128, 32, 32.0, _dense(64))]}

CONFIGS = {"A": NP_A, "B": NP_B, "C": NP_C, "D": NP_D}
PAGE_SIZE = {"A": 16, "B": 8, "C": 4, "D": 16}


def config_of(name: str) -> NupovikConfig:
    return NupovikConfig.from_dict(CONFIGS[name])


def weights_of(name: str, seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Weights large enough that every mechanism shows: gains around 1, decays between a
    memory of a few tokens and one of hundreds, blends between a row and the row before it,
    corrections of the size of the gaps between scores, a bonus of the size of the keys.
    Values are rounded to bfloat16 (and stored as ``dtype``), so that both compute dtypes see
    the same."""
    cfg = config_of(name)
    decls = declare_tensors(cfg.model_spec())
    g = torch.Generator().manual_seed(3000 + seed)
    out = {}
    for n, d in decls.items():
        shape = d.drawn_shape()
        last = n.split(".")[-1]
        if "norm" in n:
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif ".mu." in n:
            t = torch.rand(shape, generator=g)
        elif n.endswith("a2.b"):
            t = 2.0 + 2.0 * torch.randn(shape, generator=g)
        elif last == "w0":
            t = -2.0 + 1.5 * torch.randn(shape, generator=g)
        elif last == "u":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "correction":
            t = 0.3 * torch.randn(shape, generator=g)
        elif last == "router":
            t = torch.randn(shape, generator=g) * (4.0 / shape[-1] ** 0.5)
        elif n == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (2.0 / shape[-1] ** 0.5)
        out[n] = t.to(torch.bfloat16).to(dtype)
    return out


def tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
