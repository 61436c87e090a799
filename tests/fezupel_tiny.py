"""Small Fezupel configurations for the tests, and weights made for them.  The shapes differ
from each other in every size and option: looped and unlooped layers, layers without a
feed-forward, one kv head, as many kv heads as query heads, more than 16 query heads to a kv
head, windows of 1 token, of less than a page, of several pages and longer than any prompt,
one expert, all experts chosen, a shared expert or none."""
from __future__ import annotations

from typing import Dict

import torch

from zinfer_amd.config import FezupelConfig
from zinfer_amd.models.build import declare_tensors


def _layer(heads, kv, dim, window, scale, mlp):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale,
                      "mask": {"size": window}},
            "mlp": mlp}


def _moe(experts, top, ff, limit, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top},
            "expert": {"ff": ff, "limit": limit},
            "shared": None if shared is None else {"ff": shared[0], "limit": shared[1]}}


# two layers, the first one run three times; windows shorter than a page
FZ_A = {"architecture": "Fezupel", "vocab": 211, "width": 48, "max_positions": 160,
        "norm": {"eps": 1e-5}, "loop": {"start": 0, "stop": 1, "times": 3},
        "layers": [_layer(4, 2, 12, 7, 0.31, _moe(6, 2, 20, 0.4, (28, 0.9))),
                   _layer(2, 1, 24, 5, 0.2, _moe(5, 1, 36, 0.25))]}

# three layers that all differ; the second has no feed-forward; a window of several pages and
# one longer than any prompt; every expert chosen; no loop at all
FZ_B = {"architecture": "Fezupel", "vocab": 300, "width": 72, "max_positions": 256,
        "norm": {"eps": 1e-6},
        "layers": [_layer(3, 3, 16, 40, 0.25, _moe(3, 3, 24, 0.5)),
                   _layer(6, 2, 8, 1000, 0.4, None),
                   _layer(2, 2, 40, 17, 0.15, _moe(9, 4, 16, 0.3, (8, 0.2)))]}

# one layer: 20 query heads on one kv head, a head size that is no multiple of 4, a window of
# one token, one expert; a loop over no layer, and a second configuration run once
FZ_C = {"architecture": "Fezupel", "vocab": 97, "width": 50, "max_positions": 96,
        "norm": {"eps": 1e-3}, "loop": {"start": 1, "stop": 1, "times": 4},
        "layers": [_layer(20, 1, 10, 1, 0.5, _moe(1, 1, 30, 0.6, (12, 0.5))),
                   _layer(1, 1, 18, 33, 0.3, _moe(70, 66, 8, 0.8))]}

# widths the bfloat16 matrix kernels take (multiples of 64), the middle layers run twice
FZ_D = {"architecture": "Fezupel", "vocab": 512, "width": 128, "max_positions": 320,
        "norm": {"eps": 1e-6}, "loop": {"start": 1, "stop": 3, "times": 2},
        "layers": [_layer(4, 2, 64, 48, 0.125, _moe(8, 2, 64, 1.0, (128, 1.5))),
                   _layer(2, 2, 32, 16, 0.2, _moe(4, 2, 128, 0.7)),
                   _layer(8, 1, 32, 100, 0.18, None),
                   _layer(4, 4, 32, 31, 0.2, _moe(16, 3, 64, 0.5, (64, 0.5)))]}

CONFIGS = {"A": FZ_A, "B": FZ_B, "C": FZ_C, "D": FZ_D}
PAGE_SIZE = {"A": 16, "B": 8, "C": 4, "D": 16}


def config_of(name: str) -> FezupelConfig:
    return FezupelConfig.from_dict(CONFIGS[name])


def weights_of(name: str, seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Weights large enough that every mechanism shows: gains around 1, biases of some tenths,
    products that reach the experts' limits, router logits that differ by tenths.  Values are
    rounded to bfloat16 (and stored as ``dtype``), so that both compute dtypes see the same."""
    cfg = config_of(name)
    decls = declare_tensors(cfg.model_spec())
    g = torch.Generator().manual_seed(1000 + seed)
    out = {}
    for n, d in decls.items():
        last = n.split(".")[-1]
        if "norm" in n and last != "b":
            t = 1.0 + 0.3 * torch.randn(d.shape, generator=g)
        elif last == "b":
            t = 0.3 * torch.randn(d.shape, generator=g)
        elif n in ("embed", "pos"):
            t = torch.randn(d.shape, generator=g)
        else:
            t = torch.randn(d.shape, generator=g) * (2.0 / d.shape[-1] ** 0.5)
        out[n] = t.to(torch.bfloat16).to(dtype)
    return out


def tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
