"""Small Lodenex configurations for the tests, and weights made for them.  The shapes differ
from each other in every size and option: value sizes below, at and above the key size, one kv
head, as many kv heads as query heads, 20 query heads to one kv head, rotations of a part of
a head and of the whole head, with and without a rule for the frequencies, chunks and windows
of 1 token, of less than a page, of several pages and longer than any prompt, layers without a
feed-forward, widths that the vector kernels do not take, an embedding scale and caps of every
size."""
from __future__ import annotations

from typing import Dict

import torch

from zinfer_amd.config import LodenexConfig
from zinfer_amd.models.build import declare_tensors


def _attention(heads, kv, dim, vdim, chunk, scale, cap, rot_dims, base, scaling, ff):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
                      "softcap": cap, "mask": {"size": chunk},
                      "rot": {"base": base, "dims": rot_dims, "scaling": scaling}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, window, scale, base, scaling, ff):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                      "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
                      "mask": {"size": window},
                      "rot": {"base": base, "dims": rot_dim, "scaling": scaling}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _by_wavelength(factor, low, high, original):
    return {"factor": factor, "low": low, "high": high, "original": original}


def _by_turns(factor, original, fast, slow):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


# chunks and windows shorter than a page; values wider than keys; a latent layer without a
# feed-forward; frequencies that fall on every branch of their rules within 150 positions
LX_A = {"architecture": "Lodenex", "vocab": 211, "width": 48, "norm": {"eps": 1e-5},
        "embedding": {"scale": 0.7}, "logit_softcap": 9.0,
        "layers": [_attention(4, 2, 12, 20, 7, 0.31, 4.0, 8, 100.0, _by_wavelength(4.0, 1.0, 3.0, 24), 40),
                   _latent(3, 8, 4, 10, 20, 24, 5, 0.3, 50.0, _by_turns(3.0, 16, 4.0, 1.0), None),
                   _attention(2, 1, 16, 8, 11, 0.25, 30.0, 16, 10000.0, None, 36)]}

# a chunk of several pages and one longer than any prompt, a window longer than any prompt;
# kv heads = query heads; no rule for the latent layer's frequencies; two latent layers in a row;
# a layer whose scores have no cap
LX_B = {"architecture": "Lodenex", "vocab": 300, "width": 72, "norm": {"eps": 1e-6},
        "embedding": {"scale": 1.0}, "logit_softcap": 30.0,
        "layers": [_latent(2, 16, 8, 12, 40, 32, 1000, 0.2, 10000.0, None, 64),
                   _latent(5, 4, 6, 6, 12, 20, 26, 0.45, 300.0, _by_turns(8.0, 32, 16.0, 2.0), 24),
                   _attention(3, 3, 16, 16, 40, 0.25, None, 4, 1000.0, _by_wavelength(8.0, 1.0, 4.0, 64), None),
                   _attention(6, 2, 8, 12, 1000, 0.4, 2.5, 8, 20.0, _by_wavelength(2.0, 2.0, 8.0, 40), 20)]}

# 20 query heads on one kv head, sizes that are no multiple of 4, a chunk and a window of one
# token, a width the vector norm kernels do not take
LX_C = {"architecture": "Lodenex", "vocab": 97, "width": 50, "norm": {"eps": 1e-3},
        "embedding": {"scale": 2.0}, "logit_softcap": 5.0,
        "layers": [_attention(20, 1, 10, 6, 1, 0.5, 8.0, 2, 7.0, None, 30),
                   _latent(7, 6, 2, 5, 9, 11, 1, 0.6, 11.0, _by_turns(2.0, 8, 3.0, 0.5), 14),
                   _attention(1, 1, 18, 22, 33, 0.3, 12.0, 18, 500.0, _by_wavelength(16.0, 1.0, 2.0, 16), None),
                   _latent(1, 10, 10, 14, 6, 30, 17, 0.35, 80.0, None, 18)]}

# widths the bfloat16 matrix kernels take (multiples of 64), key and value widths the MFMA
# attention kernels take (with values of their own and with the keys' leading columns as values)
LX_D = {"architecture": "Lodenex", "vocab": 512, "width": 128, "norm": {"eps": 1e-6},
        "embedding": {"scale": 0.25}, "logit_softcap": 20.0,
        "layers": [_attention(4, 2, 64, 64, 48, 0.125, 15.0, 32, 10000.0, _by_wavelength(8.0, 1.0, 4.0, 128), 192),
                   _latent(4, 32, 32, 32, 64, 64, 44, 0.15, 10000.0, _by_turns(4.0, 64, 24.0, 1.0), 128),
                   _attention(8, 1, 96, 96, 100, 0.18, 25.0, 32, 250000.0, None, None),
                   _latent(2, 48, 32, 80, 112, 128, 31, 0.11, 1000.0, _by_turns(16.0, 48, 8.0, 1.0), 64)]}

CONFIGS = {"A": LX_A, "B": LX_B, "C": LX_C, "D": LX_D}
PAGE_SIZE = {"A": 16, "B": 8, "C": 4, "D": 16}


def config_of(name: str) -> LodenexConfig:
    return LodenexConfig.from_dict(CONFIGS[name])


def weights_of(name: str, seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Weights large enough that every mechanism shows: gains around 1, sinks of the size of
    the scores, gates that are neither open nor shut.  Values are rounded to bfloat16 (and
    stored as ``dtype``), so that both compute dtypes see the same."""
    cfg = config_of(name)
    decls = declare_tensors(cfg.model_spec())
    g = torch.Generator().manual_seed(2000 + seed)
    out = {}
    for n, d in decls.items():
        last = n.split(".")[-1]
        if "norm" in n:
            t = 1.0 + 0.3 * torch.randn(d.shape, generator=g)
        elif last == "sink":
            t = 1.5 * torch.randn(d.shape, generator=g)
        elif n == "embed":
            t = torch.randn(d.shape, generator=g)
        else:
            t = torch.randn(d.shape, generator=g) * (2.0 / d.shape[-1] ** 0.5)
        out[n] = t.to(torch.bfloat16).to(dtype)
    return out


def tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
