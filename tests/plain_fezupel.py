"""Plain, slow implementation of the Fezupel decoder: whole sequences, no cache, one function
for each mechanism, float64 arithmetic on the CPU.  It shares no code with the engine under
``zinfer_amd/``: it is the oracle the engine is compared with.

The design in this file's own notation (x: the residual stream of one sequence, [T, W]):

  x_t      = E[token_t] + P[t]                                   learned position, unscaled
  layer:     x += LN_1b(mix(LN_1(x)));  x += LN_2b(ff(LN_2(x)))  (no second line without ff)
  LN(v)    = (v - mean v) / sqrt(mean (v - mean v)^2 + eps) * w + b
  mix(h):    q = Wq h, k = Wk h, v = k (the keys are the values)
             s_ij = scale * q_i . k_j   for i - window < j <= i
             a_ij = exp(s_ij) / (1 + sum_j exp(s_ij))            one more, silent term of score 0
             o_i  = sum_j a_ij k_j;  mix = Wo (o * sigmoid(Wg h))
  ff(h):     z = Wr h + br;  S = the ``top`` largest of z;  c = softmax(z[S])
             ff = sum_{e in S} c_e expert_e(h) + shared(h)
  expert(h): g = min(Wgate h, L), u = clamp(Wup h, -L, L);  Wdown (g sigmoid(1.702 g) (u + 1))
  a range of layers may run several times in a row with the same weights
  logits   = H LN_final(x)
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64


def layer_norm(v: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    v = v.to(F64)
    mean = v.mean(dim=-1, keepdim=True)
    dev = v - mean
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * w.to(F64) + b.to(F64)


def sink_window_attention(q: torch.Tensor, k: torch.Tensor, n_heads: int, n_kv: int, dim: int,
                          scale: float, window: int) -> torch.Tensor:
    """q [T, n_heads * dim], k [T, n_kv * dim] (also the values) -> [T, n_heads * dim]."""
    T = q.shape[0]
    q = q.to(F64).view(T, n_heads, dim)
    k = k.to(F64).view(T, n_kv, dim)
    out = torch.zeros((T, n_heads, dim), dtype=F64)
    per = n_heads // n_kv
    for i in range(T):
        lo = max(0, i - window + 1)
        for h in range(n_heads):
            keys = k[lo:i + 1, h // per]                       # [n, dim]
            s = (keys @ q[i, h]) * scale
            e = torch.exp(s)
            a = e / (1.0 + e.sum())
            out[i, h] = a @ keys
    return out.view(T, n_heads * dim)


def gated_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    h = h.to(F64)
    q = h @ w[p + "q"].to(F64).T
    k = h @ w[p + "k"].to(F64).T
    o = sink_window_attention(q, k, m["heads"], m["kv_heads"], m["dim"], float(m["scale"]),
                              int(m["mask"]["size"]))
    gate = torch.sigmoid(h @ w[p + "g"].to(F64).T)
    return (o * gate) @ w[p + "o"].to(F64).T


def clamped_expert(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, limit: float) -> torch.Tensor:
    h = h.to(F64)
    g = torch.clamp(h @ w[p + "gate"].to(F64).T, max=limit)
    u = torch.clamp(h @ w[p + "up"].to(F64).T, min=-limit, max=limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return y @ w[p + "down"].to(F64).T


def route(h: torch.Tensor, w_router: torch.Tensor, b_router: torch.Tensor, top: int):
    """(chosen experts [T, top], their weights [T, top])."""
    z = h.to(F64) @ w_router.to(F64).T + b_router.to(F64)
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def moe_feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, f: dict) -> torch.Tensor:
    idx, c = route(h, w[p + "router"], w[p + "router.b"], int(f["router"]["top"]))
    out = torch.zeros((h.shape[0], w[p + "e0.down"].shape[0]), dtype=F64)
    for e in range(int(f["router"]["experts"])):
        share = (c * (idx == e)).sum(dim=-1, keepdim=True)          # 0 where e was not chosen
        rows = (share[:, 0] > 0).nonzero()[:, 0]
        if len(rows):
            out[rows] += share[rows] * clamped_expert(h[rows], w, f"{p}e{e}.",
                                                      float(f["expert"]["limit"]))
    if f.get("shared") is not None:
        out += clamped_expert(h, w, p + "shared.", float(f["shared"]["limit"]))
    return out


def layer_order(config: dict) -> List[int]:
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(config: dict, w: Dict[str, torch.Tensor], tokens: Sequence[int],
            streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0; ``streams`` (a list) receives the
    residual stream after every run of a layer."""
    eps = float(config["norm"]["eps"])
    T = len(tokens)
    x = w["embed"].to(F64)[list(tokens)] + w["pos"].to(F64)[:T]
    for i in layer_order(config):
        L, p = config["layers"][i], f"l{i}."
        assert L["type"] == "attention"
        h = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
        y = gated_attention_mixer(h, w, p + "mix.", L["mixer"])
        x = x + layer_norm(y, w[p + "norm1b"], w[p + "norm1b.b"], eps)
        if L.get("mlp") is not None:
            h = layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps)
            y = moe_feed_forward(h, w, p + "mlp.", L["mlp"])
            x = x + layer_norm(y, w[p + "norm2b"], w[p + "norm2b.b"], eps)
        if streams is not None:
            streams.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return x @ w["head"].to(F64).T
