"""Plain, slow implementation of the Lodenex decoder: whole sequences, no cache, one function
for each mechanism, float64 arithmetic on the CPU.  It shares no code with the engine under
``zinfer_amd/``: it is the oracle the engine is compared with.

The design in this file's own notation (x: the residual stream of one sequence, [T, W];
p: a token's position, counted from 0):

  x_p       = E[token_p] * embedding scale
  layer:      x += N_1(mix(x));  x += N_2(ff(x))       the sublayers read x as it is; the norm
                                                        stands behind them (no second line
                                                        without ff)
  N(v)      = v / sqrt(mean v^2 + eps) * w
  rot(u, p):  on the first ``dims`` elements of a head, pairs (i, i + dims/2):
              (a, b) -> (a cos t - b sin t, b cos t + a sin t) * mag,  t = p * f_i
  'attention' mixer:
              q = N_q(Wq h), k = N_k(Wk h) over the whole projection, v = Wv h
              s_ij = cap * tanh(scale * rot(q_i) . rot(k_j) / cap)   for j <= i in i's chunk
              a_ij = exp(s_ij) / (exp(sink_h) + sum_j exp(s_ij))
              o_i  = sum_j a_ij v_j;  mix = Wo (o * sigmoid(Wg h)_h)  (one gate a head)
              f_i from Llama-3.1-style scaling of base^(-2i/dims), mag = 1
  'latent_attention' mixer:
              cq = N_dq(Wdq h), q = Wuq cq, per head [dim plain | rot_dim rotated]
              (c | r) = Wdkv h: c = N_dkv(first kv_rank), r the last rot_dim (one for all heads)
              k_h = Wuk c, v_h = Wuv c
              s_ij = scale * (q_plain . k_plain + rot(q_rot) . rot(r_j))  for i - window < j <= i
              a = softmax(s);  mix = Wo ((sum_j a_ij v_j) * sigmoid(Wg h))  (a gate an element)
              f_i and mag from YaRN scaling
  ff(h)     = Wdown gelu(Wup h), gelu(z) = z/2 (1 + erf(z / sqrt 2))
  logits    = cap_L * tanh(H N_final(x) / cap_L)
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch

F64 = torch.float64


# ----------------------------------------------------------------------------- small pieces
def rms_norm(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    v = v.to(F64)
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps) * w.to(F64)


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def tanh_cap(s: torch.Tensor, cap: Optional[float]) -> torch.Tensor:
    return s if cap is None else cap * torch.tanh(s / cap)


def base_frequencies(base: float, dims: int) -> torch.Tensor:
    i = torch.arange(dims // 2, dtype=F64)
    return torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * i / dims)


def wavelength_scaled_frequencies(base: float, dims: int, sc: dict) -> torch.Tensor:
    """Long wavelengths slowed by ``factor``, short ones kept, a straight blend between."""
    f = base_frequencies(base, dims)
    factor, low, high, orig = (float(sc[k]) for k in ("factor", "low", "high", "original"))
    out = f.clone()
    for i in range(f.numel()):
        fi = float(f[i])
        wl = 2.0 * math.pi / fi
        if wl < orig / high:
            out[i] = fi
        elif wl > orig / low:
            out[i] = fi / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def yarn_frequencies(base: float, dims: int, sc: dict) -> Tuple[torch.Tensor, float]:
    """(frequencies, the factor both cosine and sine are multiplied by)."""
    f = base_frequencies(base, dims)
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(t: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    out = f.clone()
    for i in range(f.numel()):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
    return out, 0.1 * math.log(factor) + 1.0


def rotate_leading(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor, dims: int,
                   mag: float = 1.0) -> torch.Tensor:
    """x [T, heads, d]: the first ``dims`` elements of every head are rotated in the pairs
    (i, i + dims/2); the rest pass."""
    x = x.to(F64).clone()
    half = dims // 2
    ang = positions.to(F64)[:, None] * freqs[None, :]           # [T, half]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., :half].clone(), x[..., half:dims].clone()
    x[..., :half] = a * c - b * s
    x[..., half:dims] = b * c + a * s
    return x


def chunk_mask(T: int, size: int) -> torch.Tensor:
    """[T, T] True where query i sees key j: j <= i and both in the same chunk of ``size``."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def window_mask(T: int, size: int) -> torch.Tensor:
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i - j < size)


def masked_softmax_values(s: torch.Tensor, mask: torch.Tensor, v: torch.Tensor,
                          sink: Optional[torch.Tensor]) -> torch.Tensor:
    """s [H, T, T] scores, v [H, T, dv]; with ``sink`` [H] the denominator holds exp(sink_h)
    once more, which brings no value."""
    s = s.masked_fill(~mask[None], float("-inf"))
    m = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink.to(F64)[:, None, None])
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.to(F64)[:, None, None] - m)
    return (e / den) @ v


# ----------------------------------------------------------------------------- mixers
def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                    positions: torch.Tensor) -> torch.Tensor:
    h = h.to(F64)
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ w[p + "q"].to(F64).T, w[p + "q.norm"], eps).view(T, H, d)
    k = rms_norm(h @ w[p + "k"].to(F64).T, w[p + "k.norm"], eps).view(T, G, d)
    v = (h @ w[p + "v"].to(F64).T).view(T, G, dv)
    rot = m["rot"]
    f = wavelength_scaled_frequencies(rot["base"], rot["dims"], rot["scaling"]) \
        if rot.get("scaling") else base_frequencies(rot["base"], rot["dims"])
    q = rotate_leading(q, positions, f, rot["dims"])
    k = rotate_leading(k, positions, f, rot["dims"])
    per = H // G
    kk = k.repeat_interleave(per, dim=1).permute(1, 0, 2)        # [H, T, d]
    vv = v.repeat_interleave(per, dim=1).permute(1, 0, 2)
    s = tanh_cap((q.permute(1, 0, 2) @ kk.transpose(1, 2)) * float(m["scale"]), m.get("softcap"))
    o = masked_softmax_values(s, chunk_mask(T, m["mask"]["size"]), vv, w[p + "sink"])
    gate = torch.sigmoid(h @ w[p + "g"].to(F64).T)               # [T, H]
    o = o.permute(1, 0, 2) * gate[:, :, None]
    return o.reshape(T, H * dv) @ w[p + "o"].to(F64).T


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict,
                           eps: float, positions: torch.Tensor) -> torch.Tensor:
    h = h.to(F64)
    T = h.shape[0]
    H, d, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ w[p + "dq"].to(F64).T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].to(F64).T).view(T, H, d + dr)
    ckv = h @ w[p + "dkv"].to(F64).T
    c = rms_norm(ckv[:, :rank], w[p + "dkv.norm"], eps)
    r = ckv[:, rank:].view(T, 1, dr)
    rot = m["rot"]
    f, mag = yarn_frequencies(rot["base"], rot["dims"], rot["scaling"]) if rot.get("scaling") \
        else (base_frequencies(rot["base"], rot["dims"]), 1.0)
    q_rot = rotate_leading(q[..., d:], positions, f, rot["dims"], mag)
    r = rotate_leading(r, positions, f, rot["dims"], mag)
    k = (c @ w[p + "uk"].to(F64).T).view(T, H, d)
    v = (c @ w[p + "uv"].to(F64).T).view(T, H, dv)
    s = q[..., :d].permute(1, 0, 2) @ k.permute(1, 2, 0) \
        + q_rot.permute(1, 0, 2) @ r.permute(1, 2, 0)            # [H, T, T]
    s = s * float(m["scale"])
    o = masked_softmax_values(s, window_mask(T, m["mask"]["size"]), v.permute(1, 0, 2), None)
    o = o.permute(1, 0, 2).reshape(T, H * dv) * torch.sigmoid(h @ w[p + "g"].to(F64).T)
    return o @ w[p + "o"].to(F64).T


MIXERS = {"attention": attention_mixer, "latent_attention": latent_attention_mixer}


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    h = h.to(F64)
    return gelu_erf(h @ w[p + "up"].to(F64).T) @ w[p + "down"].to(F64).T


# ----------------------------------------------------------------------------- the model
def forward(config: dict, w: Dict[str, torch.Tensor], tokens: Sequence[int],
            streams: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``streams`` (a list) receives the residual
    stream after every layer."""
    eps = float(config["norm"]["eps"])
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    pos = torch.arange(len(ids))
    x = w["embed"].to(F64)[ids] * float(config["embedding"]["scale"])
    for i, L in enumerate(config["layers"]):
        p = f"l{i}."
        x = x + rms_norm(MIXERS[L["type"]](x, w, p + "mix.", L["mixer"], eps, pos),
                         w[p + "norm1"], eps)
        if L.get("mlp") is not None:
            x = x + rms_norm(dense_ff(x, w, p + "mlp."), w[p + "norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    z = rms_norm(x, w["final.norm"], eps) @ w["head"].to(F64).T
    return tanh_cap(z, config.get("logit_softcap"))


def greedy(config: dict, w: Dict[str, torch.Tensor], prompt: Sequence[int], n: int) -> List[int]:
    ids = list(prompt)
    out = []
    for _ in range(n):
        t = int(torch.argmax(forward(config, w, ids)[-1]))
        out.append(t)
        ids.append(t)
    return out
