"""Typed configuration of the Lodenex decoder, read from its config.json.

A Lodenex model is a list of layers, each with one of two mixers and an optional dense
feed-forward.  The sublayers read the residual stream as it is; an RMS norm stands behind each,
ahead of the residual sum.  Every size and every constant that can differ between models comes
from config.json; the layers may all differ.  There is no bound on positions in the file: the
rotations form their angles from the position itself.

    {"architecture": "Lodenex", "vocab": V, "width": W, "norm": {"eps": e},
     "embedding": {"scale": s}, "logit_softcap": c,
     "layers": [
       {"type": "attention",
        "mixer": {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": s, "softcap": c,
                  "mask": {"size": chunk},
                  "rot": {"base": b, "dims": r,
                          "scaling": {"factor", "low", "high", "original"}}},
        "mlp": null | {"kind": "dense", "ff": f}},
       {"type": "latent_attention",
        "mixer": {"heads": H, "dim": d, "rot_dim": r, "vdim": dv, "q_rank": a, "kv_rank": b,
                  "scale": s, "mask": {"size": window},
                  "rot": {"base": b, "dims": r,
                          "scaling": {"factor", "original", "fast", "slow"}}},
        "mlp": ...}]}

Tensor names: ``embed``, ``head``, ``final.norm``, and per layer i under ``l<i>.``: ``norm1``,
``norm2``, ``mlp.up``, ``mlp.down`` and the mixer's under ``mix.``: ``q k v o g sink q.norm
k.norm`` or ``dq dq.norm uq dkv dkv.norm uk uv g o``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError
from .registry import register_architecture
from .rotary import leading_rotary
from .specs import (DenseMlpSpec, LatentAttentionSpec, LayerNormSpec, MaskedGqaAttentionSpec,
                    ModelSpec, PostNormBlockSpec, ScheduleEntry)

# positions are 32-bit numbers in the kernels, and exact as such up to here
MAX_POSITIONS = 1 << 24
# the feed-forward's activation is the exact gelu
FF_ACTIVATION = "gelu"


def _int(d, key: str, where: str, minimum: int = 1) -> int:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json: {where}{key!r} must be an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json: {where}{key!r} must be at least {minimum}, got {v}")
    return v


def _num(d, key: str, where: str) -> float:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}{key!r} must be a number, got {v!r}")
    return float(v)


def _opt_num(d, key: str, where: str) -> Optional[float]:
    if not isinstance(d, dict) or d.get(key) is None:
        return None
    return _num(d, key, where)


def _obj(d, key: str, where: str) -> dict:
    v = d.get(key) if isinstance(d, dict) else None
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: {where}{key!r} must be an object, got {v!r}")
    return v


def _rotary(m: dict, where: str, limit: int):
    """The mixer's ``rot`` object; ``limit``: the rotated elements must fit the part of a head
    that is rotated."""
    if m.get("rot") is None:
        return None
    r = _obj(m, "rot", where)
    dims = _int(r, "dims", where + "rot.", 2)
    if dims % 2 != 0 or dims > limit:
        raise ConfigError(f"config.json: {where}rot.dims={dims} must be even and at most {limit}")
    scaling = r.get("scaling")
    if scaling is not None and not isinstance(scaling, dict):
        raise ConfigError(f"config.json: {where}rot.scaling must be an object or null")
    return leading_rotary(_num(r, "base", where + "rot."), dims, scaling)


@dataclass(frozen=True)
class LodenexConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    logit_softcap: Optional[float]
    layers: Tuple[object, ...]                 # one PostNormBlockSpec a layer
    raw: dict

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, raw: dict) -> "LodenexConfig":
        vocab = _int(raw, "vocab", "")
        width = _int(raw, "width", "")
        eps = _num(_obj(raw, "norm", ""), "eps", "norm.")
        if not eps >= 0.0:
            raise ConfigError(f"config.json: norm.eps={eps} must not be negative")
        scale = 1.0
        if raw.get("embedding") is not None:
            scale = _num(_obj(raw, "embedding", ""), "scale", "embedding.")
        cap = _opt_num(raw, "logit_softcap", "")
        if cap is not None and not cap > 0.0:
            raise ConfigError(f"config.json: logit_softcap={cap} must be positive")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        norm = cls._norm(width, eps)
        blocks = tuple(cls._block(i, L, width, eps, norm) for i, L in enumerate(layers))
        return cls(vocab, width, eps, scale, cap, blocks, copy.deepcopy(raw))

    @staticmethod
    def _norm(width: int, eps: float) -> LayerNormSpec:
        # x / sqrt(mean x^2 + eps) * w: not centred, no bias; the gain's tensor is the prefix itself
        return LayerNormSpec(width, eps, centred=False, weight_name="", bias_name=None)

    @staticmethod
    def _block(i: int, L, width: int, eps: float, norm: LayerNormSpec) -> PostNormBlockSpec:
        where = f"layers[{i}]."
        if not isinstance(L, dict):
            raise ConfigError(f"config.json: layers[{i}] must be an object")
        kind = L.get("type")
        m = _obj(L, "mixer", where)
        mw = where + "mixer."
        if kind == "attention":
            mixer = LodenexConfig._attention(m, mw, width, eps)
        elif kind == "latent_attention":
            mixer = LodenexConfig._latent(m, mw, width, eps)
        else:
            raise ConfigError(f"config.json: {where}type={kind!r}: the mixers of this design "
                              "are 'attention' and 'latent_attention'")
        ff = None
        f = L.get("mlp")
        if f is not None:
            fw = where + "mlp."
            if not isinstance(f, dict) or f.get("kind") != "dense":
                raise ConfigError(f"config.json: {fw}kind="
                                  f"{f.get('kind') if isinstance(f, dict) else f!r}: the "
                                  "feed-forward of this design is 'dense'")
            ff = DenseMlpSpec(width, _int(f, "ff", fw), FF_ACTIVATION, up_name="up",
                              down_name="down")
        return PostNormBlockSpec(mixer=mixer, feed_forward=ff, mixer_post_norm=norm,
                                 ff_post_norm=norm if ff is not None else None,
                                 mixer_prefix="mix.", ff_prefix="mlp.",
                                 mixer_post_norm_prefix="norm1", ff_post_norm_prefix="norm2")

    @staticmethod
    def _mask(m: dict, mw: str) -> Optional[int]:
        if m.get("mask") is None:
            return None
        return _int(_obj(m, "mask", mw), "size", mw + "mask.")

    @staticmethod
    def _attention(m: dict, mw: str, width: int, eps: float) -> MaskedGqaAttentionSpec:
        heads, kv_heads = _int(m, "heads", mw), _int(m, "kv_heads", mw)
        if heads % kv_heads != 0:
            raise ConfigError(f"config.json: {mw}heads={heads} is no multiple of "
                              f"kv_heads={kv_heads}")
        dim = _int(m, "dim", mw)
        cap = _opt_num(m, "softcap", mw)
        if cap is not None and not cap > 0.0:
            raise ConfigError(f"config.json: {mw}softcap={cap} must be positive")
        return MaskedGqaAttentionSpec(
            hidden_size=width, n_heads=heads, n_kv_heads=kv_heads, head_dim=dim,
            value_dim=_int(m, "vdim", mw), scale=_num(m, "scale", mw), qk_norm_eps=eps,
            rotary=_rotary(m, mw, dim), softcap=cap, chunk=LodenexConfig._mask(m, mw),
            sink=True, head_gate=True, q_name="q", k_name="k", v_name="v", o_name="o",
            q_norm_name="q.norm", k_norm_name="k.norm", sink_name="sink", gate_name="g")

    @staticmethod
    def _latent(m: dict, mw: str, width: int, eps: float) -> LatentAttentionSpec:
        rot_dim = _int(m, "rot_dim", mw, 2)
        rotary = _rotary(m, mw, rot_dim)
        if rotary is not None and rotary.dims != rot_dim:
            raise ConfigError(f"config.json: {mw}rot.dims={rotary.dims}: the rotated part of a "
                              f"head is rot_dim={rot_dim} wide and is rotated whole")
        return LatentAttentionSpec(
            hidden_size=width, n_heads=_int(m, "heads", mw), head_dim=_int(m, "dim", mw),
            rot_dim=rot_dim, value_dim=_int(m, "vdim", mw), q_rank=_int(m, "q_rank", mw),
            kv_rank=_int(m, "kv_rank", mw), scale=_num(m, "scale", mw), norm_eps=eps,
            rotary=rotary, window=LodenexConfig._mask(m, mw), element_gate=True,
            dq_name="dq", dq_norm_name="dq.norm", uq_name="uq", dkv_name="dkv",
            dkv_norm_name="dkv.norm", uk_name="uk", uv_name="uv", gate_name="g", o_name="o")

    def to_dict(self) -> dict:
        return copy.deepcopy(self.raw)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def model_type(self) -> str:
        return "lodenex"

    # ------------------------------------------------------------------ the model's parts
    def model_spec(self) -> ModelSpec:
        return ModelSpec(
            vocab_size=self.vocab, hidden_size=self.width, max_positions=MAX_POSITIONS,
            layers=self.layers, schedule=tuple(ScheduleEntry(i) for i in range(len(self.layers))),
            final_norm=self._norm(self.width, self.norm_eps), tie_word_embeddings=False,
            embed_name="embed", final_norm_prefix="final.norm", head_name="head",
            layer_prefix="l{}.", embedding_multiplier=self.embedding_scale,
            logit_softcap=self.logit_softcap)


register_architecture("Lodenex", LodenexConfig)
