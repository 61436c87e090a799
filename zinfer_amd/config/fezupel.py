"""Typed configuration of the Fezupel decoder, read from its config.json.

A Fezupel model is a list of layers, each with a mixer (``type``: "attention") and an
optional mixture-of-experts feed-forward, a norm before and after every sublayer, a learned
position table added to the embedding, and a ``loop`` that runs a range of layers several
times in a row with the same weights (every pass with a cache of its own).  Every size comes
from config.json; the layers may all differ.

    {"architecture": "Fezupel", "vocab": V, "width": W, "max_positions": P,
     "norm": {"eps": e}, "loop": {"start": a, "stop": b, "times": n},
     "layers": [{"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": s,
                           "mask": {"size": w}},
                 "mlp": null | {"kind": "moe", "router": {"experts": E, "top": k},
                                "expert": {"ff": f, "limit": L},
                                "shared": null | {"ff": f, "limit": L}}}, ...]}

Tensor names: ``embed``, ``pos``, ``head``, ``final.norm`` (+ ``.b``), and per layer i under
``l<i>.``: ``norm1 norm1b norm2 norm2b`` (+ ``.b``), ``mix.q mix.k mix.g mix.o``,
``mlp.router`` (+ ``.b``), ``mlp.e<j>.gate|up|down``, ``mlp.shared.gate|up|down``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError
from .registry import register_architecture
from .specs import (GatedExpertSpec, LayerNormSpec, ModelSpec, MoeSpec, SandwichNormBlockSpec,
                    ScheduleEntry, TiedKeyValueAttentionSpec)

# constants the design fixes: the experts' activation is g * sigmoid(1.702 g) * (u + 1)
EXPERT_ALPHA = 1.702
EXPERT_SHIFT = 1.0


def _int(d: dict, key: str, where: str, minimum: int = 1) -> int:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json: {where}{key!r} must be an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json: {where}{key!r} must be at least {minimum}, got {v}")
    return v


def _num(d: dict, key: str, where: str) -> float:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}{key!r} must be a number, got {v!r}")
    return float(v)


def _obj(d: dict, key: str, where: str) -> dict:
    v = d.get(key) if isinstance(d, dict) else None
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: {where}{key!r} must be an object, got {v!r}")
    return v


@dataclass(frozen=True)
class FezupelConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    layers: Tuple[object, ...]                 # one SandwichNormBlockSpec a layer
    loop: Optional[Tuple[int, int, int]]       # (start, stop, times)
    raw: dict

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, raw: dict) -> "FezupelConfig":
        vocab = _int(raw, "vocab", "")
        width = _int(raw, "width", "")
        max_positions = _int(raw, "max_positions", "")
        eps = _num(_obj(raw, "norm", ""), "eps", "norm.")
        if not eps >= 0.0:
            raise ConfigError(f"config.json: norm.eps={eps} must not be negative")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        norm = LayerNormSpec(width, eps, centred=True, weight_name="", bias_name=".b")
        blocks = tuple(cls._block(i, L, width, norm) for i, L in enumerate(layers))
        loop = None
        if raw.get("loop") is not None:
            lp = _obj(raw, "loop", "")
            a, b = _int(lp, "start", "loop.", 0), _int(lp, "stop", "loop.", 0)
            times = _int(lp, "times", "loop.", 1)
            if not (a <= b <= len(blocks)):
                raise ConfigError(f"config.json: loop {a}..{b} does not lie within the "
                                  f"{len(blocks)} layers")
            loop = (a, b, times)
        return cls(vocab, width, max_positions, eps, blocks, loop, copy.deepcopy(raw))

    @staticmethod
    def _block(i: int, L, width: int, norm: LayerNormSpec) -> SandwichNormBlockSpec:
        where = f"layers[{i}]."
        if not isinstance(L, dict):
            raise ConfigError(f"config.json: layers[{i}] must be an object")
        kind = L.get("type")
        if kind != "attention":
            raise ConfigError(f"config.json: {where}type={kind!r}: the mixers of this design "
                              "are: 'attention'")
        m = _obj(L, "mixer", where)
        mw = where + "mixer."
        heads, kv_heads = _int(m, "heads", mw), _int(m, "kv_heads", mw)
        dim = _int(m, "dim", mw)
        if heads % kv_heads != 0:
            raise ConfigError(f"config.json: {mw}heads={heads} is no multiple of "
                              f"kv_heads={kv_heads}")
        if m.get("vdim", dim) != dim:
            raise ConfigError(f"config.json: {mw}vdim={m.get('vdim')!r}: the values are the keys, "
                              f"so their size is dim={dim}")
        window = _int(_obj(m, "mask", mw), "size", mw + "mask.")
        mixer = TiedKeyValueAttentionSpec(
            hidden_size=width, n_heads=heads, n_kv_heads=kv_heads, head_dim=dim,
            scale=_num(m, "scale", mw), window=window, sink=True, output_gate=True,
            q_name="q", k_name="k", gate_name="g", o_name="o")
        ff = None
        f = L.get("mlp")
        if f is not None:
            fw = where + "mlp."
            if not isinstance(f, dict) or f.get("kind") != "moe":
                raise ConfigError(f"config.json: {fw}kind={f.get('kind') if isinstance(f, dict) else f!r}"
                                  ": the feed-forward of this design is 'moe'")
            r = _obj(f, "router", fw)
            experts, top = _int(r, "experts", fw + "router."), _int(r, "top", fw + "router.")
            if top > experts:
                raise ConfigError(f"config.json: {fw}router.top={top} of {experts} experts")
            shared = None
            if f.get("shared") is not None:
                shared = FezupelConfig._expert(_obj(f, "shared", fw), fw + "shared.")
            ff = MoeSpec(hidden_size=width, n_experts=experts, top_k=top,
                         expert=FezupelConfig._expert(_obj(f, "expert", fw), fw + "expert."),
                         shared=shared, router_bias=True, router_name="router",
                         router_bias_name="router.b", expert_prefix="e{}.",
                         shared_prefix="shared.", gate_name="gate", up_name="up",
                         down_name="down")
        return SandwichNormBlockSpec(
            mixer=mixer, feed_forward=ff, mixer_norm=norm, mixer_post_norm=norm,
            ff_norm=norm if ff is not None else None,
            ff_post_norm=norm if ff is not None else None,
            mixer_prefix="mix.", ff_prefix="mlp.", mixer_norm_prefix="norm1",
            mixer_post_norm_prefix="norm1b", ff_norm_prefix="norm2", ff_post_norm_prefix="norm2b")

    @staticmethod
    def _expert(e: dict, where: str) -> GatedExpertSpec:
        limit = _num(e, "limit", where)
        if not limit > 0.0:
            raise ConfigError(f"config.json: {where}limit={limit} must be positive")
        return GatedExpertSpec(_int(e, "ff", where), limit, EXPERT_ALPHA, EXPERT_SHIFT)

    def to_dict(self) -> dict:
        return copy.deepcopy(self.raw)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def model_type(self) -> str:
        return "fezupel"

    # ------------------------------------------------------------------ the model's parts
    def layer_order(self) -> Tuple[int, ...]:
        n = len(self.layers)
        if self.loop is None:
            return tuple(range(n))
        a, b, times = self.loop
        return tuple(range(a)) + tuple(range(a, b)) * times + tuple(range(b, n))

    def model_spec(self) -> ModelSpec:
        """Every run of a layer, a repeated one too, has a cache of its own."""
        norm = LayerNormSpec(self.width, self.norm_eps, centred=True, weight_name="",
                             bias_name=".b")
        return ModelSpec(
            vocab_size=self.vocab, hidden_size=self.width, max_positions=self.max_positions,
            layers=self.layers, schedule=tuple(ScheduleEntry(i) for i in self.layer_order()),
            final_norm=norm, tie_word_embeddings=False, embed_name="embed",
            final_norm_prefix="final.norm", head_name="head", layer_prefix="l{}.",
            position_table_name="pos")


register_architecture("Fezupel", FezupelConfig)
