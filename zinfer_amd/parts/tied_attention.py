from __future__ import annotations

import math
from typing import Dict

import torch

from .. import ops
from ..config.specs import TiedKeyValueAttentionSpec
from ..errors import ConfigError
from .base import KVNeed, Mixer, TensorDecl, register_part
from .linear import Linear, place_matrix


class TiedKeyValueAttention(Mixer):
    """Causal grouped-query attention whose values are its keys: q = W_q h, k = W_k h, the
    token's key row goes into a cache that holds keys only, and
    o_i = sum_j a_ij k_j with a = softmax(scale q K^T) over the positions the (optional) window
    leaves, with one more term exp(0) in the denominator when the specification has a sink.
    With an output gate the concatenated heads are multiplied by sigmoid(W_g h) before the
    output projection.  Positions do not enter the scores.  q, k and the gate come from one
    product over the stacked matrices (each output keeps its own dot product); the attention
    kernel reads q and the gate as column slices of it.  Scores, weights and their sums are
    32-bit in both dtypes."""
    graph_safe = True
    stores_output = True
    kernel_modules = ("gemm", "sink_attention")

    def __init__(self, spec: TiedKeyValueAttentionSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        s = spec
        if s.n_heads < 1 or s.n_kv_heads < 1 or s.head_dim < 1:
            raise ConfigError("InvalidDimensions: heads and head_dim must be at least 1")
        if s.n_heads % s.n_kv_heads != 0:
            raise ConfigError(f"InvalidGrouping: {s.n_heads} query heads, {s.n_kv_heads} kv heads")
        if s.head_dim > ops.MAX_HEAD_DIM:
            raise ConfigError(f"InvalidHeadDim: head_dim={s.head_dim}: the attention kernels "
                              f"take head sizes up to {ops.MAX_HEAD_DIM}")
        if s.window is not None and s.window < 1:
            raise ConfigError(f"window={s.window} must be at least 1")
        self.q_width = s.n_heads * s.head_dim
        self.kv_width = s.n_kv_heads * s.head_dim
        self.scale = s.scale if s.scale is not None else 1.0 / math.sqrt(float(s.head_dim))

    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        d = {p + s.q_name: TensorDecl((self.q_width, s.hidden_size)),
             p + s.k_name: TensorDecl((self.kv_width, s.hidden_size)),
             p + s.o_name: TensorDecl((s.hidden_size, self.q_width))}
        if s.output_gate:
            d[p + s.gate_name] = TensorDecl((self.q_width, s.hidden_size))
        return d

    def bind(self, tensors) -> None:
        s, p = self.spec, self.prefix
        rows = [tensors[p + s.q_name], tensors[p + s.k_name]]
        if s.output_gate:
            rows.append(tensors[p + s.gate_name])
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        self.qkg = Linear(place_matrix(torch.cat(rows, dim=0), self.ctx))
        self.o = Linear(place_matrix(tensors[p + s.o_name], self.ctx))

    def cache_need(self):
        return KVNeed(self.spec.n_kv_heads, self.spec.head_dim, self.spec.window, value_dim=0)

    def accept_cache(self, cache) -> None:
        if cache.k_pool is not None and cache.k_pool.dtype != self.ctx.act_dtype:
            raise ConfigError(f"the cache is kept in the compute dtype ({self.ctx.act_dtype}): "
                              f"a cache of {cache.k_pool.dtype} needs a model built with that "
                              "dtype")

    def forward(self, h, residual, step, cache, accumulate: bool = True) -> None:
        s = self.spec
        T = h.shape[0]
        act = self.ctx.act_dtype
        if hasattr(h, "materialize"):
            h = h.materialize()
        kv = step.kv_tables(cache.group)
        width = self.qkg.out_features
        qkg = step.scratch("qkg", (T, width), act)
        self.qkg.forward(h, qkg)
        q = qkg[:, :self.q_width]
        k = qkg[:, self.q_width:self.q_width + self.kv_width]
        gate = qkg[:, self.q_width + self.kv_width:] if s.output_gate else None
        if cache.writes:
            ops.kv_rows_write(k, kv.slot_mapping, cache.k_pool, s.n_kv_heads, s.head_dim,
                              cache.page_size)
        attn = step.scratch("attn", (T, self.q_width), act)
        ops.tied_attention(q, gate, cache.k_pool, kv.block_table, step.q_start, step.ctx_len,
                           step.seq_index, attn, float(self.scale),
                           0 if s.window is None else int(s.window), bool(s.sink),
                           s.n_heads, s.n_kv_heads, s.head_dim, cache.page_size,
                           step.max_q_len, step.max_ctx_len)
        self.o.forward(attn, residual, accumulate=accumulate, step=step if accumulate else None)


register_part("mixer", TiedKeyValueAttentionSpec, TiedKeyValueAttention)
