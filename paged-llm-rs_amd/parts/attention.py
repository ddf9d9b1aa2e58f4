"""Grouped-query attention over a paged cache (reference: model/attention.rs).

Order of operations, which cannot be guessed from a Llama-shaped model: project,
split into heads, normalise q and k over one head's width (when the spec asks
for it), rotate q and k, write k and v into the pages, then attend.  The write
precedes the read inside the layer, so a token attends to itself and the later
tokens of a portion read the earlier ones through the cache.
"""

from __future__ import annotations

import math

import torch

from .. import kernels
from ..cache.layout import KVCacheSpec
from ..errors import UnsupportedError
from ..weights.loader import ParamDecl
from .linear import Linear
from .registry import register_mixer
from .rotary import rotary_tables


class PagedAttention:
    @staticmethod
    def declare(spec, hidden: int) -> list:
        q, kv = spec.num_heads * spec.head_dim, spec.num_kv_heads * spec.head_dim
        decls = [
            ParamDecl("q_proj.weight", (q, hidden)), ParamDecl("k_proj.weight", (kv, hidden)),
            ParamDecl("v_proj.weight", (kv, hidden)), ParamDecl("o_proj.weight", (hidden, q)),
        ]
        if spec.qk_norm is not None:
            decls += [ParamDecl("q_norm.weight", (spec.head_dim,), "gain"),
                      ParamDecl("k_norm.weight", (spec.head_dim,), "gain")]
        if spec.qkv_bias:
            decls += [ParamDecl("q_proj.bias", (q,), "bias"), ParamDecl("k_proj.bias", (kv,), "bias"),
                      ParamDecl("v_proj.bias", (kv,), "bias")]
        if spec.out_bias:
            decls.append(ParamDecl("o_proj.bias", (hidden,), "bias"))
        return decls

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        if spec.num_heads % spec.num_kv_heads:
            raise UnsupportedError(f"{spec.num_heads} query heads over {spec.num_kv_heads} key heads, "
                                   "which do not group evenly")
        if not 1 <= spec.head_dim <= 256:
            raise UnsupportedError(f"head size {spec.head_dim}: the kernels take head sizes up to 256")
        if spec.head_dim % 16 and dtype != torch.float32:
            raise UnsupportedError(f"head size {spec.head_dim}: the bfloat16 kernels take multiples of 16 "
                                   "(the 32-bit path takes any size up to 256)")
        if spec.qk_norm is not None and spec.qk_norm.kind != "rms_norm":
            raise UnsupportedError(f"q/k norm {spec.qk_norm.kind!r}, only rms_norm is implemented")
        self.spec = spec
        self.nq, self.nkv, self.d = spec.num_heads, spec.num_kv_heads, spec.head_dim
        self.scale = spec.scale if spec.scale is not None else 1.0 / math.sqrt(spec.head_dim)
        self.window = int(spec.window or 0)
        # one product for q, k and v: the output row is [q | k | v]
        self.qkv_proj = Linear.fused([params["q_proj.weight"], params["k_proj.weight"], params["v_proj.weight"]],
                                     [params.get("q_proj.bias"), params.get("k_proj.bias"), params.get("v_proj.bias")])
        self.o_proj = Linear(params["o_proj.weight"], params.get("o_proj.bias"))
        self.q_gain = params.get("q_norm.weight")
        self.k_gain = params.get("k_norm.weight")
        self.eps = float(spec.qk_norm.eps) if spec.qk_norm is not None else 0.0
        self.rotary = rotary_tables(spec.position, device, shared) if spec.position is not None else None
        if self.rotary is not None and self.rotary.dim > self.d:
            raise UnsupportedError(f"a rotation over {self.rotary.dim} values of a head of {self.d}")

    def cache_spec(self):
        return KVCacheSpec(self.nkv, self.d, self.window or None)

    def state_spec(self):
        return None

    # requests that bring fewer tokens than this go to a kernel of their own, which a step sizes by their tokens
    short_portion = kernels.SHORT_PORTION

    # forward takes a norm still to run in place of rows, and may add its result into ctx.residual
    fuses = True
    # ... and records named activations into ctx.trace
    records = True

    def forward(self, x, ctx):
        """``x``: normalised rows, or a PendingNorm.  Where ``ctx.residual`` is given and the output
        projection can add into it, None comes back."""
        batch = ctx.batch
        kv = ctx.kv()
        qkv = self.qkv_proj.forward(x)
        cos = self.rotary.cos if self.rotary is not None else None
        sin = self.rotary.sin if self.rotary is not None else None
        rot = self.rotary.dim if self.rotary is not None else 0
        prepare = kernels.QkFusion(self.q_gain, self.k_gain, self.eps, cos, sin, rot, ctx.writes_cache,
                                   neighbours=bool(getattr(self.rotary, "neighbours", False)))
        out = torch.empty((qkv.shape[0], self.nq * self.d), dtype=qkv.dtype, device=qkv.device)
        if ctx.trace is not None:
            self._record_projections(qkv, batch, kv, ctx.trace)
        kernels.attention_step(qkv, out, batch, kv, self.nq, self.nkv, self.d, self.scale, self.window, prepare)
        if ctx.trace is not None:
            ctx.trace.record("o_proj.in", out)
            out = self.o_proj.forward(out)
            ctx.trace.record("o_proj.out", out)
            return out
        return self.o_proj.forward(out, add_into=ctx.residual,
                                   hand=getattr(ctx, "hand", None) if ctx.residual is not None else None)

    def _record_projections(self, qkv, batch, kv, trace) -> None:
        """q, k and v as projected, and q and k after their per-head norm (before the rotation).  The
        norm, the rotation and the cache write are one kernel; for the record it runs once more on copies,
        without rotation and without writing, the keys standing in the place of queries."""
        q_width, kv_width = self.nq * self.d, self.nkv * self.d
        q, k, v = qkv[:, :q_width], qkv[:, q_width:q_width + kv_width], qkv[:, q_width + kv_width:]
        trace.record("q_proj.out", q)
        trace.record("k_proj.out", k)
        trace.record("v_proj.out", v)
        if self.q_gain is None:
            return
        for name, heads, count, gain in (("q_norm.out", q, self.nq, self.q_gain), ("k_norm.out", k, self.nkv, self.k_gain)):
            copy = torch.cat([heads, k, v], dim=1).contiguous()
            kernels.qk_norm_rope_kv_write(copy, gain, gain, self.eps, None, None, 0, batch.positions, batch.seq_of,
                                          kv.block_table, kv.block_size, kv.k_pool, kv.v_pool, count, self.nkv, self.d,
                                          write_kv=False)
            trace.record(name, copy[:, :count * self.d])


register_mixer("paged_attention", PagedAttention)
