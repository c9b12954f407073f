"""Causal self-attention with grouped key/value heads over the cache
(/root/reference/crates/nnis-model/src/runtime.rs:959-1038; formula
/root/reference/crates/nnis-model/src/kernels.rs:66-125).  Queries, keys and
values come from one fused projection; queries and keys are rotated by the
position encoding handed in; keys and values go into the cache before the
scores are taken, so the same code runs whole prompts and single tokens.
"""

from __future__ import annotations

import math

import torch

from ..errors import InvalidInput
from .base import KVRequest, Mixer, TensorSpec, register_part
from .linear import Projection


class CausalSelfAttention(Mixer):
    graph_safe = True

    def __init__(self, width, heads, kv_heads, head_dim, q, k, v, o, position=None, window=None, positions=None):
        if heads % kv_heads != 0:
            raise InvalidInput(f"{heads} query heads do not divide into {kv_heads} key/value heads")
        self.width, self.heads, self.kv_heads, self.head_dim = int(width), int(heads), int(kv_heads), int(head_dim)
        self.names = {"q": q, "k": k, "v": v, "o": o}
        self.window = None if not window else int(window)
        self.position = None
        if position is not None:
            if positions is None or position not in positions:
                raise InvalidInput(f"attention names position encoding {position!r}, which the model does not define")
            self.position = positions[position]
        self.scale = 1.0 / math.sqrt(self.head_dim)  # runtime.rs:943
        self.qkv = None
        self.out = None

    def tensors(self):
        q_width, kv_width = self.heads * self.head_dim, self.kv_heads * self.head_dim
        return [
            TensorSpec(self.names["q"], (q_width, self.width)),
            TensorSpec(self.names["k"], (kv_width, self.width)),
            TensorSpec(self.names["v"], (kv_width, self.width)),
            TensorSpec(self.names["o"], (self.width, q_width)),
        ]

    def bind(self, weights, rt):
        # one projection for queries, keys and values: rows q heads, k heads, v heads
        self.qkv = Projection(torch.cat([weights[self.names["q"]], weights[self.names["k"]], weights[self.names["v"]]], dim=0), rt)
        self.out = Projection(weights[self.names["o"]], rt)

    def weight_bytes(self):
        return self.qkv.weight_bytes() + self.out.weight_bytes()

    def cache_request(self):
        return KVRequest(self.kv_heads, self.head_dim, self.window)

    def check(self, rt):
        rt.ops.attention_check(self.head_dim)

    def _matrix_cores(self, rt) -> bool:
        return rt.dtype == torch.bfloat16 and self.head_dim % 16 == 0

    def decode_plan(self, batch, longest, rt):
        # (runs of the keys, waves of a block) of a step of single tokens with these sizes
        return rt.ops.decode_plan(batch, self.kv_heads, longest, width=self.heads * self.head_dim)

    def prompt_plan(self, batch, rows, longest, rt):
        # (waves of a block, columns a wave carries) of the matrix-core kernel; the 32-bit kernel has no plan
        if not self._matrix_cores(rt):
            return None
        return rt.ops.prefill_plan(longest, rows, self.heads, self.head_dim, self.kv_heads)

    def held_buffers(self, rt):
        # the runs of a decode step's keys meet in a scratch that the kernels' wrapper keeps per device
        held = rt.ops.decode_scratch_held(rt.device)
        return [] if held is None else [held]

    takes_pending_norm = True
    adds_to_residual = True

    def _project_rotate_store(self, x, ctx, view, rt):
        """Queries [tokens, heads * head_dim], rotated; keys and values of the
        step's tokens in the cache."""
        from .lazy import PendingNorm

        tables = self.position.rotary() if self.position is not None else None
        writes = not view.read_only
        if isinstance(x, PendingNorm):
            if (x.can_fuse(self.qkv.weight) and tables is not None and tables.rot_dim == self.head_dim
                    and self.head_dim % 32 == 0 and view.k_pages.dtype == torch.bfloat16):
                # residual sum, norm, the three projections, the rotation and the cache write in one kernel
                rope = dict(cos=tables.cos, sin=tables.sin, tok_slot=ctx.tok_slot, tok_pos=ctx.tok_pos,
                            tables=ctx.step_tables(rt, tables, view.block_table),
                            k_pages=view.k_pages if writes else None, v_pages=view.v_pages if writes else None,
                            block_table=view.block_table if writes else None, heads=self.heads,
                            kv_heads=self.kv_heads, head_dim=self.head_dim)
                return x.fused(self.qkv.weight, rt.empty(x.rows, self.heads * self.head_dim), rt.ops.EPILOGUE_ROPE, rope)
            x = x.materialize()
        tokens = x.shape[0]
        qkv = self.qkv(x, rt)
        q = rt.empty(tokens, self.heads * self.head_dim)
        rt.ops.rope_kv_write(
            qkv, q,
            tables.cos if tables else None, tables.sin if tables else None, tables.rot_dim if tables else 0,
            ctx.tok_slot, ctx.tok_pos,
            view.k_pages if writes else None, view.v_pages if writes else None, view.block_table if writes else None,
            self.heads, self.kv_heads, self.head_dim,
        )
        return q

    def forward(self, x, ctx, view, rt, into=None):
        q = self._project_rotate_store(x, ctx, view, rt)
        tokens = q.shape[0]
        attn = rt.empty(tokens, self.heads * self.head_dim)
        # a decode step over long sequences leaves its runs of keys to the output projection, if that takes them
        step = None
        if ctx.decode and q.dtype == torch.bfloat16:
            step = ctx.step_tables(rt, self.position.rotary() if self.position is not None else None, view.block_table)
        plan = ctx.options.get("causal_attention")  # (a test or a sweep names the launch; else the sizes choose)
        if plan is None:
            plan = (self.decode_plan(ctx.batch, ctx.planned_len, rt) if ctx.decode
                    else self.prompt_plan(ctx.batch, ctx.planned_rows, ctx.planned_len, rt))
        attn = rt.ops.attention(q, attn, view, ctx, self.heads, self.kv_heads, self.head_dim, self.scale, self.window or 0,
                                keep_runs=into is not None, tables=step, plan=plan)
        if isinstance(attn, rt.ops.KeyRuns) and not (into.can_take(attn, self.out.weight) and attn.fits(self.out.weight.shape[0])):
            attn = attn.combine()
        if into is not None and into.can_take(attn, self.out.weight):
            return into.take(attn, self.out.weight)  # the output projection adds to the stream itself
        return self.out(attn, rt)


register_part("mixer", "causal_attention", CausalSelfAttention)
