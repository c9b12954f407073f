"""Plain, slow implementation of the Llama decoder for the tests.

Whole sequences, no cache, one function per part, written from the reference's
formulas and sharing no code with ``nnis_amd``.  It reads ``config.json`` and
``model.safetensors`` itself (with the ``safetensors`` package and ``json``),
so a fault in the library's loader cannot hide behind a shared reader.

All reference citations are paths under /root/reference/.

``round_to`` lets a caller emulate storage in a narrower type at the places
where the engine stores activations (the reference's 16-bit policy rounds once
at each tensor boundary and accumulates in 32-bit,
crates/nnis-model/src/f16_reference_kernels.rs:75-315); with ``None`` every
value stays in the working precision.
"""

from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np
import torch

Round = Optional[Callable[[torch.Tensor], torch.Tensor]]


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    """Round to nearest-even bfloat16 and widen back (exact widening is
    ``bits << 16``: crates/nnis-model/src/safetensors_loader.rs:610-624)."""
    return x.to(torch.bfloat16).to(x.dtype)


def _r(x: torch.Tensor, round_to: Round) -> torch.Tensor:
    return x if round_to is None else round_to(x)


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------

def embedding(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    """x_t = E[id_t, :], a row copy without scaling
    (crates/nnis-kernels/src/gather.rs:17-33; crates/nnis-model/src/runtime.rs:933-940)."""
    return table[torch.as_tensor(list(ids), dtype=torch.long)]


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y[c] = (x[c] * rsqrt(sum(x^2) * (1/cols) + eps)) * w[c]; eps inside the
    root, mean over the row, multiplicative weight without "+1"
    (crates/nnis-model/src/kernels.rs:15-48)."""
    cols = x.shape[-1]
    sumsq = (x * x).sum(dim=-1, keepdim=True)
    scale = 1.0 / torch.sqrt(sumsq * (1.0 / cols) + eps)
    return (x * scale) * weight


def linear(x: torch.Tensor, weight_out_in: torch.Tensor) -> torch.Tensor:
    """y = W x with the checkpoint's [out, in] weight, no bias.  The reference
    transposes to [in, out] at load and computes sum_k x[k] * W[k, n]
    (crates/nnis-model/src/safetensors_loader.rs:590-607,734-747;
    crates/nnis-kernels/src/gemv.rs:45-62)."""
    return x @ weight_out_in.t()


def rope_tables(positions: int, head_dim: int, theta: float):
    """cos/sin[pos][pair] as the reference builds them, in 32-bit:
    exponent = (2*pair)/head_dim, inv_freq = 1/theta**exponent,
    angle = pos * inv_freq, then cos and sin of that 32-bit angle
    (crates/nnis-model/src/runtime.rs:1166-1184).  ``powf``, ``cos`` and
    ``sin`` of 32-bit arguments are taken as correctly rounded: each is
    evaluated in 64-bit on the 32-bit argument and rounded once."""
    half = head_dim // 2
    pair = np.arange(half, dtype=np.float32)
    exponent = (np.float32(2.0) * pair) / np.float32(head_dim)  # 32-bit quotient
    power = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64)).astype(np.float32)
    inv_freq = (np.float32(1.0) / power).astype(np.float32)
    pos = np.arange(positions, dtype=np.float32)[:, None]
    angle = (pos * inv_freq[None, :]).astype(np.float32)  # 32-bit product
    cos = np.cos(angle.astype(np.float64)).astype(np.float32)
    sin = np.sin(angle.astype(np.float64)).astype(np.float32)
    return cos, sin


def rope_rotate_half(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x: [tokens, heads, head_dim]; cos/sin: [tokens, head_dim/2] (the table
    row of each token's position).  out[j] = x[j]*c - x[j+half]*s and
    out[j+half] = x[j+half]*c + x[j]*s, the same (c, s) for both halves
    (crates/nnis-model/src/runtime_kernels.rs:38-66)."""
    half = x.shape[-1] // 2
    left, right = x[..., :half], x[..., half:]
    c = cos[:, None, :].to(x.dtype)
    s = sin[:, None, :].to(x.dtype)
    return torch.cat([left * c - right * s, right * c + left * s], dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """q: [t, nh, hd]; k, v: [t, nkv, hd] of one whole sequence.  Query head h
    reads KV head h // (nh/nkv) (crates/nnis-model/src/kernels.rs:84-85); the
    score is the dot product times ``scale`` applied after the sum
    (kernels.rs:103-106); key p is visible to query i iff p <= i
    (crates/nnis-kernels/src/attention.rs:99-100); softmax over visible keys
    and the weighted sum of values (kernels.rs:97-124)."""
    t, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    out = torch.empty_like(q)
    visible = torch.tril(torch.ones(t, t, dtype=torch.bool))
    for head in range(nh):
        kv_head = head // group
        scores = (q[:, head, :] @ k[:, kv_head, :].t()) * scale
        scores = scores.masked_fill(~visible, float("-inf"))
        weights = torch.softmax(scores, dim=-1)
        out[:, head, :] = weights @ v[:, kv_head, :]
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)) (crates/nnis-kernels/src/lib.rs:111-122)."""
    return x / (1.0 + torch.exp(-x))


def swiglu(x: torch.Tensor, gate_w, up_w, down_w, round_to: Round = None) -> torch.Tensor:
    """down( silu(gate x) * up x ): SiLU on the gate branch
    (crates/nnis-model/src/runtime.rs:1054-1087; fused_swiglu.rs:14-28)."""
    gate = linear(x, gate_w)
    up = linear(x, up_w)
    hidden = _r(silu(gate) * up, round_to)
    return linear(hidden, down_w)


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------

class PlainLlama:
    """Reads a model folder and runs whole sequences."""

    def __init__(self, model_dir: str, dtype: torch.dtype = torch.float32):
        from safetensors import safe_open

        with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as handle:
            cfg = json.load(handle)
        self.cfg = cfg
        self.dtype = dtype
        self.L = cfg["num_hidden_layers"]
        self.H = cfg["hidden_size"]
        self.nh = cfg["num_attention_heads"]
        # default = number of query heads: safetensors_loader.rs:177-179
        self.nkv = cfg.get("num_key_value_heads") or self.nh
        # the reference derives head_dim = H / nh (config.rs:103-105)
        self.hd = cfg.get("head_dim") or self.H // self.nh
        self.eps = float(cfg["rms_norm_eps"])
        self.theta = float(cfg["rope_theta"])
        self.V = cfg["vocab_size"]
        self.tied = bool(cfg.get("tie_word_embeddings", False))
        self.w: Dict[str, torch.Tensor] = {}
        with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as handle:
            for name in handle.keys():
                self.w[name] = handle.get_tensor(name).to(dtype)
        cos, sin = rope_tables(cfg["max_position_embeddings"], self.hd, self.theta)
        self.cos = torch.from_numpy(cos)
        self.sin = torch.from_numpy(sin)

    def lm_head_weight(self) -> torch.Tensor:
        """lm_head.weight wins when present; else the embedding if tied
        (crates/nnis-model/src/safetensors_loader.rs:755-786)."""
        if "lm_head.weight" in self.w:
            return self.w["lm_head.weight"]
        assert self.tied, "no lm_head.weight and tie_word_embeddings is false"
        return self.w["model.embed_tokens.weight"]

    def hidden_states(self, ids: Sequence[int], first_position: int = 0, round_to: Round = None) -> torch.Tensor:
        """The residual stream after the last layer, [t, H].  Order of
        operations per layer: crates/nnis-model/src/runtime.rs:945-1095."""
        w = self.w
        t = len(ids)
        x = embedding(w["model.embed_tokens.weight"], ids)
        pos = torch.arange(first_position, first_position + t)
        cos, sin = self.cos[pos], self.sin[pos]
        scale = 1.0 / math.sqrt(self.hd)  # runtime.rs:943
        for layer in range(self.L):
            p = f"model.layers.{layer}."
            normed = _r(rms_norm(x, w[p + "input_layernorm.weight"], self.eps), round_to)
            q = _r(linear(normed, w[p + "self_attn.q_proj.weight"]), round_to).view(t, self.nh, self.hd)
            k = _r(linear(normed, w[p + "self_attn.k_proj.weight"]), round_to).view(t, self.nkv, self.hd)
            v = _r(linear(normed, w[p + "self_attn.v_proj.weight"]), round_to).view(t, self.nkv, self.hd)
            q = _r(rope_rotate_half(q, cos, sin), round_to)
            k = _r(rope_rotate_half(k, cos, sin), round_to)  # V is not rotated: runtime.rs:997-1007
            attn = _r(causal_attention(q, k, v, scale), round_to).reshape(t, self.nh * self.hd)
            x = x + _r(linear(attn, w[p + "self_attn.o_proj.weight"]), round_to)  # runtime.rs:1030-1044
            normed = _r(rms_norm(x, w[p + "post_attention_layernorm.weight"], self.eps), round_to)
            mlp = swiglu(
                normed,
                w[p + "mlp.gate_proj.weight"],
                w[p + "mlp.up_proj.weight"],
                w[p + "mlp.down_proj.weight"],
                round_to,
            )
            x = x + _r(mlp, round_to)  # runtime.rs:1088-1093
        return x

    def logits(self, ids: Sequence[int], round_to: Round = None) -> torch.Tensor:
        """Logits at every position, [t, V] in the working precision
        (final norm + head: crates/nnis-model/src/runtime.rs:1100-1116)."""
        x = self.hidden_states(ids, 0, round_to)
        normed = _r(rms_norm(x, self.w["model.norm.weight"], self.eps), round_to)
        return linear(normed, self.lm_head_weight())

    def greedy(self, ids: Sequence[int], max_new_tokens: int, stop: Sequence[int] = ()) -> List[int]:
        """Greedy continuation: lowest index on ties (numpy argmax returns the
        first maximum; crates/nnis-kernels/src/top_k.rs:41-92), the stop token
        is part of the result (crates/nnis-model/src/runtime.rs:885-890)."""
        ids = list(ids)
        out: List[int] = []
        for _ in range(max_new_tokens):
            row = self.logits(ids)[-1].to(torch.float32).numpy()
            token = int(np.argmax(row))
            out.append(token)
            ids.append(token)
            if token in stop:
                break
        return out


# --------------------------------------------------------------------------
# sampling (host, exact order of the reference)
# --------------------------------------------------------------------------

_MASK64 = (1 << 64) - 1


class PlainSplitMix64:
    """crates/nnis-model/src/sampling.rs:261-284."""

    def __init__(self, seed: int):
        self.state = seed & _MASK64

    def next_u64(self) -> int:
        self.state = (self.state + 0x9E3779B97F4A7C15) & _MASK64
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
        return z ^ (z >> 31)

    def next_unit(self) -> float:
        return (self.next_u64() >> 11) * (1.0 / float(1 << 53))


def plain_sample(logits: np.ndarray, rng: PlainSplitMix64, temperature: float = 1.0,
                 top_k: Optional[int] = None, top_p: Optional[float] = None) -> int:
    """One draw, step by step as crates/nnis-model/src/sampling.rs:113-202:
    sort by logit descending (ties: lower id), top-k cut, weights
    exp((l - max)/T) in 64-bit, top-p keeps the crossing candidate, then the
    first candidate whose cumulative weight exceeds u * total."""
    logits = np.asarray(logits, dtype=np.float32)
    if not np.all(np.isfinite(logits)):
        raise ValueError("non-finite logit")
    order = sorted(range(len(logits)), key=lambda i: (-float(logits[i]), i))
    if top_k is not None:
        order = order[:top_k]
    inv_t = 1.0 / float(np.float32(temperature))
    max_scaled = float(logits[order[0]]) * inv_t
    weights = [math.exp(float(logits[i]) * inv_t - max_scaled) for i in order]
    total = 0.0
    for wgt in weights:
        total += wgt
    if top_p is not None:
        threshold = float(np.float32(top_p)) * total
        cumulative = 0.0
        retained = len(order)
        for index, wgt in enumerate(weights):
            cumulative += wgt
            if cumulative >= threshold:
                retained = index + 1
                break
        order = order[: max(retained, 1)]
        weights = weights[: max(retained, 1)]
        total = 0.0
        for wgt in weights:
            total += wgt
    draw = rng.next_unit() * total
    cumulative = 0.0
    for token, wgt in zip(order, weights):
        cumulative += wgt
        if draw < cumulative:
            return token
    return order[-1]
