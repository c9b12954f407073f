"""Pins the plain implementation by what fixes it beside the reference's text:
vectors the reference's own tests hold, special cases that reduce to a library
routine, and invariants.  Each is chosen so that a plausible mistake fails it.
"""

import math

import numpy as np
import pytest
import torch

import plain_llama as P


def test_rmsnorm_reference_vector():
    # /root/reference/crates/nnis-model/src/kernels.rs:470-488
    x = torch.tensor([[1.0, -2.0, 3.0, -4.0], [2.0, 1.0, -1.0, 0.5]], dtype=torch.float64)
    w = torch.tensor([0.5, 1.0, 1.5, 2.0], dtype=torch.float64)
    got = P.rms_norm(x, w, 1e-5)
    # row 0: mean square 7.5; row 1: 1.5625 -- worked by hand, eps inside the root
    s0, s1 = 1.0 / math.sqrt(7.5 + 1e-5), 1.0 / math.sqrt(1.5625 + 1e-5)
    want = torch.tensor([[0.5 * s0, -2.0 * s0, 4.5 * s0, -8.0 * s0], [1.0 * s1, 1.0 * s1, -1.5 * s1, 1.0 * s1]])
    assert torch.allclose(got, want.double(), atol=1e-12)
    # eps outside the root, a sum instead of a mean, or a "1 + w" gain would all miss these
    assert abs(got[0, 0].item() - 0.18257406) < 1e-7
    assert abs(got[1, 2].item() - (-1.19999616)) < 1e-7


def test_rmsnorm_invariants():
    torch.manual_seed(0)
    x = torch.randn(5, 37, dtype=torch.float64)
    ones = torch.ones(37, dtype=torch.float64)
    y = P.rms_norm(x, ones, 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-9)  # unit RMS
    assert torch.allclose(P.rms_norm(3.0 * x, ones, 1e-12), y, atol=1e-9)  # scale invariance
    w = torch.randn(37, dtype=torch.float64)
    assert torch.allclose(P.rms_norm(x, w, 1e-6), x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w)


def test_linear_orientation():
    # the checkpoint's [out, in] matrix; /root/reference/crates/nnis-model/src/safetensors_loader.rs:1063-1072
    w = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    x = torch.tensor([[1.0, 0.0, -1.0]])
    assert torch.equal(P.linear(x, w), torch.tensor([[-2.0, -2.0]]))
    assert torch.equal(w.t().contiguous().flatten(), torch.tensor([1.0, 4.0, 2.0, 5.0, 3.0, 6.0]))


def test_rope_reference_vector():
    # /root/reference/crates/nnis-model/src/runtime_kernels.rs:306-341: 2 heads of 4, table row 1
    x = torch.tensor([1.0, 2.0, 3.0, 4.0, -1.0, 0.5, 2.0, -3.0]).view(1, 2, 4)
    cos = torch.tensor([[0.5, -0.25]])
    sin = torch.tensor([[0.25, 0.75]])
    got = P.rope_rotate_half(x, cos, sin).flatten()
    want = torch.tensor([-0.25, -3.5, 1.75, 0.5, -1.0, 2.125, 0.75, 1.125])
    assert torch.allclose(got, want, atol=1e-6)


def test_rope_tables_and_invariants():
    cos, sin = P.rope_tables(64, 16, 10000.0)
    assert cos.dtype == np.float32 and cos.shape == (64, 8)
    assert np.all(cos[0] == 1.0) and np.all(sin[0] == 0.0)  # position 0 is the identity
    assert np.allclose(cos[:, 0], np.cos(np.arange(64)), atol=1e-6)  # pair 0 turns by one radian a position
    inv = 1.0 / 10000.0 ** (np.arange(8) * 2 / 16)
    assert np.allclose(cos[7], np.cos(7 * inv), atol=1e-6) and np.allclose(sin[7], np.sin(7 * inv), atol=1e-6)

    torch.manual_seed(1)
    x = torch.randn(64, 3, 16, dtype=torch.float64)
    c, s = torch.from_numpy(cos).double(), torch.from_numpy(sin).double()
    y = P.rope_rotate_half(x, c, s)
    assert torch.equal(y[0], x[0])
    # each (x[j], x[j+half]) pair keeps its norm
    assert torch.allclose(y[..., :8] ** 2 + y[..., 8:] ** 2, x[..., :8] ** 2 + x[..., 8:] ** 2, atol=1e-9)
    # equals the complex product (x[j] + i x[j+half]) * exp(i pos inv_freq_j)
    z = torch.complex(x[..., :8], x[..., 8:]) * torch.complex(c, s)[:, None, :]
    assert torch.allclose(y, torch.cat([z.real, z.imag], -1), atol=1e-12)
    # only distances count: <rope(q, m), rope(k, n)> depends on m - n (a wrong sign or pairing breaks this)
    q, k = torch.randn(1, 1, 16, dtype=torch.float64), torch.randn(1, 1, 16, dtype=torch.float64)

    def score(m, n):
        a = P.rope_rotate_half(q, c[m:m + 1], s[m:m + 1])
        b = P.rope_rotate_half(k, c[n:n + 1], s[n:n + 1])
        return (a * b).sum().item()

    assert abs(score(5, 2) - score(40, 37)) < 1e-5
    assert abs(score(9, 9) - score(0, 0)) < 1e-5
    assert abs(score(5, 2) - score(2, 5)) > 1e-3  # and the direction of the distance matters


def test_attention_reference_vectors():
    # /root/reference/crates/nnis-model/src/kernels.rs:501-558: two cached positions, scale 1
    k = torch.tensor([[[1.0, 0.0], [1.0, 1.0]], [[0.0, 1.0], [-1.0, 1.0]]])  # [pos][kv head][d]
    v = torch.tensor([[[10.0, 0.0], [1.0, 2.0]], [[0.0, 20.0], [3.0, 4.0]]])
    e, e2 = math.e, math.exp(2.0)
    q = torch.zeros(2, 2, 2)
    q[1] = torch.tensor([[1.0, 0.0], [0.0, 1.0]])
    out = P.causal_attention(q, k, v, 1.0)[1].flatten()
    assert torch.allclose(out, torch.tensor([10 * e / (e + 1), 20 / (e + 1), 2.0, 3.0]), atol=2e-5)
    # four query heads on two key/value heads: consecutive query heads share one
    q = torch.zeros(2, 4, 2)
    q[1] = torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 0.0], [0.0, 1.0]])
    out = P.causal_attention(q, k, v, 1.0)[1].flatten()
    want = torch.tensor([10 * e / (e + 1), 20 / (e + 1), 10 / (e + 1), 20 * e / (e + 1),
                         (e2 + 3) / (e2 + 1), (2 * e2 + 4) / (e2 + 1), 2.0, 3.0])
    assert torch.allclose(out, want, atol=2e-5)


def test_attention_special_cases():
    torch.manual_seed(2)
    t, nh, nkv, hd = 9, 6, 2, 8
    q = torch.randn(t, nh, hd, dtype=torch.float64)
    k = torch.randn(t, nkv, hd, dtype=torch.float64)
    v = torch.randn(t, nkv, hd, dtype=torch.float64)
    scale = 1.0 / math.sqrt(hd)
    out = P.causal_attention(q, k, v, scale)
    # a single visible position gives back its value row
    assert torch.allclose(out[0], v[0].repeat_interleave(nh // nkv, dim=0))
    # grouped heads equal full heads after repeating keys and values per group
    kk, vv = k.repeat_interleave(nh // nkv, dim=1), v.repeat_interleave(nh // nkv, dim=1)
    assert torch.allclose(out, P.causal_attention(q, kk, vv, scale), atol=1e-12)
    # the library routine: causal, and the last row against the unmasked product
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True, scale=scale).transpose(0, 1)
    assert torch.allclose(out, lib, atol=1e-10)
    full = torch.softmax(torch.einsum("hd,thd->ht", q[-1], kk) * scale, -1)
    assert torch.allclose(out[-1], torch.einsum("ht,thd->hd", full, vv), atol=1e-10)
    # equal keys: the output is the mean of the visible values
    same = k[:1].expand(t, nkv, hd)
    mean = P.causal_attention(q, same, v, scale)
    assert torch.allclose(mean[4, 0], v[:5, 0].mean(0), atol=1e-10)
    # a key far ahead of the query changes nothing (causality)
    k2, v2 = k.clone(), v.clone()
    k2[-1] += 100.0
    v2[-1] -= 50.0
    assert torch.equal(P.causal_attention(q, k2, v2, scale)[:-1], out[:-1])


def test_silu_and_gated_feed_forward():
    from scipy.special import expit

    x = torch.linspace(-6, 6, 25, dtype=torch.float64)
    assert torch.allclose(P.silu(x), x * torch.from_numpy(expit(x.numpy())), atol=1e-12)
    assert P.silu(torch.zeros(1)).item() == 0.0
    torch.manual_seed(3)
    m = torch.randn(4, 6, dtype=torch.float64)
    wg, wu, wd = (torch.randn(s, dtype=torch.float64) for s in ((10, 6), (10, 6), (6, 10)))
    got = P.swiglu(m, wg, wu, wd)
    assert torch.allclose(got, (P.silu(m @ wg.t()) * (m @ wu.t())) @ wd.t())
    # the activation sits on the gate branch: swapping gate and up changes the result
    assert not torch.allclose(got, P.swiglu(m, wu, wg, wd))


def test_bf16_widening_is_bits_shift():
    # /root/reference/crates/nnis-model/src/safetensors_loader.rs:951-968: every one of the 65,536 encodings
    bits = torch.arange(65536, dtype=torch.int32)
    as_bf16 = bits.to(torch.int16).view(torch.bfloat16)
    widened = as_bf16.to(torch.float32).view(torch.int32)
    finite = ~torch.isnan(as_bf16.to(torch.float32))
    assert torch.equal(widened[finite], (bits << 16)[finite])
    assert torch.equal(P.bf16_round(as_bf16.to(torch.float32))[finite], as_bf16.to(torch.float32)[finite])


def test_splitmix_vector_and_sampler_rules():
    # /root/reference/crates/nnis-model/src/sampling.rs:319-362
    rng = P.PlainSplitMix64(42)
    assert [P.plain_sample(np.zeros(4, np.float32), rng) for _ in range(10)] == [2, 0, 1, 1, 0, 3, 0, 3, 1, 2]
    assert P.plain_sample(np.array([1.0, 4.0, 4.0, -2.0], np.float32), P.PlainSplitMix64(7), top_k=1) == 1
    rng = P.PlainSplitMix64(9)
    assert all(P.plain_sample(np.array([3.0, 2.0, 1.0], np.float32), rng, top_p=0.1) == 0 for _ in range(32))
    rng = P.PlainSplitMix64(123)
    assert all(P.plain_sample(np.array([4.0, 3.0, 2.0, 1.0], np.float32), rng, top_k=2) <= 1 for _ in range(64))
    with pytest.raises(ValueError):
        P.plain_sample(np.array([1.0, np.nan], np.float32), P.PlainSplitMix64(1))


def test_sampler_frequencies_follow_softmax():
    logits = np.array([2.0, 1.0, 0.0, -1.0, -30.0], np.float32)
    rng = P.PlainSplitMix64(2024)
    draws = np.bincount([P.plain_sample(logits, rng, temperature=0.7) for _ in range(20000)], minlength=5)
    want = np.exp(logits / 0.7)
    want /= want.sum()
    assert np.abs(draws / draws.sum() - want).max() < 0.012
    assert draws[4] == 0


def test_whole_model_special_cases(model_dirs, tmp_path):
    """Zero output and down projections make every layer the identity, so the
    logits are head(norm(embedding)); a model whose embedding rows are all
    equal gives equal logits and greedy token 0
    (/root/reference/crates/nnis-model/src/runtime.rs:1220-1275)."""
    model = P.PlainLlama(model_dirs["B"], torch.float64)
    for name in list(model.w):
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            model.w[name] = torch.zeros_like(model.w[name])
    ids = [3, 999, 17, 3]
    want = P.linear(P.rms_norm(P.embedding(model.w["model.embed_tokens.weight"], ids), model.w["model.norm.weight"],
                               model.eps), model.w["lm_head.weight"])
    assert torch.allclose(model.logits(ids), want, atol=1e-12)
    model.w["lm_head.weight"] = torch.zeros_like(model.w["lm_head.weight"])
    assert model.greedy([1, 2], 2) == [0, 0]


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_model_invariants(model_dirs, name):
    model = P.PlainLlama(model_dirs[name], torch.float64)
    torch.manual_seed(4)
    ids = torch.randint(0, model.V, (23,)).tolist()
    logits = model.logits(ids)
    assert logits.shape == (23, model.V)
    # causality: a position's logits do not change when later tokens change
    other = ids[:11] + [(t + 1) % model.V for t in ids[11:]]
    assert torch.allclose(model.logits(other)[:11], logits[:11], atol=1e-12)
    assert not torch.allclose(model.logits(other)[11:], logits[11:], atol=1e-6)
    # the 32-bit run agrees with the 64-bit one
    low = P.PlainLlama(model_dirs[name], torch.float32).logits(ids)
    assert (low.double() - logits).abs().max().item() < 2e-5
    # tied head: the embedding stands in
    if model.tied:
        assert "lm_head.weight" not in model.w


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_model_from_library_routines(model_dirs, name):
    """The same model put together a second time from the library's own
    routines, each with its defaults: ``rms_norm`` (eps inside the root, a
    mean), ``scaled_dot_product_attention`` (causal, its default scale
    1/sqrt(head size), grouped heads by repetition), ``silu``, and a rotation
    written as a complex product.  A scale taken before the dot product or
    left out, a norm with eps outside the root, a gate without its
    activation or heads grouped the other way round would all miss this."""
    import torch.nn.functional as F

    model = P.PlainLlama(model_dirs[name], torch.float64)
    w, t = model.w, 29
    torch.manual_seed(5)
    ids = torch.randint(0, model.V, (t,))
    x = F.embedding(ids, w["model.embed_tokens.weight"])
    half = model.hd // 2
    inv_freq = 1.0 / model.theta ** (torch.arange(half, dtype=torch.float64) * 2 / model.hd)
    turn = torch.polar(torch.ones(t, half, dtype=torch.float64), torch.arange(t, dtype=torch.float64)[:, None] * inv_freq)

    def rotate(v):  # [t, heads, hd]: (v[j] + i v[j + half]) * exp(i pos inv_freq_j)
        z = torch.complex(v[..., :half], v[..., half:]) * turn[:, None, :]
        return torch.cat([z.real, z.imag], -1)

    for layer in range(model.L):
        p = f"model.layers.{layer}."
        h = F.rms_norm(x, (model.H,), w[p + "input_layernorm.weight"], model.eps)
        q = rotate(F.linear(h, w[p + "self_attn.q_proj.weight"]).view(t, model.nh, model.hd))
        k = rotate(F.linear(h, w[p + "self_attn.k_proj.weight"]).view(t, model.nkv, model.hd))
        v = F.linear(h, w[p + "self_attn.v_proj.weight"]).view(t, model.nkv, model.hd)
        group = model.nh // model.nkv
        k, v = k.repeat_interleave(group, dim=1), v.repeat_interleave(group, dim=1)
        attn = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        x = x + F.linear(attn.transpose(0, 1).reshape(t, model.nh * model.hd), w[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (model.H,), w[p + "post_attention_layernorm.weight"], model.eps)
        x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                         w[p + "mlp.down_proj.weight"])
    want = F.linear(F.rms_norm(x, (model.H,), w["model.norm.weight"], model.eps), model.lm_head_weight())
    got = model.logits(ids.tolist())
    # the rotation table is built in 32-bit as the reference builds it; in 64-bit here: angles differ by rounding
    assert (got - want).abs().max().item() < 5e-6, (got - want).abs().max().item()
