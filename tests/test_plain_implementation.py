"""Pins the plain implementation by what fixes it beside the reference's text: vectors
the reference's tests hold, special cases that reduce to a library routine, and
invariants, each chosen so that a plausible mistake fails it."""

from __future__ import annotations

import math

import pytest
import torch
import torch.nn.functional as F

from tests.helpers import TINY_A, TINY_B, random_tokens
from tests.plain import llama as plain
from tests.plain import sampling as plain_sampling

torch.manual_seed(0)


# ------------------------------------------------------------------------------ norm
def test_rms_norm_with_unit_gain_is_the_library_routine():
    x = torch.randn(5, 96, dtype=torch.float64)
    got = plain.rms_norm(x, torch.ones(96, dtype=torch.float64), 1e-6)
    want = F.rms_norm(x, (96,), eps=1e-6)
    assert torch.allclose(got, want, atol=1e-12)


def test_rms_norm_eps_is_inside_the_root_and_gain_is_last():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    w = torch.tensor([2.0, 0.5], dtype=torch.float64)
    eps = 0.5  # large, so that eps outside the root or on the squares would show
    want = w * x / math.sqrt((9 + 16) / 2 + eps)
    assert torch.allclose(plain.rms_norm(x, w, eps), want, atol=1e-12)


def test_rms_norm_is_scale_free_and_has_unit_mean_square():
    x = torch.randn(4, 64, dtype=torch.float64)
    one = torch.ones(64, dtype=torch.float64)
    y = plain.rms_norm(x, one, 1e-12)
    assert torch.allclose(plain.rms_norm(7.5 * x, one, 1e-12), y, atol=1e-9)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(4, dtype=torch.float64), atol=1e-9)


# -------------------------------------------------------------------------- rotation
def test_rope_position_zero_is_the_identity_and_norms_are_kept():
    inv = plain.rope_inv_freq(32, 10000.0)
    x = torch.randn(3, 2, 32, dtype=torch.float64)
    assert torch.allclose(plain.apply_rope(x, torch.zeros(3, dtype=torch.long), inv), x)
    y = plain.apply_rope(x, torch.tensor([5, 17, 101]), inv)
    half = 16
    pair_norm = lambda t: t[..., :half] ** 2 + t[..., half:] ** 2  # noqa: E731
    assert torch.allclose(pair_norm(y), pair_norm(x), atol=1e-12)


def test_rope_pairs_element_j_with_j_plus_half():
    inv = plain.rope_inv_freq(16, 10000.0)
    for j in range(8):
        x = torch.zeros(1, 1, 16, dtype=torch.float64)
        x[0, 0, j] = 1.0
        y = plain.apply_rope(x, torch.tensor([3]), inv)[0, 0]
        moved = set(torch.nonzero(y.abs() > 1e-12).flatten().tolist())
        assert moved <= {j, j + 8} and j + 8 in moved
        # rotation by a positive angle: (1, 0) -> (cos, +sin); a wrong sign gives -sin
        assert y[j] == pytest.approx(math.cos(3 * float(inv[j])))
        assert y[j + 8] == pytest.approx(math.sin(3 * float(inv[j])))


def test_rope_scores_depend_on_distance_only():
    inv = plain.rope_inv_freq(32, 500000.0)
    q = torch.randn(1, 1, 32, dtype=torch.float64)
    k = torch.randn(1, 1, 32, dtype=torch.float64)
    def score(m, n):
        return float((plain.apply_rope(q, torch.tensor([m]), inv) * plain.apply_rope(k, torch.tensor([n]), inv)).sum())
    assert score(9, 4) == pytest.approx(score(109, 104), abs=1e-9)
    assert score(9, 4) != pytest.approx(score(9, 5), abs=1e-6)


def test_inv_freq_is_the_reference_table():
    inv = plain.rope_inv_freq(8, 10000.0)
    want = [1.0, 10000 ** -0.25, 10000 ** -0.5, 10000 ** -0.75]
    assert torch.allclose(inv, torch.tensor(want, dtype=torch.float64))


def test_llama3_scaling_bands():
    d, theta = 32, 500000.0
    inv = plain.rope_inv_freq(d, theta)
    kw = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    out = plain.llama3_scale_inv_freq(inv, **kw)
    wavelen = 2 * math.pi / inv
    high = wavelen < 64 / 4
    low = wavelen > 64 / 1
    mid = ~high & ~low
    assert high.sum() == 2 and mid.sum() == 1 and low.sum() == 13  # every band is hit
    assert torch.equal(out[high], inv[high])
    assert torch.allclose(out[low], inv[low] / 8.0, rtol=1e-15)
    assert (out[mid] < inv[mid]).all() and (out[mid] > inv[mid] / 8.0).all()
    # factor 1 changes nothing; the result stays monotone in the index
    same = plain.llama3_scale_inv_freq(inv, **{**kw, "factor": 1.0})
    assert torch.allclose(same, inv, rtol=1e-15)
    assert (out[1:] < out[:-1]).all()


def test_llama3_blend_is_continuous_at_both_band_edges_and_hits_a_hand_worked_value():
    """What pins the blend's direction.  At a wavelength just inside the middle band next to
    the short-wave edge (``original / high``) the result must meet the kept frequency, and
    next to the long-wave edge (``original / low``) the divided one; a blend with ``s`` and
    ``1 - s`` exchanged jumps by a factor of ``factor`` at both.  And config B's one blended
    index, worked by hand from the rule of the config keys: d = 32, theta = 5e5, index 2:
    ln 5e5 = 13.1223634, so inv_freq = exp(-13.1223634 / 8) = 0.193923, wavelength 2 pi /
    inv_freq = 32.4004, original / wavelength = 64 / 32.4004 = 1.975284, s = (1.975284 - 1) /
    (4 - 1) = 0.325095, (1 - s) / 8 + s = 0.084363 + 0.325095 = 0.409458 (with s and 1 - s
    exchanged it would be 0.715542)."""
    from kvcore_amd.parts.rotary import rotary_inv_freq

    kw = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    inv = plain.rope_inv_freq(32, 500000.0)
    out = plain.llama3_scale_inv_freq(inv, **kw)
    assert float(out[2] / inv[2]) == pytest.approx(0.409458, abs=5e-6)
    product = rotary_inv_freq(32, 500000.0, {"rope_type": "llama3", **kw})
    assert float(product[2]) / float(inv[2]) == pytest.approx(0.409458, abs=5e-6)

    def scaled(wavelen):
        f = torch.tensor([2 * math.pi / wavelen], dtype=torch.float64)
        return float(plain.llama3_scale_inv_freq(f, **kw)[0]), float(f[0])

    short_edge, long_edge = 64 / 4.0, 64 / 1.0
    got, f = scaled(short_edge * (1 + 1e-9))   # just inside the middle band
    assert got == pytest.approx(f, rel=1e-6)   # meets the band that is kept
    got, f = scaled(short_edge * (1 - 1e-9))
    assert got == f
    got, f = scaled(long_edge * (1 - 1e-9))    # just inside the middle band
    assert got == pytest.approx(f / 8.0, rel=1e-6)  # meets the band that is divided
    got, f = scaled(long_edge * (1 + 1e-9))
    assert got == pytest.approx(f / 8.0, rel=1e-12)
    # the middle of the band in original / wavelength (2.5 of 1..4) is the mean of both
    got, f = scaled(64 / 2.5)
    assert got == pytest.approx(0.5 * (f + f / 8.0), rel=1e-12)
    # the product's own table follows the same rule at the sizes of the large models
    for d, theta, factor in ((128, 500000.0, 8.0), (64, 500000.0, 32.0)):
        big = dict(factor=factor, low_freq_factor=1.0, high_freq_factor=4.0,
                   original_max_position_embeddings=8192)
        want = plain.llama3_scale_inv_freq(plain.rope_inv_freq(d, theta), **big)
        have = rotary_inv_freq(d, theta, {"rope_type": "llama3", **big})
        assert torch.allclose(have.double(), want, rtol=1e-6)
        wl = 2 * math.pi / plain.rope_inv_freq(d, theta)
        assert ((wl >= 8192 / 4) & (wl <= 8192)).sum() >= 3, "some indices are blended at these sizes"


# ------------------------------------------------------------------------- attention
def test_attention_equals_library_causal_attention():
    T, nh, nkv, d = 9, 6, 2, 16
    q = torch.randn(T, nh, d, dtype=torch.float64)
    k = torch.randn(T, nkv, d, dtype=torch.float64)
    v = torch.randn(T, nkv, d, dtype=torch.float64)
    got = plain.causal_gqa_attention(q, k, v, d ** -0.5)
    kr = k.repeat_interleave(nh // nkv, dim=1)
    vr = v.repeat_interleave(nh // nkv, dim=1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kr.transpose(0, 1)[None],
                                          vr.transpose(0, 1)[None], is_causal=True, scale=d ** -0.5)
    assert torch.allclose(got, want[0].transpose(0, 1), atol=1e-12)


def test_attention_first_token_returns_its_value_and_equal_keys_average():
    T, d = 5, 16
    q = torch.randn(T, 1, d, dtype=torch.float64)
    v = torch.randn(T, 1, d, dtype=torch.float64)
    k = torch.randn(1, 1, d, dtype=torch.float64).expand(T, 1, d)
    out = plain.causal_gqa_attention(q, k, v, 0.3)
    assert torch.allclose(out[0], v[0])
    assert torch.allclose(out[-1, 0], v[:, 0].mean(0))


def test_attention_group_mapping_is_head_floor_div_group():
    T, nh, nkv, d = 4, 6, 3, 16
    q = torch.randn(T, nh, d, dtype=torch.float64)
    k = torch.randn(T, nkv, d, dtype=torch.float64)
    v = torch.arange(nkv, dtype=torch.float64)[None, :, None].expand(T, nkv, d).clone()
    out = plain.causal_gqa_attention(q, k, v, d ** -0.5)
    for h in range(nh):
        assert torch.allclose(out[:, h], torch.full((T, d), float(h // 2), dtype=torch.float64))


def test_attention_decode_after_prefill_vector():
    """The shape of the reference's decode-after-prefill case
    (tests/test_torch_paged_attention.py:211-265): one query at position 4 over five keys
    equals explicit softmax(q K^T * scale) V."""
    d = 8
    k = torch.randn(5, 1, d, dtype=torch.float64)
    v = torch.randn(5, 1, d, dtype=torch.float64)
    q = torch.randn(5, 1, d, dtype=torch.float64)
    out = plain.causal_gqa_attention(q, k, v, d ** -0.5)[4, 0]
    probs = torch.softmax((k[:, 0] @ q[4, 0]) * d ** -0.5, dim=0)
    assert torch.allclose(out, probs @ v[:, 0], atol=1e-12)


def test_attention_window_keeps_the_last_w_keys():
    T, d = 12, 16
    q = torch.randn(T, 2, d, dtype=torch.float64)
    k = torch.randn(T, 1, d, dtype=torch.float64)
    v = torch.randn(T, 1, d, dtype=torch.float64)
    w = 4
    got = plain.causal_gqa_attention(q, k, v, 0.25, window=w)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)) & ~torch.tril(torch.ones(T, T, dtype=torch.bool), -w)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.expand(T, 2, d).transpose(0, 1)[None],
                                          v.expand(T, 2, d).transpose(0, 1)[None], attn_mask=mask, scale=0.25)
    assert torch.allclose(got, want[0].transpose(0, 1), atol=1e-12)


# ---------------------------------------------------------------------- feed-forward
def test_silu_and_mul_gate_is_the_first_half():
    x = torch.randn(3, 10, dtype=torch.float64)
    assert torch.allclose(plain.silu_and_mul(x), F.silu(x[:, :5]) * x[:, 5:])
    x[:, :5] = 0
    assert torch.equal(plain.silu_and_mul(x), torch.zeros(3, 5, dtype=torch.float64))


# ------------------------------------------------------------------------ whole model
def _random_weights(config, seed=0, zero_linear=False):
    g = torch.Generator().manual_seed(seed)
    c = plain.llama_config_values(config)
    H, I, V = c["H"], config["intermediate_size"], config["vocab_size"]
    w = {}
    def lin(*shape):
        t = torch.randn(*shape, generator=g, dtype=torch.float64) * 0.05
        return torch.zeros_like(t) if zero_linear else t
    w["model.embed_tokens.weight"] = torch.randn(V, H, generator=g, dtype=torch.float64)
    for i in range(c["L"]):
        p = f"model.layers.{i}"
        w[f"{p}.input_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g, dtype=torch.float64)
        w[f"{p}.post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g, dtype=torch.float64)
        w[f"{p}.self_attn.q_proj.weight"] = lin(c["nh"] * c["d"], H)
        w[f"{p}.self_attn.k_proj.weight"] = lin(c["nkv"] * c["d"], H)
        w[f"{p}.self_attn.v_proj.weight"] = lin(c["nkv"] * c["d"], H)
        w[f"{p}.self_attn.o_proj.weight"] = lin(H, c["nh"] * c["d"])
        w[f"{p}.mlp.gate_proj.weight"] = lin(I, H)
        w[f"{p}.mlp.up_proj.weight"] = lin(I, H)
        w[f"{p}.mlp.down_proj.weight"] = lin(H, I)
    w["model.norm.weight"] = 1 + 0.1 * torch.randn(H, generator=g, dtype=torch.float64)
    if not c["tied"]:
        w["lm_head.weight"] = torch.randn(V, H, generator=g, dtype=torch.float64) * 0.05
    return w


def test_zero_linear_layers_reduce_the_model_to_head_of_norm_of_embedding():
    w = _random_weights(TINY_A, zero_linear=True)
    w["lm_head.weight"] = torch.randn(TINY_A["vocab_size"], TINY_A["hidden_size"], dtype=torch.float64)
    ids = random_tokens(6, TINY_A["vocab_size"], 1)
    want = plain.rms_norm(w["model.embed_tokens.weight"][ids], w["model.norm.weight"],
                          TINY_A["rms_norm_eps"]) @ w["lm_head.weight"].T
    assert torch.allclose(plain.llama_forward(TINY_A, w, ids), want, atol=1e-12)


def test_tied_head_uses_the_embedding_matrix():
    w = _random_weights(TINY_B)
    ids = random_tokens(5, TINY_B["vocab_size"], 2)
    logits = plain.llama_forward(TINY_B, w, ids)
    w2 = dict(w)
    w2["lm_head.weight"] = torch.zeros(TINY_B["vocab_size"], TINY_B["hidden_size"], dtype=torch.float64)
    assert torch.equal(plain.llama_forward(TINY_B, w2, ids), logits)


def test_model_is_causal_and_depends_on_position_distances_only():
    w = _random_weights(TINY_A, seed=3)
    ids = random_tokens(12, TINY_A["vocab_size"], 3)
    full = plain.llama_forward(TINY_A, w, ids)
    assert torch.allclose(plain.llama_forward(TINY_A, w, ids[:7]), full[:7], atol=1e-12)
    shifted = plain.llama_forward(TINY_A, w, ids, position_offset=37)
    assert torch.allclose(shifted, full, atol=1e-9)
    swapped = list(ids)
    swapped[2], swapped[5] = swapped[5], swapped[2]
    assert not torch.allclose(plain.llama_forward(TINY_A, w, swapped)[-1], full[-1], atol=1e-6)


def test_layer_order_matches_the_carried_residual_form():
    """kvcore/model/models/llama3.py:124-142 carries (hidden, residual) and lets each norm
    add first; the plain model writes r += f(norm(r)).  Both are computed here."""
    config = dict(TINY_A)
    w = _random_weights(config, seed=5)
    c = plain.llama_config_values(config)
    ids = torch.tensor(random_tokens(9, config["vocab_size"], 4))
    pos = torch.arange(9)
    inv = plain.model_inv_freq(config)
    hidden, residual = w["model.embed_tokens.weight"][ids], None
    for i in range(c["L"]):
        p = f"model.layers.{i}"
        if residual is None:
            residual = hidden
        else:
            residual = hidden + residual
        hidden = plain.rms_norm(residual, w[f"{p}.input_layernorm.weight"], c["eps"])
        hidden = plain.attention_block(hidden, pos, w, f"{p}.self_attn", num_heads=c["nh"],
                                       num_kv_heads=c["nkv"], head_dim=c["d"], inv_freq=inv)
        residual = hidden + residual
        hidden = plain.rms_norm(residual, w[f"{p}.post_attention_layernorm.weight"], c["eps"])
        hidden = plain.swiglu_mlp(hidden, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                                  w[f"{p}.mlp.down_proj.weight"])
    out = plain.rms_norm(hidden + residual, w["model.norm.weight"], c["eps"]) @ w["lm_head.weight"].T
    assert torch.allclose(plain.llama_forward(config, w, ids.tolist()), out, atol=1e-12)


# -------------------------------------------------------------------------- sampling
def test_greedy_vectors_of_the_reference():
    """tests/test_sampler.py:29-35."""
    assert plain_sampling.sample(torch.tensor([0.0, 2.0, 1.0]), temperature=0.0) == 1
    assert plain_sampling.sample(torch.tensor([4.0, 3.0, 2.0]), temperature=0.0) == 0


def test_top_k_and_top_p_vectors_of_the_reference():
    """tests/test_sampler.py:49-68."""
    f = plain_sampling.apply_top_k_top_p(torch.tensor([1.0, 2.0, 3.0, 4.0]), 2, None)
    assert torch.isneginf(f[:2]).all() and torch.isfinite(f[2:]).all()
    f = plain_sampling.apply_top_k_top_p(torch.tensor([10.0, 9.0, 0.0, -1.0]), None, 0.8)
    assert torch.isfinite(f[:2]).all() and torch.isneginf(f[2:]).all()


def test_top_k_one_is_greedy_whatever_the_noise():
    """tests/test_sampler.py:71-81: top_k=1 with a seed returns the argmax."""
    assert plain_sampling.sample(torch.tensor([5.0, 1.0]), temperature=1.0, top_k=1, seed=7) == 0


def test_sampling_is_reproducible_fresh_per_token_and_follows_the_probabilities():
    logits = torch.tensor([1.0, 0.0, 2.0, -1.0, 0.5])
    draws = [plain_sampling.sample(logits, temperature=0.8, seed=42, index=i) for i in range(4000)]
    again = [plain_sampling.sample(logits, temperature=0.8, seed=42, index=i) for i in range(50)]
    assert draws[:50] == again
    assert len(set(draws[:50])) > 1  # successive tokens draw different noise
    probs = torch.softmax(logits.double() / 0.8, dim=0)
    counts = torch.bincount(torch.tensor(draws), minlength=5).double()
    chi2 = float(((counts - 4000 * probs) ** 2 / (4000 * probs)).sum())
    assert chi2 < 18.5  # 4 degrees of freedom, p = 0.001
    u = plain_sampling.uniform_noise(1, 0, 1000)
    assert float(u.min()) > 0.0 and float(u.max()) < 1.0
