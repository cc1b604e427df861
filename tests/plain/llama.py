"""A plain, slow Llama 3 decoder: whole sequences, no cache, no pages, no batching.

Every function follows one formula of the reference and cites it.  Nothing here
imports from the product package; the tests compare the engine with this file.

All functions take and return ``torch`` tensors on the CPU and work in the dtype
of their inputs (the tests use float64 or float32).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------- norm
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``w * x * rsqrt(mean(x^2) + eps)`` over the last dim.

    Reference: kvcore/model/layer/rmsnorm.py:23-26 (variance is the mean of the
    squares, eps is added inside the root, the gain multiplies last).
    """
    variance = x.pow(2).mean(dim=-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps))


# ------------------------------------------------------------------- position code
def rope_inv_freq(head_dim: int, theta: float, dtype=torch.float64) -> torch.Tensor:
    """``theta ** (-2j / head_dim)`` for ``j = 0 .. head_dim/2 - 1``.

    Reference: kvcore/model/layer/rotary_embedding.py:63-70.
    """
    exponents = torch.arange(0, head_dim, 2, dtype=dtype) / head_dim
    return 1.0 / (torch.tensor(theta, dtype=dtype) ** exponents)


def llama3_scale_inv_freq(
    inv_freq: torch.Tensor,
    *,
    factor: float,
    low_freq_factor: float,
    high_freq_factor: float,
    original_max_position_embeddings: int,
) -> torch.Tensor:
    """Frequency rescaling named ``rope_type: "llama3"`` in config.json.

    The reference has no rope scaling at all (rotary_embedding.py:52-70 reads only
    the base), so this follows the rule the config keys describe: a frequency whose
    wavelength is shorter than ``original/high_freq_factor`` is kept, one whose
    wavelength is longer than ``original/low_freq_factor`` is divided by ``factor``,
    and between the two the result is a linear blend in ``original/wavelength``.
    """
    out = torch.empty_like(inv_freq)
    orig = float(original_max_position_embeddings)
    for j in range(inv_freq.numel()):
        f = float(inv_freq[j])
        wavelen = 2.0 * math.pi / f
        if wavelen < orig / high_freq_factor:
            out[j] = f
        elif wavelen > orig / low_freq_factor:
            out[j] = f / factor
        else:
            smooth = (orig / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
            out[j] = (1.0 - smooth) * f / factor + smooth * f
    return out


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """``cat(-x[d/2:], x[:d/2])``.  Reference: rotary_embedding.py:10-13."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """Rotate ``x [T, heads, d]`` by the angles ``positions[t] * inv_freq[j]``.

    Element ``j`` pairs with ``j + d/2``.  Reference: rotary_embedding.py:93-97
    (angles, duplicated to the full head) and :33-34 (``x*cos + rotate_half(x)*sin``).
    """
    angles = positions.to(inv_freq.dtype)[:, None] * inv_freq[None, :]
    emb = torch.cat((angles, angles), dim=-1)
    cos = emb.cos().to(x.dtype)[:, None, :]
    sin = emb.sin().to(x.dtype)[:, None, :]
    return x * cos + rotate_half(x) * sin


# ----------------------------------------------------------------------- attention
def causal_gqa_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: float,
    window: int | None = None,
) -> torch.Tensor:
    """Causal attention of one whole sequence with grouped query heads.

    ``q [T, nh, d]``, ``k, v [T, nkv, d]`` -> ``[T, nh, d]``.  Query head ``h`` reads
    KV head ``h // (nh/nkv)``; token ``t`` sees keys ``0..t`` (with ``window`` only the
    last ``window`` of them); scores are scaled, then softmax, then times V.
    Reference: kvcore/model/attn_backend/torch_paged.py:90-117 (loop per token and
    head over the visible keys) and :169-201 (scores * scale, softmax, probs @ V).
    """
    T, nh, _ = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    out = torch.empty_like(q)
    for t in range(T):
        first = 0 if window is None else max(0, t - window + 1)
        for h in range(nh):
            hk = h // group
            keys = k[first : t + 1, hk]
            values = v[first : t + 1, hk]
            scores = (keys @ q[t, h]) * scale
            probs = torch.softmax(scores, dim=0)
            out[t, h] = probs @ values
    return out


# -------------------------------------------------------------------- feed-forward
def silu_and_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(first half) * second half``.  Reference: layer/activation.py:14-16."""
    half = gate_up.shape[-1] // 2
    gate, up = gate_up[..., :half], gate_up[..., half:]
    return gate * torch.sigmoid(gate) * up


def swiglu_mlp(
    x: torch.Tensor,
    gate_w: torch.Tensor,
    up_w: torch.Tensor,
    down_w: torch.Tensor,
    gate_b: torch.Tensor | None = None,
    up_b: torch.Tensor | None = None,
    down_b: torch.Tensor | None = None,
) -> torch.Tensor:
    """``down(silu(gate(x)) * up(x))``.  Reference: models/llama3.py:42-45 with the
    stacked gate_up projection of :34-38 (gate rows first, then up rows)."""
    gate = x @ gate_w.T
    up = x @ up_w.T
    if gate_b is not None:
        gate = gate + gate_b
    if up_b is not None:
        up = up + up_b
    y = silu_and_mul(torch.cat((gate, up), dim=-1)) @ down_w.T
    if down_b is not None:
        y = y + down_b
    return y


# ------------------------------------------------------------------------- a layer
def attention_block(
    x: torch.Tensor,
    positions: torch.Tensor,
    w: dict[str, torch.Tensor],
    prefix: str,
    *,
    num_heads: int,
    num_kv_heads: int,
    head_dim: int,
    inv_freq: torch.Tensor,
    window: int | None = None,
) -> torch.Tensor:
    """q/k/v projections, rotation of q and k, attention, output projection.

    Reference: models/llama3.py:92-103; the scale ``head_dim ** -0.5`` is :60.
    """
    T = x.shape[0]

    def proj(name: str) -> torch.Tensor:
        y = x @ w[f"{prefix}.{name}.weight"].T
        bias = w.get(f"{prefix}.{name}.bias")
        return y if bias is None else y + bias

    q = proj("q_proj").view(T, num_heads, head_dim)
    k = proj("k_proj").view(T, num_kv_heads, head_dim)
    v = proj("v_proj").view(T, num_kv_heads, head_dim)
    q = apply_rope(q, positions, inv_freq)
    k = apply_rope(k, positions, inv_freq)
    o = causal_gqa_attention(q, k, v, head_dim**-0.5, window=window)
    y = o.reshape(T, num_heads * head_dim) @ w[f"{prefix}.o_proj.weight"].T
    bias = w.get(f"{prefix}.o_proj.bias")
    return y if bias is None else y + bias


def llama_config_values(config: dict) -> dict:
    """The numbers the forward pass needs, with the reference's defaults.

    ``num_key_value_heads`` defaults to the head count (engine_core.py:164),
    ``head_dim`` to ``hidden // heads`` (llama3.py:59), the rope base to
    ``rope_parameters.rope_theta``, ``rope_theta`` or 10000 (rotary_embedding.py:38-49).
    """
    nh = config["num_attention_heads"]
    rope_params = config.get("rope_parameters") or {}
    theta = rope_params.get("rope_theta", rope_params.get("theta", config.get("rope_theta", 10000.0)))
    scaling = config.get("rope_scaling")
    if scaling is None and rope_params.get("rope_type", "default") not in ("default", None):
        scaling = rope_params
    return dict(
        L=config["num_hidden_layers"],
        H=config["hidden_size"],
        nh=nh,
        nkv=config.get("num_key_value_heads") or nh,
        d=config.get("head_dim") or config["hidden_size"] // nh,
        eps=config["rms_norm_eps"],
        theta=float(theta),
        scaling=scaling,
        tied=bool(config.get("tie_word_embeddings", False)),
    )


def model_inv_freq(config: dict, dtype=torch.float64) -> torch.Tensor:
    c = llama_config_values(config)
    inv_freq = rope_inv_freq(c["d"], c["theta"], dtype=dtype)
    scaling = c["scaling"]
    if scaling is not None and scaling.get("rope_type", scaling.get("type", "default")) == "llama3":
        inv_freq = llama3_scale_inv_freq(
            inv_freq,
            factor=scaling["factor"],
            low_freq_factor=scaling["low_freq_factor"],
            high_freq_factor=scaling["high_freq_factor"],
            original_max_position_embeddings=scaling["original_max_position_embeddings"],
        )
    return inv_freq


def llama_forward(
    config: dict,
    weights: dict[str, torch.Tensor],
    token_ids: list[int] | torch.Tensor,
    *,
    dtype=torch.float64,
    position_offset: int = 0,
) -> torch.Tensor:
    """Logits ``[T, V]`` of one whole sequence.

    Reference: models/llama3.py:189-200 (embedding, layers, final norm) and :124-142
    (layer: norm, attention, add, norm, MLP, add; written there with a carried
    ``residual``, which is the same sum); the head is :245-247 and, when
    ``tie_word_embeddings`` is set, shares the embedding matrix (:224-225).
    ``position_offset`` shifts every position (for the test of the rotation).
    """
    c = llama_config_values(config)
    w = {name: t.to(dtype) for name, t in weights.items()}
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    positions = torch.arange(ids.numel()) + position_offset
    inv_freq = model_inv_freq(config, dtype=dtype)

    r = w["model.embed_tokens.weight"][ids]
    for i in range(c["L"]):
        p = f"model.layers.{i}"
        x = rms_norm(r, w[f"{p}.input_layernorm.weight"], c["eps"])
        r = r + attention_block(
            x, positions, w, f"{p}.self_attn",
            num_heads=c["nh"], num_kv_heads=c["nkv"], head_dim=c["d"], inv_freq=inv_freq,
        )
        x = rms_norm(r, w[f"{p}.post_attention_layernorm.weight"], c["eps"])
        r = r + swiglu_mlp(
            x,
            w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"], w[f"{p}.mlp.down_proj.weight"],
            w.get(f"{p}.mlp.gate_proj.bias"), w.get(f"{p}.mlp.up_proj.bias"), w.get(f"{p}.mlp.down_proj.bias"),
        )
    x = rms_norm(r, w["model.norm.weight"], c["eps"])
    head = w["model.embed_tokens.weight"] if c["tied"] else w["lm_head.weight"]
    return x @ head.T


def load_model_folder(folder: str | Path) -> tuple[dict, dict[str, torch.Tensor]]:
    """config.json and every tensor of the folder's safetensors files, read with the
    safetensors library (the product has a reader of its own)."""
    from safetensors.torch import load_file

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    weights: dict[str, torch.Tensor] = {}
    for file in sorted(folder.glob("*.safetensors")):
        weights.update(load_file(str(file)))
    return config, weights


def greedy_generate(config: dict, weights: dict, prompt: list[int], n: int, dtype=torch.float64) -> list[int]:
    """``n`` tokens by repeated whole-sequence forward and argmax of the last row."""
    ids = list(prompt)
    out: list[int] = []
    for _ in range(n):
        logits = llama_forward(config, weights, ids, dtype=dtype)
        nxt = int(torch.argmax(logits[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out
