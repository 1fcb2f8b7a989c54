"""Plain, slow Qwen2 forward: whole sequences, no cache, one function per part.

This file is the oracle of the test-suite. It shares no code with the
`distie_amd` package: it reads `config.json` as a plain dict, reads weights
with the `safetensors` library, and computes in whatever dtype the caller
gives (float32 by default, float64 for the pinning tests).

Every function cites the lines of the reference (paths relative to the
reference checkout) whose formula it restates.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch


# --------------------------------------------------------------------------
# configuration (plain dict; only what the formulas need)
# --------------------------------------------------------------------------

def read_config(model_dir) -> dict:
    """config.json as a dict. Keys read: worker/src/inference/qwen2/model.py:41-74."""
    return json.loads((Path(model_dir) / "config.json").read_text())


def head_dim_of(cfg: dict) -> int:
    """`head_dim` if given, else hidden // heads: worker/src/inference/qwen2/model.py:47-48."""
    explicit = cfg.get("head_dim")
    return int(explicit) if explicit else int(cfg["hidden_size"]) // int(cfg["num_attention_heads"])


def rope_theta_of(cfg: dict) -> float:
    """`rope_parameters.rope_theta` wins over `rope_theta`: worker/src/inference/qwen2/model.py:413-419."""
    params = cfg.get("rope_parameters") or {}
    if "rope_theta" in params:
        return float(params["rope_theta"])
    return float(cfg["rope_theta"])


def layer_windows(cfg: dict) -> list:
    """Window of each layer (None = every earlier key is visible).

    The reference rejects windowed layers (worker/src/inference/qwen2/model.py:58-60),
    so the rule is this build's: `layer_types` wins when present (the strings are
    those of worker/tests/test_qwen2.py:67); otherwise layer l is windowed iff
    `use_sliding_window` and l >= `max_window_layers`.
    """
    n = int(cfg["num_hidden_layers"])
    window = cfg.get("sliding_window")
    types = cfg.get("layer_types")
    if types:
        return [int(window) if t == "sliding_attention" else None for t in types]
    if not cfg.get("use_sliding_window", False) or window is None:
        return [None] * n
    first = int(cfg.get("max_window_layers", n))
    return [int(window) if l >= first else None for l in range(n)]


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * weight: worker/src/inference/qwen2/model.py:85-90."""
    variance = x.pow(2).mean(-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps))


def rope_inv_freq(head_dim: int, theta: float, dtype=torch.float32) -> torch.Tensor:
    """theta^(-2i/D), i = 0..D/2-1: worker/src/inference/qwen2/model.py:98."""
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=dtype) / head_dim))


def rope_cos_sin(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float32,
                 angle_dtype=torch.float32):
    """cos/sin of concat(ang, ang), ang = pos * inv_freq: worker/src/inference/qwen2/model.py:101-105.
    Frequencies, angles and the trigonometry are float32 whatever `dtype` is (`.float()` at :98 and
    :103), and only the results take the dtype of the activations (:105): at position 2,000 a
    float32 angle is off by up to 1e-4 rad, which is part of what the reference computes.
    (`angle_dtype=float64` is for tests of the formula itself.)"""
    freqs = positions.to(angle_dtype)[:, None] * rope_inv_freq(head_dim, theta, angle_dtype).to(positions.device)[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """concat(-x[D/2:], x[:D/2]): worker/src/inference/qwen2/model.py:115-117."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x*cos + rotate_half(x)*sin; x [T, heads, D], cos/sin [T, D]:
    worker/src/inference/qwen2/model.py:108-112."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """Each kv head repeated n_rep times in a row; x [T, KH, D] -> [T, KH*n_rep, D]:
    worker/src/inference/qwen2/model.py:120-125."""
    t, kh, d = x.shape
    return x[:, :, None, :].expand(t, kh, n_rep, d).reshape(t, kh * n_rep, d)


def visibility(q_len: int, window, device=None) -> torch.Tensor:
    """[q, k] bool: key k visible to query q iff k <= q (worker/src/inference/qwen2/model.py:128-135)
    and, on a windowed layer, q - k < window (this build's rule)."""
    q = torch.arange(q_len, device=device)[:, None]
    k = torch.arange(q_len, device=device)[None, :]
    seen = k <= q
    if window is not None:
        seen = seen & (q - k < window)
    return seen


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window=None) -> torch.Tensor:
    """softmax(q k^T * D^-0.5 + mask) v with q [T,H,D], k/v [T,KH,D] -> [T,H,D]:
    worker/src/inference/qwen2/model.py:154-161 (scale after the product, :157)."""
    t, h, d = q.shape
    n_rep = h // k.shape[1]
    k = repeat_kv(k, n_rep)
    v = repeat_kv(v, n_rep)
    scores = torch.einsum("qhd,khd->hqk", q, k) * (d ** -0.5)
    scores = scores.masked_fill(~visibility(t, window, q.device)[None], float("-inf"))
    weights = torch.softmax(scores, dim=-1)
    return torch.einsum("hqk,khd->qhd", weights, v)


def silu(x: torch.Tensor) -> torch.Tensor:
    """z * sigmoid(z): the activation of worker/src/inference/qwen2/model.py:236."""
    return x / (1.0 + torch.exp(-x))


def swiglu(x, w_gate, w_up, w_down) -> torch.Tensor:
    """down(silu(gate x) * up x), no biases: worker/src/inference/qwen2/model.py:228-236."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def self_attention(x, w: dict, prefix: str, positions, cfg: dict, window, angle_dtype=torch.float32) -> torch.Tensor:
    """q/k/v with bias, rope on q and k, attention, o without bias:
    worker/src/inference/qwen2/model.py:149-152, 214-225."""
    t = x.shape[0]
    h = int(cfg["num_attention_heads"])
    kh = int(cfg["num_key_value_heads"])
    d = head_dim_of(cfg)
    q = (x @ w[prefix + "q_proj.weight"].T + w[prefix + "q_proj.bias"]).view(t, h, d)
    k = (x @ w[prefix + "k_proj.weight"].T + w[prefix + "k_proj.bias"]).view(t, kh, d)
    v = (x @ w[prefix + "v_proj.weight"].T + w[prefix + "v_proj.bias"]).view(t, kh, d)
    cos, sin = rope_cos_sin(positions, d, rope_theta_of(cfg), x.dtype, angle_dtype)
    q = apply_rope(q, cos, sin)
    k = apply_rope(k, cos, sin)
    mixed = attention(q, k, v, window)
    return mixed.reshape(t, h * d) @ w[prefix + "o_proj.weight"].T


def decoder_layer(x, w: dict, index: int, positions, cfg: dict, window, angle_dtype=torch.float32) -> torch.Tensor:
    """h += attn(norm(h)); h += mlp(norm(h)): worker/src/inference/qwen2/model.py:247-249."""
    p = f"model.layers.{index}."
    eps = float(cfg["rms_norm_eps"])
    x = x + self_attention(rms_norm(x, w[p + "input_layernorm.weight"], eps), w, p + "self_attn.",
                           positions, cfg, window, angle_dtype)
    normed = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
    return x + swiglu(normed, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                      w[p + "mlp.down_proj.weight"])


def forward(w: dict, cfg: dict, ids, dtype=torch.float32, first_position: int = 0,
            angle_dtype=torch.float32, rows=None) -> torch.Tensor:
    """Token ids [T] -> logits [T, vocab] of one whole sequence:
    worker/src/inference/qwen2/model.py:305-314 (tied head: :302-303). It runs where the weights
    lie. `rows`: only these positions go through the final norm and the head (the reference's batched
    forward selects rows before the head too: model.py:376-379), so that a long sequence against a large
    vocabulary fits in memory."""
    w = {k: v.to(dtype) for k, v in w.items()}
    device = w["model.embed_tokens.weight"].device
    ids = torch.as_tensor(ids, dtype=torch.long, device=device)
    x = w["model.embed_tokens.weight"][ids]
    positions = torch.arange(first_position, first_position + ids.shape[0], device=device)
    for index, window in enumerate(layer_windows(cfg)):
        x = decoder_layer(x, w, index, positions, cfg, window, angle_dtype)
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long, device=device)]
    x = rms_norm(x, w["model.norm.weight"], float(cfg["rms_norm_eps"]))
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return x @ head.T


# --------------------------------------------------------------------------
# files and random weights (independent of the package's own writer)
# --------------------------------------------------------------------------

def tensor_shapes(cfg: dict) -> dict:
    """name -> shape, names from the attribute paths of
    worker/src/inference/qwen2/model.py:386-400, 442-452."""
    hd = int(cfg["hidden_size"])
    h = int(cfg["num_attention_heads"])
    kh = int(cfg["num_key_value_heads"])
    d = head_dim_of(cfg)
    inter = int(cfg["intermediate_size"])
    v = int(cfg["vocab_size"])
    shapes = {"model.embed_tokens.weight": (v, hd)}
    for l in range(int(cfg["num_hidden_layers"])):
        p = f"model.layers.{l}."
        shapes[p + "self_attn.q_proj.weight"] = (h * d, hd)
        shapes[p + "self_attn.q_proj.bias"] = (h * d,)
        shapes[p + "self_attn.k_proj.weight"] = (kh * d, hd)
        shapes[p + "self_attn.k_proj.bias"] = (kh * d,)
        shapes[p + "self_attn.v_proj.weight"] = (kh * d, hd)
        shapes[p + "self_attn.v_proj.bias"] = (kh * d,)
        shapes[p + "self_attn.o_proj.weight"] = (hd, h * d)
        shapes[p + "mlp.gate_proj.weight"] = (inter, hd)
        shapes[p + "mlp.up_proj.weight"] = (inter, hd)
        shapes[p + "mlp.down_proj.weight"] = (hd, inter)
        shapes[p + "input_layernorm.weight"] = (hd,)
        shapes[p + "post_attention_layernorm.weight"] = (hd,)
    shapes["model.norm.weight"] = (hd,)
    if not cfg.get("tie_word_embeddings", False):
        shapes["lm_head.weight"] = (v, hd)
    return shapes


def random_weights(cfg: dict, seed: int, std: float = 0.02, norm_jitter: float = 0.0,
                   dtype=torch.float32) -> dict:
    """Matrices, embeddings and biases ~ N(0, std); norm weights 1 (+ jitter so a
    missing or misplaced norm weight shows). A std of 0.5 keeps logits away from
    uniform, as benchmarks/correctness/test_hf_parity.py:61-62 advises."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith("norm.weight"):
            t = torch.ones(shape) + norm_jitter * torch.randn(shape, generator=gen)
        else:
            t = std * torch.randn(shape, generator=gen)
        out[name] = t.to(dtype)
    return out


def write_model_dir(path, cfg: dict, weights: dict) -> None:
    """A model folder as the engine expects it: config.json + model.safetensors."""
    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg, indent=1))
    save_file({k: v.contiguous() for k, v in weights.items()}, str(path / "model.safetensors"))


def read_weights(model_dir) -> dict:
    from safetensors.torch import load_file

    return load_file(str(Path(model_dir) / "model.safetensors"))


# Two tiny configurations that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "num_hidden_layers": 2,
    "hidden_size": 64,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "intermediate_size": 172,
    "vocab_size": 256,
    "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True,
    "use_sliding_window": False,
    "sliding_window": 4096,
    "max_window_layers": 2,
    "max_position_embeddings": 128,
    "hidden_act": "silu",
    "torch_dtype": "float32",
}

TINY_B = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "num_hidden_layers": 3,
    "hidden_size": 96,
    "num_attention_heads": 3,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "intermediate_size": 250,
    "vocab_size": 323,
    "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
    "use_sliding_window": True,
    "sliding_window": 8,
    "max_window_layers": 1,
    "max_position_embeddings": 256,
    "hidden_act": "silu",
    "torch_dtype": "float32",
}

# A third one whose head size is no power of two and whose heads are not grouped.
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "num_hidden_layers": 2,
    "hidden_size": 240,
    "num_attention_heads": 5,
    "num_key_value_heads": 5,
    "head_dim": 48,
    "intermediate_size": 100,
    "vocab_size": 1000,
    "rope_theta": 50000.0,
    "rms_norm_eps": 1e-3,
    "tie_word_embeddings": False,
    "layer_types": ["sliding_attention", "full_attention"],
    "sliding_window": 20,
    "max_position_embeddings": 512,
    "hidden_act": "silu",
    "torch_dtype": "float32",
}

