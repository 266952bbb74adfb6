"""A plain, slow Qwen3 forward pass: whole sequences, no cache, one function per part.

Written from the reference's formulas; every function cites the file and lines it
follows. It shares no code with ``socrates_amd``: it reads config.json with ``json``
and the tensors with ``safetensors`` directly, and computes in float32 (or float64)
with explicit matrix products, masks and softmax.
"""

import json
import math
from pathlib import Path

import torch
from safetensors.torch import load_file


def read_folder(folder, dtype=torch.float32):
    """config dict and {name: tensor} of a model folder, values upcast to ``dtype``."""
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    tensors = {k: v.to(dtype) for k, v in load_file(str(folder / "model.safetensors")).items()}
    return cfg, tensors


def rms_norm(x, weight, eps):
    """model/qwen/qwen_kv_cont.py:51-53: rms = sqrt(mean(x^2) + eps); x / rms * weight."""
    rms = torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return x / rms * weight


def rope_angles(head_dim, theta, positions):
    """model/qwen/qwen_kv_cont.py:58-64: inv_freq = 1 / theta^(2j/D) in float32,
    angles = position * inv_freq, duplicated to the full head width."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))
    angles = positions.float()[..., None] * inv_freq
    angles = torch.cat([angles, angles], dim=-1)
    return angles.cos(), angles.sin()


def rotate_half(x):
    """model/qwen/qwen_kv_cont.py:67-69: (x1, x2) -> (-x2, x1), halves of the head."""
    h = x.shape[-1] // 2
    return torch.cat([-x[..., h:], x[..., :h]], dim=-1)


def apply_rope(x, cos, sin):
    """model/qwen/qwen_kv_cont.py:72-77. x: [T, heads, D]; cos, sin: [T, D]."""
    cos = cos[:, None, :].to(x.dtype)
    sin = sin[:, None, :].to(x.dtype)
    return x * cos + rotate_half(x) * sin


def attention_scores(q, k, v, scale, positions_q=None, positions_k=None, window=None):
    """model/qwen/qwen.py:106-126 (explicit form): every query head h uses kv head
    h // G; scores = q k^T * scale; a key is masked when its position is greater than
    the query's (model/qwen/qwen_kv.py:172-177); softmax over keys; weighted values.

    q: [Tq, Hq, D]; k, v: [Tk, Hkv, D]. Returns [Tq, Hq, D]. ``window`` (not in the
    reference) keeps only the keys with position > p - window.
    """
    Tq, Hq, D = q.shape
    Tk, Hkv, _ = k.shape
    G = Hq // Hkv
    if positions_q is None:
        positions_q = torch.arange(Tk - Tq, Tk)
    if positions_k is None:
        positions_k = torch.arange(Tk)
    out = torch.empty_like(q)
    for h in range(Hq):
        kh, vh = k[:, h // G], v[:, h // G]                     # [Tk, D]
        s = (q[:, h] @ kh.T) * scale                            # [Tq, Tk]
        hidden = positions_k[None, :] > positions_q[:, None]
        if window is not None:
            hidden = hidden | (positions_k[None, :] <= positions_q[:, None] - window)
        s = s.masked_fill(hidden, float("-inf"))
        out[:, h] = s.softmax(dim=-1) @ vh
    return out


def attention_layer(x, w, prefix, cfg, positions, window=None):
    """model/qwen/qwen_kv_paged.py:147-175: projections without bias, heads packed by
    index; q_norm / k_norm per head over D, then rotation; scale D^-0.5 (:139); heads
    concatenated in order into o_proj."""
    T = x.shape[0]
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    q = (x @ w[prefix + "q_proj.weight"].T).view(T, Hq, D)
    k = (x @ w[prefix + "k_proj.weight"].T).view(T, Hkv, D)
    v = (x @ w[prefix + "v_proj.weight"].T).view(T, Hkv, D)
    cos, sin = rope_angles(D, cfg["rope_theta"], positions)
    q = apply_rope(rms_norm(q, w[prefix + "q_norm.weight"], eps), cos, sin)
    k = apply_rope(rms_norm(k, w[prefix + "k_norm.weight"], eps), cos, sin)
    o = attention_scores(q, k, v, D ** -0.5, positions, positions, window)
    return o.reshape(T, Hq * D) @ w[prefix + "o_proj.weight"].T


def swiglu_mlp(x, w, prefix):
    """model/qwen/qwen_kv_cont.py:259-266: down(up(x) * silu(gate(x)))."""
    g = x @ w[prefix + "gate_proj.weight"].T
    u = x @ w[prefix + "up_proj.weight"].T
    return (u * (g * torch.sigmoid(g))) @ w[prefix + "down_proj.weight"].T


def block(x, w, i, cfg, positions):
    """model/qwen/qwen_kv_paged.py:186-189: x + attn(norm(x)); then + mlp(norm(.))."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    x = x + attention_layer(rms_norm(x, w[p + "input_layernorm.weight"], eps), w,
                            p + "self_attn.", cfg, positions)
    return x + swiglu_mlp(rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p + "mlp.")


def forward(cfg, w, ids, first_position=0, rows=None):
    """model/qwen/qwen_kv_paged.py:219-224: embed, blocks, final norm, logits = x E^T.
    The reference always uses the embedding table as the head (:224); a folder with
    tie_word_embeddings=false carries lm_head.weight, used instead.

    ids: sequence of token ids. Returns logits [T, V] for every position, or for the
    positions listed in ``rows`` only (a large vocabulary makes all of them costly).
    """
    ids = torch.as_tensor(ids, dtype=torch.long)
    positions = torch.arange(first_position, first_position + len(ids))
    x = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        x = block(x, w, i, cfg, positions)
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long)]
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return x @ head.T


def greedy(cfg, w, prompt, n_new):
    """Argmax continuation, recomputing the whole sequence for every token
    (model/inference_paged.py:166, 193: argmax of the last position's logits)."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        nxt = int(forward(cfg, w, ids)[-1].argmax())
        out.append(nxt)
        ids.append(nxt)
    return out
