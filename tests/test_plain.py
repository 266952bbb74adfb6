"""Pins the plain implementation by what fixes it beside the reference's text: library
routines it must reduce to, vectors the reference's own tests hold, and invariants. Each
check is chosen so that a plausible mistake (a wrong sign or pairing, eps outside the
root, a norm in the wrong place, heads mapped i % G instead of i // G) fails it."""

import math

import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from helpers import TINY_A, TINY_B, random_prompts, write_tiny

torch.manual_seed(0)


def test_rms_norm_is_the_library_routine_with_eps_inside_the_root():
    x, w = torch.randn(5, 7, 48) * 1e-3, 1 + 0.3 * torch.randn(48)      # tiny rows: eps matters
    for eps in (1e-6, 1e-5):
        torch.testing.assert_close(plain.rms_norm(x, w, eps), F.rms_norm(x, (48,), w, eps))
    outside = x / (torch.sqrt(x.pow(2).mean(-1, keepdim=True)) + 1e-5) * w
    assert not torch.allclose(plain.rms_norm(x, w, 1e-5), outside, rtol=1e-3)
    assert not torch.allclose(plain.rms_norm(x, w, 1e-5), plain.rms_norm(x, w, 1e-6), rtol=1e-3)
    big = torch.randn(3, 48)
    y = plain.rms_norm(big, torch.ones(48), 1e-12)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(3))        # unit RMS
    torch.testing.assert_close(plain.rms_norm(3.7 * big, w, 1e-12), plain.rms_norm(big, w, 1e-12))
    assert not torch.allclose(plain.rms_norm(big, w, 1e-6), plain.rms_norm(big, 1 + w, 1e-6))  # plain gain


def test_rope():
    D, theta = 32, 1e4
    x = torch.randn(9, 3, D)
    cos0, sin0 = plain.rope_angles(D, theta, torch.zeros(9))
    torch.testing.assert_close(plain.apply_rope(x, cos0, sin0), x)      # position 0 is the identity
    pos = torch.tensor([0, 1, 2, 3, 50, 100, 1000, 2047, 4095])
    cos, sin = plain.rope_angles(D, theta, pos)
    assert cos.shape == (9, D) and math.isclose(float(sin[1, 0]), math.sin(1.0), rel_tol=1e-6)  # inv_freq[0] = 1
    y = plain.apply_rope(x, cos, sin)
    h = D // 2
    # rotate-half pairing: (j, j + D/2) is rotated as a complex number by e^{i pos theta^(-2j/D)}
    z = torch.complex(x[..., :h].double(), x[..., h:].double())
    ang = pos.double()[:, None] * (theta ** (-torch.arange(0, D, 2).double() / D))
    zr = z * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    # float32 angles resolve 4095 * 2^-24 rad at the last position; a wrong pairing is off by O(1)
    torch.testing.assert_close(y[..., :h].double(), zr.real, atol=1.5e-3, rtol=0)
    torch.testing.assert_close(y[..., h:].double(), zr.imag, atol=1.5e-3, rtol=0)
    torch.testing.assert_close(y[:6, :, :h].double(), zr.real[:6], atol=2e-5, rtol=0)
    # interleaved pairing (j, j+1) would fail the above; a wrong sign fails this:
    torch.testing.assert_close(y[..., :h] ** 2 + y[..., h:] ** 2, x[..., :h] ** 2 + x[..., h:] ** 2,
                               atol=1e-5, rtol=1e-5)
    q, k = torch.randn(1, 1, D), torch.randn(1, 1, D)

    def dot(m, n):
        cm, sm = plain.rope_angles(D, theta, torch.tensor([m]))
        cn, sn = plain.rope_angles(D, theta, torch.tensor([n]))
        return float((plain.apply_rope(q, cm, sm) * plain.apply_rope(k, cn, sn)).sum())
    assert abs(dot(5, 2) - dot(105, 102)) < 1e-3 and abs(dot(5, 2) - dot(2, 5)) > 1e-3


def test_attention_reduces_to_the_library_routine():
    T, H, D = 13, 4, 16
    q, k, v = torch.randn(T, H, D), torch.randn(T, H, D), torch.randn(T, H, D)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                          is_causal=True, scale=0.3).transpose(0, 1)
    torch.testing.assert_close(plain.attention_scores(q, k, v, 0.3), want, atol=1e-5, rtol=1e-5)
    one = plain.attention_scores(q[:, :1], k[:, :1], v[:, :1], 0.3)                  # one head
    torch.testing.assert_close(one, want[:, :1], atol=1e-5, rtol=1e-5)
    # decode: the last query against all keys, no mask at all
    last = F.scaled_dot_product_attention(q[-1:].transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), scale=0.3)
    torch.testing.assert_close(plain.attention_scores(q[-1:], k, v, 0.3), last.transpose(0, 1), atol=1e-5, rtol=1e-5)
    # q = 0: uniform weights, the output is the running mean of V
    mean = torch.cumsum(v, 0) / torch.arange(1, T + 1)[:, None, None]
    torch.testing.assert_close(plain.attention_scores(torch.zeros_like(q), k, v, 0.3), mean, atol=1e-5, rtol=1e-5)
    # softmax is shift invariant: one more coordinate, 1 in every query and c in every key, adds
    # 0.3 c to all scores of a query and changes nothing (an unnormalised or overflowing exp would)
    for c in (5.0, -200.0, 200.0):
        q1 = torch.cat([q, torch.ones(T, H, 1)], -1)
        k1 = torch.cat([k, torch.full((T, H, 1), c)], -1)
        v1 = torch.cat([v, torch.zeros(T, H, 1)], -1)
        shifted = plain.attention_scores(q1, k1, v1, 0.3)
        torch.testing.assert_close(shifted[..., :D], want, atol=1e-5, rtol=1e-5)
    # and a shift that differs from key to key is not: the check above can fail
    k1[3:, :, -1] += 4.0
    assert not torch.allclose(plain.attention_scores(q1, k1, v1, 0.3)[..., :D], want, atol=1e-3)


def test_attention_layer_takes_the_library_routines_default_scale(tmp_path):
    """The reference's prompt pass hands q, k, v to the library's attention without a scale
    (model/qwen/qwen_kv_paged.py:171-173), whose default is 1 / sqrt(last dimension of q); its
    decode pass passes head_dim ** -0.5 to its own kernel (:139). The plain layer against the
    same layer put together from library routines, with no scale written anywhere, at a head
    size (32) that is neither hidden / heads (12) nor one at which 1 / sqrt(D) and 1 / D or 1
    give like results: the scores are several units wide."""
    folder = write_tiny(tmp_path / "B", TINY_B, seed=4)
    cfg, w = plain.read_folder(folder)
    T, Hq, Hkv, D = 19, cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    assert D == 32 and cfg["hidden_size"] // Hq == 12
    p = "model.layers.1.self_attn."
    x = 3.0 * torch.randn(T, cfg["hidden_size"])
    pos = torch.arange(T)
    q = F.rms_norm((x @ w[p + "q_proj.weight"].T).view(T, Hq, D), (D,), 4.0 * w[p + "q_norm.weight"], cfg["rms_norm_eps"])
    k = F.rms_norm((x @ w[p + "k_proj.weight"].T).view(T, Hkv, D), (D,), w[p + "k_norm.weight"], cfg["rms_norm_eps"])
    v = (x @ w[p + "v_proj.weight"].T).view(T, Hkv, D)
    # the rotation as a complex multiplication of (x[j], x[j + D/2]) by exp(i position inv_freq[j])
    inv_freq = 1.0 / (cfg["rope_theta"] ** (torch.arange(0, D, 2).float() / D))
    turn = torch.polar(torch.ones(T, D // 2), pos[:, None].float() * inv_freq)[:, None]
    def rotate(t):
        z = torch.complex(t[..., :D // 2], t[..., D // 2:]) * turn
        return torch.cat([z.real, z.imag], -1)
    o = F.scaled_dot_product_attention(rotate(q).transpose(0, 1)[None], rotate(k).transpose(0, 1)[None],
                                       v.transpose(0, 1)[None], is_causal=True, enable_gqa=True)[0]
    want = o.transpose(0, 1).reshape(T, Hq * D) @ w[p + "o_proj.weight"].T
    w4 = dict(w)
    w4[p + "q_norm.weight"] = 4.0 * w[p + "q_norm.weight"]           # sharper scores: the scale shows
    got = plain.attention_layer(x, w4, p, cfg, pos)
    torch.testing.assert_close(got, want, atol=2e-5, rtol=1e-4)
    # the same routine with the scales a misreading would give is far away
    for wrong in (1.0 / D, 1.0, (cfg["hidden_size"] // Hq) ** -0.5):
        o = F.scaled_dot_product_attention(rotate(q).transpose(0, 1)[None], rotate(k).transpose(0, 1)[None],
                                           v.transpose(0, 1)[None], is_causal=True, enable_gqa=True, scale=wrong)[0]
        other = o.transpose(0, 1).reshape(T, Hq * D) @ w[p + "o_proj.weight"].T
        assert (other - want).abs().max() > 50 * (got - want).abs().max() + 1e-3


def test_attention_needles_fix_length_bound_and_head_mapping():
    """tests/test_kernel_cuda.py:70-107 of the reference: q = 0, V zero except one slot that
    holds 8 * (kv head + 1); query head i reads kv head i // G with weight 1/n."""
    Hq, Hkv, D = 8, 2, 16
    G = Hq // Hkv
    for n, slot in [(1, 0), (16, 15), (17, 16), (40, 39), (40, 0), (33, 17)]:
        k = torch.randn(n, Hkv, D)
        v = torch.zeros(n, Hkv, D)
        for h in range(Hkv):
            v[slot, h] = 8.0 * (h + 1)
        out = plain.attention_scores(torch.zeros(1, Hq, D), k, v, 0.1)
        want = torch.tensor([8.0 * (i // G + 1) / n for i in range(Hq)])[None, :, None].expand(1, Hq, D)
        torch.testing.assert_close(out, want, atol=1e-5, rtol=1e-5)
    # a key past the query's position is not read
    k, v = torch.randn(10, Hkv, D), torch.zeros(10, Hkv, D)
    v[9] = 5.0
    out = plain.attention_scores(torch.zeros(1, Hq, D), k, v, 0.1, positions_q=torch.tensor([8]))
    assert out.abs().max() == 0


def test_window_keeps_the_last_w_keys():
    T, D = 12, 16
    q, k, v = torch.randn(T, 2, D), torch.randn(T, 1, D), torch.randn(T, 1, D)
    got = plain.attention_scores(q, k, v, 0.25, window=4)
    for t in range(T):
        lo = max(0, t - 3)
        want = plain.attention_scores(q[t:t + 1], k[lo:t + 1], v[lo:t + 1], 0.25)
        torch.testing.assert_close(got[t:t + 1], want, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(plain.attention_scores(q, k, v, 0.25, window=T), plain.attention_scores(q, k, v, 0.25))


def test_swiglu_is_silu_on_the_gate():
    x = torch.randn(6, 10)
    w = {"p.gate_proj.weight": torch.randn(14, 10), "p.up_proj.weight": torch.randn(14, 10),
         "p.down_proj.weight": torch.randn(10, 14)}
    want = (F.silu(x @ w["p.gate_proj.weight"].T) * (x @ w["p.up_proj.weight"].T)) @ w["p.down_proj.weight"].T
    torch.testing.assert_close(plain.swiglu_mlp(x, w, "p."), want)
    swapped = dict(w, **{"p.gate_proj.weight": w["p.up_proj.weight"], "p.up_proj.weight": w["p.gate_proj.weight"]})
    assert not torch.allclose(plain.swiglu_mlp(x, swapped, "p."), want)
    zero_gate = dict(w, **{"p.gate_proj.weight": torch.zeros(14, 10)})
    assert plain.swiglu_mlp(x, zero_gate, "p.").abs().max() == 0


def test_block_residuals_and_heads(tmp_path):
    folder = write_tiny(tmp_path / "B", TINY_B, seed=2)
    cfg, w = plain.read_folder(folder)
    ids = random_prompts([11], cfg["vocab_size"], seed=0)[0]
    x = w["model.embed_tokens.weight"][torch.tensor(ids)]
    pos = torch.arange(11)
    # zeroed o_proj and down_proj: the block is the identity (both branches are added, not chained)
    w0 = dict(w)
    w0["model.layers.0.self_attn.o_proj.weight"] = torch.zeros_like(w["model.layers.0.self_attn.o_proj.weight"])
    w0["model.layers.0.mlp.down_proj.weight"] = torch.zeros_like(w["model.layers.0.mlp.down_proj.weight"])
    torch.testing.assert_close(plain.block(x, w0, 0, cfg, pos), x)
    # only down_proj zeroed: x + attn(norm(x))
    w1 = dict(w)
    w1["model.layers.0.mlp.down_proj.weight"] = w0["model.layers.0.mlp.down_proj.weight"]
    attn = plain.attention_layer(plain.rms_norm(x, w["model.layers.0.input_layernorm.weight"], cfg["rms_norm_eps"]),
                                 w, "model.layers.0.self_attn.", cfg, pos)
    torch.testing.assert_close(plain.block(x, w1, 0, cfg, pos), x + attn)
    # untied: the head is lm_head.weight, not the embedding table
    logits = plain.forward(cfg, w, ids)
    tied = plain.forward(dict(cfg, tie_word_embeddings=True), w, ids)
    assert logits.shape == (11, cfg["vocab_size"]) and not torch.allclose(logits, tied)
    # causal: logits of a prefix do not change when tokens are appended
    torch.testing.assert_close(plain.forward(cfg, w, ids[:6]), logits[:6], atol=1e-5, rtol=1e-5)
    # only distances count: shifting every position leaves the logits unchanged
    shifted = plain.forward(cfg, w, ids, first_position=37)
    torch.testing.assert_close(shifted, logits, atol=2e-4, rtol=2e-4)


def test_qk_norm_is_per_head_before_rotation(tmp_path):
    folder = write_tiny(tmp_path / "A", TINY_A, seed=3)
    cfg, w = plain.read_folder(folder)
    x = torch.randn(7, cfg["hidden_size"])
    p = "model.layers.0.self_attn."
    base = plain.attention_layer(x, w, p, cfg, torch.arange(7))
    # scaling q_proj changes nothing: q is normed per head right after the projection
    w2 = dict(w)
    w2[p + "q_proj.weight"] = 5.0 * w[p + "q_proj.weight"]
    torch.testing.assert_close(plain.attention_layer(x, w2, p, cfg, torch.arange(7)), base, atol=1e-4, rtol=1e-4)
    # v is not normed
    w3 = dict(w)
    w3[p + "v_proj.weight"] = 5.0 * w[p + "v_proj.weight"]
    torch.testing.assert_close(plain.attention_layer(x, w3, p, cfg, torch.arange(7)), 5.0 * base, atol=1e-4, rtol=1e-4)
