"""The plain implementation is pinned by facts that do not come from the reference's text:
library routines it must reduce to, invariants, and vectors the reference's own files hold."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as plain

torch.manual_seed(0)


def test_rms_norm_equals_library_routine_and_eps_matters():
    x = torch.randn(5, 48, dtype=torch.float64)
    w = torch.randn(48, dtype=torch.float64)
    for eps in (1e-6, 1e-5, 0.3):
        torch.testing.assert_close(plain.rms_norm(x, w, eps), F.rms_norm(x, (48,), w, eps))
    assert not torch.allclose(plain.rms_norm(x, w, 1e-6), plain.rms_norm(x, w, 0.3))
    # weight 1: each row has mean square ms / (ms + eps); a "1 + w" or a bias would break this
    y = plain.rms_norm(x, torch.ones(48, dtype=torch.float64), 1e-2)
    ms = (x * x).mean(-1)
    torch.testing.assert_close((y * y).mean(-1), ms / (ms + 1e-2))
    # scale invariance as eps -> 0 (eps outside the root, or added to the sum, would not scale this way)
    torch.testing.assert_close(plain.rms_norm(7 * x, w, 1e-12), plain.rms_norm(x, w, 1e-12))


def test_rope_invariants():
    d, theta = 8, 10000.0
    x = torch.randn(6, 3, d, dtype=torch.float64)
    pos = torch.tensor([0, 1, 5, 17, 100, 1000])
    y = plain.rope(x, pos, theta)
    torch.testing.assert_close(y[0], x[0])                                        # position 0 is the identity
    half = d // 2
    torch.testing.assert_close(y[..., :half] ** 2 + y[..., half:] ** 2,           # pairs are (j, j + D/2)
                               x[..., :half] ** 2 + x[..., half:] ** 2)
    # the same data with interleaved pairing (j, j+1) does NOT keep these pair norms -> pairing is pinned
    inter = x[..., 0::2] ** 2 + x[..., 1::2] ** 2
    assert not torch.allclose(y[..., 0::2] ** 2 + y[..., 1::2] ** 2, inter)
    # only distances count: <rope(q, m), rope(k, n)> depends on m - n
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)
    def dot(m, n):
        return (plain.rope(q, torch.tensor([m]), theta) * plain.rope(k, torch.tensor([n]), theta)).sum()
    torch.testing.assert_close(dot(9, 4), dot(105, 100), atol=1e-5, rtol=1e-5)    # fp32 angles limit this
    assert not torch.allclose(dot(9, 4), dot(4, 9))                               # the sign of the rotation
    # D = 2 is the plane rotation by `position` radians (inv_freq_0 = 1), counter-clockwise
    v = plain.rope(torch.tensor([[[1.0, 0.0]]], dtype=torch.float64), torch.tensor([1]), theta)
    torch.testing.assert_close(v[0, 0], torch.tensor([math.cos(1.0), math.sin(1.0)], dtype=torch.float64),
                               atol=1e-7, rtol=0)
    # the slowest pair turns by theta^(-(D-2)/D) per position
    e = torch.zeros(1, 1, d, dtype=torch.float64)
    e[0, 0, half - 1] = 1.0
    r = plain.rope(e, torch.tensor([1]), theta)
    assert abs(float(r[0, 0, d - 1]) - math.sin(theta ** (-(d - 2) / d))) < 1e-7
    assert not torch.allclose(plain.rope(x, pos, 10000.0), plain.rope(x, pos, 1e6))


def test_attention_reduces_to_library_routines():
    t, h, d = 9, 4, 16
    q, k, v = (torch.randn(t, h, d, dtype=torch.float64) for _ in range(3))
    pos = torch.arange(t)
    got = plain.attention(q, k, v, pos)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                          is_causal=True)[0].transpose(0, 1)
    torch.testing.assert_close(got, want)                      # scale D^-0.5, causal mask, softmax over keys
    # grouped queries: head h reads kv head h // group, i.e. repeat_interleave of k and v
    k2, v2 = k[:, :2], v[:, :2]
    got = plain.attention(q, k2, v2, pos)
    want = plain.attention(q, k2.repeat_interleave(2, 1), v2.repeat_interleave(2, 1), pos)
    torch.testing.assert_close(got, want)
    assert not torch.allclose(got, plain.attention(q, k2.repeat(1, 2, 1), v2.repeat(1, 2, 1), pos))
    # a portion at an offset equals the last rows of the whole (the chunk-offset mask)
    torch.testing.assert_close(plain.attention(q[6:], k, v, pos[6:]), plain.attention(q, k, v, pos)[6:])
    # the last row of a prompt is what a decode step computes: all keys allowed
    one = plain.attention(q[-1:], k, v, pos[-1:])
    w = torch.softmax((q[-1, 0] @ k[:, 0].T) * d ** -0.5, -1)
    torch.testing.assert_close(one[0, 0], w @ v[:, 0])
    # a window of w keys: position t sees t-w+1 .. t
    win = plain.attention(q, k, v, pos, window=3)
    torch.testing.assert_close(win[:3], plain.attention(q, k, v, pos)[:3])
    torch.testing.assert_close(win[8:], plain.attention(q[8:], k[6:], v[6:], pos[8:], pos[6:]))


def test_swiglu_equals_library_and_order_of_halves():
    x = torch.randn(3, 10, dtype=torch.float64)
    g, u, dn = torch.randn(14, 10, dtype=torch.float64), torch.randn(14, 10, dtype=torch.float64), torch.randn(10, 14, dtype=torch.float64)
    torch.testing.assert_close(plain.swiglu(x, g, u, dn), F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), dn))
    assert not torch.allclose(plain.swiglu(x, g, u, dn), plain.swiglu(x, u, g, dn))


def tiny(tied, layers=2):
    cfg = dict(model_type="qwen2", vocab_size=50, hidden_size=24, intermediate_size=40, num_hidden_layers=layers,
               num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=64, rms_norm_eps=1e-6,
               rope_theta=10000.0, tie_word_embeddings=tied)
    w, g = {}, torch.Generator().manual_seed(3)
    def r(*shape, base=0.0):
        return base + torch.randn(*shape, generator=g, dtype=torch.float64) * 0.2
    w["model.embed_tokens.weight"] = r(50, 24)
    for i in range(layers):
        p = f"model.layers.{i}."
        for name, rows in (("q_proj", 24), ("k_proj", 12), ("v_proj", 12)):
            w[p + f"self_attn.{name}.weight"], w[p + f"self_attn.{name}.bias"] = r(rows, 24), r(rows)
        w[p + "self_attn.o_proj.weight"] = r(24, 24)
        w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"] = r(40, 24), r(40, 24), r(24, 40)
        w[p + "input_layernorm.weight"], w[p + "post_attention_layernorm.weight"] = r(24, base=1.0), r(24, base=1.0)
    w["model.norm.weight"] = r(24, base=1.0)
    if not tied:
        w["lm_head.weight"] = r(50, 24)
    return cfg, w


def test_whole_model_structure():
    cfg, w = tiny(tied=False)
    tokens = [3, 9, 4, 4, 17, 30, 2]
    logits = plain.forward(cfg, w, tokens)
    assert logits.shape == (7, 50) and logits.dtype == torch.float32
    # causal: logits at a position do not depend on later tokens
    torch.testing.assert_close(plain.forward(cfg, w, tokens[:4]), logits[:4])
    # q/k/v biases are really applied
    w2 = dict(w)
    w2["model.layers.0.self_attn.k_proj.bias"] = torch.zeros(12, dtype=torch.float64)
    w2["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(24, dtype=torch.float64)
    assert not torch.allclose(plain.forward(cfg, w2, tokens), logits)
    # a one-layer model with zeroed o_proj and down_proj is embedding -> norm -> head (one-hot through the head)
    cfg1, w1 = tiny(tied=False, layers=1)
    w1["model.layers.0.self_attn.o_proj.weight"].zero_()
    w1["model.layers.0.mlp.down_proj.weight"].zero_()
    x = w1["model.embed_tokens.weight"][torch.tensor(tokens)]
    want = plain.rms_norm(x, w1["model.norm.weight"], 1e-6) @ w1["lm_head.weight"].T
    torch.testing.assert_close(plain.forward(cfg1, w1, tokens), want.float())
    # tied head uses the embedding matrix
    cfgt, wt = tiny(tied=True)
    lt = plain.forward(cfgt, wt, tokens)
    wu = dict(wt)
    wu["lm_head.weight"] = wt["model.embed_tokens.weight"]
    cfgu = dict(cfgt, tie_word_embeddings=False)
    torch.testing.assert_close(plain.forward(cfgu, wu, tokens), lt)
    # positions are absolute: shifting all positions changes nothing but through RoPE distances
    torch.testing.assert_close(plain.forward(cfg, w, tokens, first_position=0),
                               plain.forward(cfg, w, tokens, first_position=11), atol=2e-5, rtol=1e-4)


def test_greedy_and_temperature_helpers():
    cfg, w = tiny(tied=True)
    out = plain.greedy(cfg, w, [1, 2, 3], 4)
    # each token is the arg max of the last position's logits over everything before it; the logits of the
    # whole sequence, computed once, hold those of every prefix (causality), so a helper that forgets to
    # append, appends twice or reads another position fails
    whole = plain.forward(cfg, w, [1, 2, 3] + out)
    assert out == [int(whole[2 + i].argmax()) for i in range(4)]
    # the margin of each choice is far above float32 noise, so the comparison above is not a coin toss
    top2 = torch.topk(whole[2:6], 2, dim=-1).values
    assert float((top2[:, 0] - top2[:, 1]).min()) > 1e-4
    # a token changed in the prompt changes what follows (the helper reads its prompt)
    assert plain.greedy(cfg, w, [1, 2, 4], 4) != out or plain.greedy(cfg, w, [7, 2, 3], 4) != out
    logits = torch.tensor([1.0, 2.0, 3.0])
    p = plain.softmax_temperature(logits, 0.5)
    torch.testing.assert_close(p, torch.softmax(logits / 0.5, -1))
    # temperature sharpens: T -> 0 puts everything on the largest logit, T large flattens
    assert plain.softmax_temperature(logits, 0.01)[2] > 0.999
    torch.testing.assert_close(plain.softmax_temperature(logits, 1e6), torch.full((3,), 1 / 3), atol=1e-5, rtol=0)
