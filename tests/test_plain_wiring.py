"""How the plain implementation wires its parts together, pinned by closed forms.

test_plain.py pins each formula (norm, rotation, attention, feed-forward) against library
routines and invariants. Here whole layers and whole models are driven into special cases whose
result can be written down with library routines and elementary mathematics alone, each chosen so
that a plausible mistake of wiring changes the result:

  one token          softmax over a single key is 1: attention returns v. Pins pre-norm wiring with
                     two residuals (the feed-forward reads the UPDATED stream), the v bias, no o bias,
                     the final norm, which kv head a query head reads.
  zero queries       all scores are 0: attention is the running mean of v over the keys allowed.
                     Pins the causal mask inside the model, and that v is not rotated.
  bias-only q and k  with zero q/k matrices the scores are sin((p - n) * theta_j) * a_q * a_k / sqrt(D):
                     a function of the distance only. Pins bias BEFORE rotation, rotation of q and of k
                     with the same sense, the pairing (j, j + D/2), theta^(-2j/D), the scale D^-0.5 with
                     the configuration's head_dim, and the query-head to kv-head map.
  scaling            a pre-norm branch does not see the scale of the stream it reads.

No model code of any installed package is used: the other side of every comparison is
torch.nn.functional's rms_norm / linear / silu, cumsum, and math.sin.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as plain

F64 = torch.float64


def make(heads, kv_heads, head_dim, hidden, layers=2, tied=False, explicit_head_dim=False, seed=3,
         eps=1e-6, theta=10000.0, vocab=50, inter=40):
    cfg = dict(model_type="qwen2", vocab_size=vocab, hidden_size=hidden, intermediate_size=inter,
               num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=kv_heads,
               max_position_embeddings=64, rms_norm_eps=eps, rope_theta=theta, tie_word_embeddings=tied)
    if explicit_head_dim:
        cfg["head_dim"] = head_dim
    else:
        assert hidden == heads * head_dim
    g = torch.Generator().manual_seed(seed)

    def r(*shape, base=0.0):
        return base + torch.randn(*shape, generator=g, dtype=F64) * 0.3
    w = {"model.embed_tokens.weight": r(vocab, hidden)}
    for i in range(layers):
        p = f"model.layers.{i}."
        for name, rows in (("q_proj", heads * head_dim), ("k_proj", kv_heads * head_dim), ("v_proj", kv_heads * head_dim)):
            w[p + f"self_attn.{name}.weight"], w[p + f"self_attn.{name}.bias"] = r(rows, hidden), r(rows)
        w[p + "self_attn.o_proj.weight"] = r(hidden, heads * head_dim)
        w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"] = r(inter, hidden), r(inter, hidden)
        w[p + "mlp.down_proj.weight"] = r(hidden, inter)
        w[p + "input_layernorm.weight"], w[p + "post_attention_layernorm.weight"] = r(hidden, base=1.0), r(hidden, base=1.0)
    w["model.norm.weight"] = r(hidden, base=1.0)
    if not tied:
        w["lm_head.weight"] = r(vocab, hidden)
    return cfg, w


SHAPES = [dict(heads=4, kv_heads=2, head_dim=6, hidden=24),                               # head_dim implied
          dict(heads=3, kv_heads=1, head_dim=8, hidden=20, explicit_head_dim=True, eps=1e-5, theta=1e6, tied=True),
          dict(heads=2, kv_heads=2, head_dim=4, hidden=8, layers=3, inter=12)]


def closed_form(cfg, w, tokens, attention_of):
    """The model with library routines; ATTENTION_OF(layer, h [T, hidden]) -> [T, heads * D] replaces attention."""
    hidden, eps = cfg["hidden_size"], cfg["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = F.rms_norm(x, (hidden,), w[p + "input_layernorm.weight"], eps)
        x = x + F.linear(attention_of(i, h), w[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (hidden,), w[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                         w[p + "mlp.down_proj.weight"])
    x = F.rms_norm(x, (hidden,), w["model.norm.weight"], eps)
    return F.linear(x, w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"])


def values(cfg, w, i, h, head_dim):
    """v of layer i, one copy per QUERY head: [T, heads, D] (query head q reads kv head q // group)."""
    p = f"model.layers.{i}.self_attn."
    kv, heads = cfg["num_key_value_heads"], cfg["num_attention_heads"]
    v = F.linear(h, w[p + "v_proj.weight"], w[p + "v_proj.bias"]).view(-1, kv, head_dim)
    return v.repeat_interleave(heads // kv, dim=1)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("position", [0, 13])
def test_a_single_token_gets_its_own_value_back(shape, position):
    cfg, w = make(**shape)
    d = shape["head_dim"]
    for token in (0, 7, 31):
        want = closed_form(cfg, w, [token], lambda i, h: values(cfg, w, i, h, d).reshape(1, -1))
        got = plain.forward(cfg, w, [token], first_position=position)
        torch.testing.assert_close(got.to(F64), want, atol=1e-5, rtol=1e-5)
    # the closed form itself notices the mistakes it is there for (so the comparison above can fail)
    base = closed_form(cfg, w, [7], lambda i, h: values(cfg, w, i, h, d).reshape(1, -1))
    no_bias = dict(w)
    no_bias["model.layers.0.self_attn.v_proj.bias"] = torch.zeros_like(w["model.layers.0.self_attn.v_proj.bias"])
    assert not torch.allclose(plain.forward(cfg, no_bias, [7]).to(F64), base, atol=1e-4)
    if shape["heads"] != shape["kv_heads"] and shape["kv_heads"] > 1:
        tiled = closed_form(cfg, w, [7], lambda i, h: F.linear(
            h, w[f"model.layers.{i}.self_attn.v_proj.weight"], w[f"model.layers.{i}.self_attn.v_proj.bias"])
            .view(1, shape["kv_heads"], d).repeat(1, shape["heads"] // shape["kv_heads"], 1).reshape(1, -1))
        assert not torch.allclose(tiled, base, atol=1e-4)


@pytest.mark.parametrize("shape", SHAPES)
def test_zero_queries_average_the_values_seen_so_far(shape):
    cfg, w = make(**shape)
    d = shape["head_dim"]
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.q_proj.weight"].zero_()
        w[f"model.layers.{i}.self_attn.q_proj.bias"].zero_()
    tokens = [3, 9, 4, 4, 17, 30, 2, 41, 8]
    t = len(tokens)

    def running_mean(i, h):
        v = values(cfg, w, i, h, d)
        return (v.cumsum(0) / torch.arange(1, t + 1, dtype=F64)[:, None, None]).reshape(t, -1)
    want = closed_form(cfg, w, tokens, running_mean)
    for first in (0, 21):          # rotation of v (a mistake) would also make this depend on the positions
        got = plain.forward(cfg, w, tokens, first_position=first)
        torch.testing.assert_close(got.to(F64), want, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("shape", SHAPES)
def test_scores_of_bias_only_queries_and_keys_are_sines_of_the_distance(shape):
    cfg, w = make(**shape)
    heads, kv, d = shape["heads"], shape["kv_heads"], shape["head_dim"]
    half, group, theta = d // 2, heads // kv, cfg["rope_theta"]
    pair = {}                                # (layer, kv head) -> which pair of the head carries the signal
    amp_q, amp_k = {}, {}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}.self_attn."
        w[p + "q_proj.weight"].zero_()
        w[p + "k_proj.weight"].zero_()
        bq, bk = torch.zeros(heads * d, dtype=F64), torch.zeros(kv * d, dtype=F64)
        for g in range(kv):
            j = (g + i) % half
            pair[i, g] = j
            amp_k[i, g] = 2.0 + 0.5 * g
            bk[g * d + j + half] = amp_k[i, g]              # k = (0, a): the second element of pair j
        for q in range(heads):
            amp_q[i, q] = 3.0 - 0.4 * q + 0.3 * i
            bq[q * d + pair[i, q // group]] = amp_q[i, q]   # q = (a, 0): the first element of pair j
        w[p + "q_proj.bias"], w[p + "k_proj.bias"] = bq, bk
    tokens = [5, 1, 44, 20, 20, 3, 12, 37, 9, 28, 6]
    t = len(tokens)

    def by_distance(i, h):
        v = values(cfg, w, i, h, d)                          # [T, heads, D]
        out = torch.zeros(t, heads, d, dtype=F64)
        for q in range(heads):
            g = q // group
            rate = theta ** (-2.0 * pair[i, g] / d)
            for p_ in range(t):
                s = [amp_q[i, q] * amp_k[i, g] * math.sin((p_ - n) * rate) / math.sqrt(d) for n in range(p_ + 1)]
                top = max(s)
                e = [math.exp(x - top) for x in s]
                z = sum(e)
                for n in range(p_ + 1):
                    out[p_, q] += e[n] / z * v[n, q]
        return out.reshape(t, -1)
    want = closed_form(cfg, w, tokens, by_distance)
    got = plain.forward(cfg, w, tokens)
    torch.testing.assert_close(got.to(F64), want, atol=2e-5, rtol=2e-5)
    # the attention is far from uniform here (so that a bias added after the rotation, which would make
    # every score equal, cannot pass): compare with the running mean of the test above
    def running_mean(i, h):
        v = values(cfg, w, i, h, d)
        return (v.cumsum(0) / torch.arange(1, t + 1, dtype=F64)[:, None, None]).reshape(t, -1)
    assert not torch.allclose(closed_form(cfg, w, tokens, running_mean), want, atol=1e-3)
    # and the sense of the rotation matters: distances counted the other way give other logits
    def reversed_sense(i, h):
        v = values(cfg, w, i, h, d)
        out = torch.zeros(t, heads, d, dtype=F64)
        for q in range(heads):
            g = q // group
            rate = theta ** (-2.0 * pair[i, g] / d)
            for p_ in range(t):
                s = torch.tensor([amp_q[i, q] * amp_k[i, g] * math.sin((n - p_) * rate) / math.sqrt(d)
                                  for n in range(p_ + 1)], dtype=F64)
                out[p_, q] = torch.softmax(s, 0) @ v[:p_ + 1, q]
        return out.reshape(t, -1)
    assert not torch.allclose(closed_form(cfg, w, tokens, reversed_sense), want, atol=1e-3)


def test_a_pre_norm_branch_does_not_see_the_scale_of_its_input():
    cfg, w = make(heads=4, kv_heads=2, head_dim=6, hidden=24, eps=1e-12)
    s = plain.sizes(cfg)
    x = torch.randn(5, 24, dtype=F64, generator=torch.Generator().manual_seed(1))
    pos = torch.arange(5)
    w0 = dict(w)
    w0["model.layers.0.mlp.down_proj.weight"] = torch.zeros_like(w["model.layers.0.mlp.down_proj.weight"])
    branch = plain.decoder_layer(x, pos, w0, 0, s) - x
    torch.testing.assert_close(plain.decoder_layer(7.5 * x, pos, w0, 0, s) - 7.5 * x, branch, atol=1e-8, rtol=1e-8)
    # the feed-forward branch alone (o_proj zeroed) likewise, and it reads the stream the mixer has updated:
    w1 = dict(w)
    w1["model.layers.0.self_attn.o_proj.weight"] = torch.zeros_like(w["model.layers.0.self_attn.o_proj.weight"])
    ff = plain.decoder_layer(x, pos, w1, 0, s) - x
    torch.testing.assert_close(plain.decoder_layer(0.2 * x, pos, w1, 0, s) - 0.2 * x, ff, atol=1e-8, rtol=1e-8)
    both = plain.decoder_layer(x, pos, w, 0, s) - x
    assert not torch.allclose(both, branch + ff, atol=1e-3)      # a parallel block would be exactly the sum
    # the model's output does not see the scale of the last stream either (final norm before the head)
    h = F.rms_norm(x, (24,), w["model.norm.weight"], 1e-12)
    torch.testing.assert_close(plain.rms_norm(3 * x, w["model.norm.weight"], 1e-12), h)
