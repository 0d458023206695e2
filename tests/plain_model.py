"""A plain, slow implementation of the Qwen2.5 dense decoder: whole sequences, no cache.

Written from the reference's formulas (each function cites them). It shares no
code with the package under test: it reads config.json and the safetensors file
itself and uses only elementary torch operations. The reference was read, not run.
"""
import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


def read_folder(folder, dtype=torch.float32, device="cpu"):
    """(config dict, {tensor name: tensor in DTYPE on DEVICE}) of a model folder."""
    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    tensors = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device=str(device)) as f:
        for key in f.keys():
            tensors[key] = f.get_tensor(key).to(dtype)
    return config, tensors


def sizes(config):
    """Sizes with the reference's defaults (flow_engine/config.py:38-49)."""
    hidden = config["hidden_size"]
    heads = config["num_attention_heads"]
    return dict(hidden=hidden, heads=heads,
                kv_heads=config.get("num_key_value_heads") or heads,
                head_dim=config.get("head_dim") or hidden // heads,
                layers=config["num_hidden_layers"],
                eps=config.get("rms_norm_eps", 1e-6),
                theta=config.get("rope_theta", 10000.0),
                tied=bool(config.get("tie_word_embeddings", False)))


def rms_norm(x, weight, eps):
    """flow_engine/model.py:21-23: x * rsqrt(mean(x^2) + eps), then times the weight.

    eps is added to the mean square, inside the root; the weight multiplies the
    normalised value (no "1 + weight", no bias).
    """
    mean_square = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    return x / torch.sqrt(mean_square + eps) * weight


def rope(x, positions, theta):
    """flow_engine/model.py:26-33: rotate-half RoPE over the whole head.

    x [T, heads, D]; pair j is (x[j], x[j + D/2]) and turns by the angle
    position * theta^(-2j/D):  x'[j] = x[j] cos - x[j+D/2] sin,
    x'[j+D/2] = x[j+D/2] cos + x[j] sin.
    """
    d = x.shape[-1]
    half = d // 2
    # fp32 as the reference, and always on the host: a float32 power differs in its last bit between the host's
    # and a GPU's routine, and an angle is that rate times a position of thousands (at position 4,000 the two
    # rotations are 2e-4 rad apart, which shows in the logits as 7e-5: as much as four layers of float32
    # rounding). The engine computes the rates on the host; so does this, wherever the rest of it runs.
    inv = (theta ** (-torch.arange(0, d, 2, dtype=torch.float32, device="cpu") / d)).to(x.device)
    angle = positions.to(device=x.device, dtype=torch.float32)[:, None] * inv[None, :]   # [T, D/2] in fp32
    cos, sin = angle.cos().to(x.dtype)[:, None, :], angle.sin().to(x.dtype)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return torch.cat((lo * cos - hi * sin, hi * cos + lo * sin), -1)


def attention(q, k, v, q_positions, k_positions=None, window=None, scale=None):
    """flow_engine/model.py:192-200 and kernels/paged_decode.py:20-43.

    q [Tq, Hq, D]; k, v [Tk, Hk, D]. Query head h reads kv head h // (Hq/Hk).
    Key p is allowed for the query at position t iff p <= t (and, with a window
    of w keys, p > t - w); scores are q.k * D^-0.5; softmax over allowed keys.
    """
    tq, hq, d = q.shape
    tk, hk, _ = k.shape
    if k_positions is None:
        k_positions = torch.arange(tk)
    scale = d ** -0.5 if scale is None else scale
    out = torch.zeros(tq, hq, v.shape[-1], dtype=q.dtype)
    group = hq // hk
    for h in range(hq):
        g = h // group
        scores = (q[:, h, :] @ k[:, g, :].T) * scale                        # [Tq, Tk]
        allowed = k_positions[None, :] <= q_positions[:, None]
        if window is not None:
            allowed &= k_positions[None, :] > q_positions[:, None] - window
        scores = scores.masked_fill(~allowed, float("-inf"))
        weights = torch.exp(scores - scores.max(-1, keepdim=True).values)
        weights = weights / weights.sum(-1, keepdim=True)
        out[:, h, :] = weights @ v[:, g, :]
    return out


def swiglu(x, gate_w, up_w, down_w):
    """flow_engine/model.py:75-80: down( silu(gate(x)) * up(x) ), silu(z) = z * sigmoid(z), no biases."""
    gate = x @ gate_w.T
    up = x @ up_w.T
    return (gate / (1.0 + torch.exp(-gate)) * up) @ down_w.T


def attention_block(x, positions, w, prefix, s, window=None):
    """flow_engine/model.py:183-201: q/k/v with bias, RoPE on q and k, attention, o_proj without bias."""
    t = x.shape[0]
    q = x @ w[prefix + "q_proj.weight"].T + w[prefix + "q_proj.bias"]
    k = x @ w[prefix + "k_proj.weight"].T + w[prefix + "k_proj.bias"]
    v = x @ w[prefix + "v_proj.weight"].T + w[prefix + "v_proj.bias"]
    q = rope(q.reshape(t, s["heads"], s["head_dim"]), positions, s["theta"])
    k = rope(k.reshape(t, s["kv_heads"], s["head_dim"]), positions, s["theta"])
    v = v.reshape(t, s["kv_heads"], s["head_dim"])
    out = attention(q, k, v, positions, positions, window)
    return out.reshape(t, s["heads"] * s["head_dim"]) @ w[prefix + "o_proj.weight"].T


def decoder_layer(x, positions, w, i, s):
    """flow_engine/model.py:179-202: x += attn(norm1(x)); x += mlp(norm2(x))."""
    p = f"model.layers.{i}."
    x = x + attention_block(rms_norm(x, w[p + "input_layernorm.weight"], s["eps"]),
                            positions, w, p + "self_attn.", s)
    h = rms_norm(x, w[p + "post_attention_layernorm.weight"], s["eps"])
    return x + swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                      w[p + "mlp.down_proj.weight"])


def forward(config, w, tokens, first_position=0):
    """Logits [T, V] at every position of TOKENS (flow_engine/model.py:176-204, all_logits)."""
    s = sizes(config)
    ids = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(first_position, first_position + len(ids))
    x = w["model.embed_tokens.weight"][ids]
    for i in range(s["layers"]):
        x = decoder_layer(x, positions, w, i, s)
    x = rms_norm(x, w["model.norm.weight"], s["eps"])
    head = w["model.embed_tokens.weight"] if s["tied"] else w["lm_head.weight"]
    return (x @ head.T).to(torch.float32)


def greedy(config, w, prompt, count):
    """COUNT greedy tokens after PROMPT by re-running the growing sequence (tests/test_engine.py:41-49)."""
    tokens, out = list(prompt), []
    for _ in range(count):
        nxt = int(forward(config, w, tokens)[-1].argmax())
        out.append(nxt)
        tokens.append(nxt)
    return out


def softmax_temperature(logits, temperature):
    """flow_engine/engine.py:157: probabilities softmax(logits / T) in float32."""
    z = logits.to(torch.float32) / temperature
    z = z - z.max()
    e = torch.exp(z)
    return e / e.sum()
