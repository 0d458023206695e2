"""Randomly drawn configurations through trace replay against the plain implementation.

Each seed draws every size and option (head sizes in steps of 16 up to 256, odd counts of heads and
groups, feed-forward widths and vocabularies that are multiples of nothing, number of layers, eps, theta,
tied or untied head, page sizes from 4 to 64) and replays four requests whole, with the last 32 tokens one
by one, and mixed with few pages, in both precisions: bfloat16 with the bar of test_replay_gpu, float32 with
its calibrated bar (against the plain implementation in float64, at most four times the plain float32's own
error: widths from 16 to 2,064 round very differently). Head sizes that
are even but no multiple of 16 (18, 24, 72, 2, 250) replay the same way; above 256 the model is refused.
"""
import random

import pytest
import torch

import plain_model as plain
import test_replay_gpu as replay_tests

pytestmark = pytest.mark.gpu


def draw(seed):
    rng = random.Random(seed)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 208, 256])
    kv = rng.choice([1, 1, 2, 3, 4])
    heads = kv * rng.choice([1, 2, 3, 5, 7, 8])
    if heads * head_dim > 1600:
        heads = kv = 1
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=rng.choice([1, 2, 3]),
               hidden_size=heads * head_dim, num_attention_heads=heads, num_key_value_heads=kv, head_dim=head_dim,
               intermediate_size=rng.choice([16, 40, 88, 100, 136, 200, 328, 1000, 1023, 2064]),
               vocab_size=rng.choice([17, 100, 255, 389, 1001, 4099]), rope_theta=rng.choice([1e4, 5e5, 1e6]),
               rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-3]), tie_word_embeddings=rng.random() < 0.5,
               use_sliding_window=False, max_position_embeddings=1024, hidden_act="silu")
    return cfg, rng.choice([4, 8, 16, 32, 64]), [rng.randrange(34, 140) for _ in range(4)]


@pytest.mark.parametrize("seed", [3, 14, 15, 92, 65, 35, 89, 79])
def test_a_random_configuration_replays_like_the_plain_implementation(seed, tmp_path, device):
    cfg, page, lengths = draw(seed)
    replay_three_ways(cfg, page, lengths, seed, tmp_path)


def replay_three_ways(cfg, page, lengths, seed, tmp_path):
    from tessweave_engine_amd.config import config_from_dict
    from tessweave_engine_amd.weights import write_model_folder
    folder = tmp_path / "model"
    write_model_folder(folder, config_from_dict(cfg), seed)
    config, weights = plain.read_folder(folder)
    g = torch.Generator().manual_seed(seed)
    requests = {f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}
    want = {rid: plain.forward(config, weights, toks).numpy() for rid, toks in requests.items()}
    weights64 = {k: v.double() for k, v in weights.items()}
    exact = {rid: plain.forward(config, weights64, toks).numpy() for rid, toks in requests.items()}    # summed in float64
    model = dict(name=f"seed {seed}: {cfg}", folder=folder, page=page, cfg=cfg, requests=requests, want=want, exact=exact)
    biggest = max(replay_tests.round64(len(t)) for t in requests.values())
    for dtype in ("float32", "bfloat16"):
        steps, starts = replay_tests.sequential(model, lambda t: [t])
        got = replay_tests.run_trace(model, dtype, steps, biggest, tmp_path / f"whole_{dtype}")
        replay_tests.compare(model, dtype, steps, got, starts)
        steps, starts = replay_tests.sequential(model, lambda t: ([t - 32] if t > 32 else []) + [1] * min(t, 32))
        got = replay_tests.run_trace(model, dtype, steps, biggest, tmp_path / f"last32_{dtype}")
        replay_tests.compare(model, dtype, steps, got, starts)
        steps, starts, peak = replay_tests.mixed_trace(model, seed)
        got = replay_tests.run_trace(model, dtype, steps, peak, tmp_path / f"mixed_{dtype}")
        replay_tests.compare(model, dtype, steps, got, starts)


@pytest.mark.parametrize("head_dim,heads,kv,page", [(18, 4, 2, 8), (24, 6, 1, 16), (72, 2, 2, 4), (2, 8, 4, 16), (250, 2, 1, 32)])
def test_head_sizes_that_are_no_multiple_of_16(head_dim, heads, kv, page, tmp_path, device):
    """Any even head size the configuration allows (flow_engine/config.py:41) runs: on the device such a
    head carries a tail of zeros up to the next multiple of 16, which changes no result."""
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=2, hidden_size=heads * head_dim,
               num_attention_heads=heads, num_key_value_heads=kv, head_dim=head_dim, intermediate_size=88, vocab_size=211,
               rope_theta=1e4, rms_norm_eps=1e-6, tie_word_embeddings=head_dim % 4 == 0, max_position_embeddings=512)
    replay_three_ways(cfg, page, [37, 70, 45, 66], 1000 + head_dim, tmp_path)


def test_a_head_size_above_256_is_refused():
    """The configuration itself is valid; building the model for it is refused with a message that says why."""
    from tessweave_engine_amd.config import build_model, config_from_dict
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=1, hidden_size=2 * 258,
               num_attention_heads=2, num_key_value_heads=1, head_dim=258, intermediate_size=40, vocab_size=50,
               max_position_embeddings=128)
    with pytest.raises(ValueError, match="even head sizes up to 256"):
        build_model(config_from_dict(cfg))
