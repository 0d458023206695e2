"""Tiny configurations of the architecture that differ in every size and option. A and B have small
heads (16, 32); C has the head size of the real checkpoints (128), whose kernels are separate
instantiations, two query heads per kv head, and pages of 32."""

TINY_A = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, use_sliding_window=False, max_position_embeddings=512, hidden_act="silu")
TINY_A_PAGE, TINY_A_SEED = 16, 0

TINY_B = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=3, hidden_size=192, num_attention_heads=6, num_key_value_heads=1, head_dim=32,
    intermediate_size=328, vocab_size=389, rope_theta=1e6, rms_norm_eps=1e-5,
    tie_word_embeddings=False, use_sliding_window=False, max_position_embeddings=1024, hidden_act="silu")
TINY_B_PAGE, TINY_B_SEED = 8, 1

TINY_C = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=2, hidden_size=256, num_attention_heads=2, num_key_value_heads=1, head_dim=128,
    intermediate_size=336, vocab_size=300, rope_theta=5e5, rms_norm_eps=1e-6,
    tie_word_embeddings=False, use_sliding_window=False, max_position_embeddings=1024, hidden_act="silu")
TINY_C_PAGE, TINY_C_SEED = 32, 2

# B with the intermediate size 320 (a multiple of 16: gate and up rows interleave and the SiLU-multiply runs in
# the matrix kernel's epilogue, where B's 328 takes the separate kernel)
TINY_B320 = dict(TINY_B, intermediate_size=320)

TINY = {"A": (TINY_A, TINY_A_PAGE, TINY_A_SEED), "B": (TINY_B, TINY_B_PAGE, TINY_B_SEED),
        "C": (TINY_C, TINY_C_PAGE, TINY_C_SEED), "B320": (TINY_B320, TINY_B_PAGE, TINY_B_SEED)}


def make_folder(path, name):
    """Write tiny configuration NAME with random weights into PATH; returns (config dict, page size)."""
    from tessweave_engine_amd.config import config_from_dict
    from tessweave_engine_amd.weights import write_model_folder
    cfg, page, seed = TINY[name]
    write_model_folder(path, config_from_dict(cfg), seed)
    return cfg, page
