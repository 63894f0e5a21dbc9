"""Tiny configurations of the architecture that differ in every size and option.

A: tied head, head_dim = hidden / heads, group 2, theta 1e4, eps 1e-6, 2 layers.
B: untied head, head_dim decoupled (H * D = 256 vs hidden 96), group 4, theta 1e6,
   eps 1e-5, 3 layers, intermediate 224 (no power of two), vocab 512.
C: sliding window of 24 keys on the layers from index 2 on (two cache groups),
   group 3, head_dim 48, hidden 80, vocab 331 and intermediate 136 (no powers of two),
   5 layers, theta 5e4, eps 3e-6, tied.
"""


def _cfg(**kw):
    base = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", attention_bias=False)
    base.update(kw)
    return base


CONFIGS = {
    "A": (_cfg(vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
               num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-6, rope_theta=10000.0,
               max_position_embeddings=128, tie_word_embeddings=True, eos_token_id=7), 11),
    "B": (_cfg(vocab_size=512, hidden_size=96, intermediate_size=224, num_hidden_layers=3, num_attention_heads=8,
               num_key_value_heads=2, head_dim=32, rms_norm_eps=1e-5, rope_theta=1000000.0,
               max_position_embeddings=256, tie_word_embeddings=False, eos_token_id=[3, 5]), 22),
    "C": (_cfg(vocab_size=331, hidden_size=80, intermediate_size=136, num_hidden_layers=5, num_attention_heads=6,
               num_key_value_heads=2, head_dim=48, rms_norm_eps=3e-6, rope_theta=50000.0,
               max_position_embeddings=512, tie_word_embeddings=True, use_sliding_window=True, sliding_window=24,
               max_window_layers=2), 33),
}

# page size used with each configuration in the engine tests
PAGE = {"A": 4, "B": 8, "C": 16}
