"""The tiny configurations the tests run: they differ in every size and option.

A and B are the benchmark description's tiny models; C makes num_heads * head_dim
differ from hidden_size (an explicit head_dim key) and uses sizes that are no powers
of two, which neither A nor B pins.
"""

TINY_A = dict(
    model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=512, hidden_size=64,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, intermediate_size=176,
    rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True, hidden_act="silu",
    use_sliding_window=False, max_position_embeddings=256,
)
TINY_B = dict(
    model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=1000, hidden_size=192,
    num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1, intermediate_size=384,
    rms_norm_eps=1e-5, rope_theta=1000000.0, tie_word_embeddings=False, hidden_act="silu",
    use_sliding_window=False, max_position_embeddings=512,
)
TINY_C = dict(
    model_type="qwen2", vocab_size=777, hidden_size=80, head_dim=48,
    num_hidden_layers=2, num_attention_heads=3, num_key_value_heads=3, intermediate_size=100,
    rms_norm_eps=3e-6, rope_theta=50000.0, tie_word_embeddings=False,
)
# name -> (config, weight seed, cache block size)
TINY_CONFIGS = {"A": (TINY_A, 0, 16), "B": (TINY_B, 1, 8), "C": (TINY_C, 5, 16)}

# Sizes that none of the above pins: groups of 5, 7, 14, 17 and 66 query heads (17 and more: more than one
# workgroup of the decode kernel takes), widths that are multiples of 2 only or odd, a feed-forward of 7,
# pages of 4, 24 and 48 tokens, head sizes 32 to 256. name -> (config, weight seed, block size)
ODD_CONFIGS = {
    "group14": (dict(model_type="qwen2", vocab_size=1001, hidden_size=66, head_dim=96, num_hidden_layers=2,
                     num_attention_heads=42, num_key_value_heads=3, intermediate_size=255, rms_norm_eps=1e-5,
                     rope_theta=50000.0, tie_word_embeddings=False), 11, 16),
    "pages_of_4": (dict(model_type="qwen2", vocab_size=127, hidden_size=130, head_dim=256, num_hidden_layers=3,
                        num_attention_heads=15, num_key_value_heads=3, intermediate_size=33, rms_norm_eps=3e-4,
                        rope_theta=10000.0, tie_word_embeddings=False), 12, 4),
    "narrow": (dict(model_type="qwen2", vocab_size=51, hidden_size=66, head_dim=32, num_hidden_layers=2,
                    num_attention_heads=14, num_key_value_heads=2, intermediate_size=7, rms_norm_eps=1e-6,
                    rope_theta=1000000.0, tie_word_embeddings=True), 13, 24),
    "group17": (dict(model_type="qwen2", vocab_size=2049, hidden_size=1032, head_dim=160, num_hidden_layers=1,
                     num_attention_heads=34, num_key_value_heads=2, intermediate_size=1000, rms_norm_eps=1e-6,
                     rope_theta=1000000.0, tie_word_embeddings=True), 14, 48),
    # odd widths (rows that no 16-byte load fits) and a group of 66 query heads on one key head
    "odd_widths": (dict(model_type="qwen2", vocab_size=33, hidden_size=65, head_dim=16, num_hidden_layers=2,
                        num_attention_heads=3, num_key_value_heads=1, intermediate_size=9, rms_norm_eps=1e-6,
                        rope_theta=10000.0, tie_word_embeddings=False), 15, 8),
    "group66": (dict(model_type="qwen2", vocab_size=300, hidden_size=72, head_dim=32, num_hidden_layers=1,
                     num_attention_heads=66, num_key_value_heads=1, intermediate_size=50, rms_norm_eps=1e-6,
                     rope_theta=10000.0, tie_word_embeddings=False), 16, 16),
}

# Layers wide enough for the decode kernels that only take large shapes (the persistent
# weight-streaming product, the norm fused into the gate/up product): hidden >= 1024 and at least
# 512 row tiles of 8 in the feed-forward. Two layers and a small vocabulary keep it quick.
WIDE = dict(
    model_type="qwen2", vocab_size=1203, hidden_size=1024, num_hidden_layers=2, num_attention_heads=8,
    num_key_value_heads=2, intermediate_size=4360, rms_norm_eps=2e-6, rope_theta=300000.0,
    tie_word_embeddings=False,
)

# One layer each of the larger models the engine is meant for (Qwen2.5-7B and -32B layer sizes, a
# small vocabulary): products whose K does not fit the streaming kernel's registers, groups of 7
# and 5 query heads per key head, 18944 / 27648-wide feed-forwards.
# One layer of exactly the benchmark's model (Qwen2.5-1.5B): its widths, its full vocabulary, its
# tied output head.
LAYER_1P5B = dict(
    model_type="qwen2", vocab_size=151936, hidden_size=1536, num_hidden_layers=1, num_attention_heads=12,
    num_key_value_heads=2, intermediate_size=8960, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=True,
)
LAYER_7B = dict(
    model_type="qwen2", vocab_size=1501, hidden_size=3584, num_hidden_layers=1, num_attention_heads=28,
    num_key_value_heads=4, intermediate_size=18944, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=False,
)
LAYER_32B = dict(
    model_type="qwen2", vocab_size=1302, hidden_size=5120, num_hidden_layers=1, num_attention_heads=40,
    num_key_value_heads=8, intermediate_size=27648, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=False,
)
