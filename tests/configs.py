"""Tiny Qwen3 configurations for tests.  A and B differ in every size and option; W adds
a sliding window on some layers (two cache groups), a head size that is no power of
two and biases on the q, k and v projections; Y scales its rotation (YaRN) and rotates half of
a head; all have widths and vocabularies that are
no power of two where they can."""

def _cfg(**kw):
    base = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu")
    base.update(kw)
    return base


TINY = {
    "A": dict(
        config=_cfg(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
                    head_dim=32, intermediate_size=128, vocab_size=256, rope_theta=10000.0,
                    rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=128),
        seed=0, linear_std=0.02, norm_std=0.1, page_size=16),
    "B": dict(
        config=_cfg(num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=2,
                    head_dim=16, intermediate_size=224, vocab_size=509, rope_theta=1e6,
                    rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=512),
        seed=1, linear_std=0.03, norm_std=0.05, page_size=8),
    "W": dict(
        config=_cfg(num_hidden_layers=3, hidden_size=80, num_attention_heads=5, num_key_value_heads=5,
                    head_dim=48, intermediate_size=176, vocab_size=300, rope_theta=50000.0,
                    rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=320,
                    sliding_window=24, attention_bias=True,
                    layer_types=["sliding_attention", "full_attention", "sliding_attention"]),
        seed=2, linear_std=0.05, norm_std=0.2, page_size=16),
}

# O: widths that are multiples of neither 8 nor 4, a group of three heads and one layer: every
# kernel's vectorized form has to step aside for its plain one.
TINY["O"] = dict(
    config=_cfg(num_hidden_layers=1, hidden_size=102, num_attention_heads=3, num_key_value_heads=1,
                head_dim=16, intermediate_size=182, vocab_size=257, rope_theta=777.0,
                rms_norm_eps=3e-6, tie_word_embeddings=True, max_position_embeddings=256),
    seed=5, linear_std=0.04, norm_std=0.15, page_size=8)

# Y: YaRN scaling over a given original length (so the model runs further than
# max_position_embeddings: round(40 * 4) = 160 positions), with bounds of the blend that fall
# inside its 8 frequencies, and half of every head rotated.
TINY["Y"] = dict(
    config=_cfg(num_hidden_layers=2, hidden_size=72, num_attention_heads=6, num_key_value_heads=3,
                head_dim=32, intermediate_size=104, vocab_size=211, rope_theta=5000.0,
                rms_norm_eps=2e-6, tie_word_embeddings=True, max_position_embeddings=64,
                partial_rotary_factor=0.5,
                rope_scaling=dict(rope_type="yarn", factor=4.0, original_max_position_embeddings=40,
                                  beta_fast=4.0, beta_slow=1.0, attn_factor=1.25)),
    seed=8, linear_std=0.05, norm_std=0.1, page_size=16)


# Real layer sizes (Qwen3-0.6B, 4B, 8B, 14B and 32B) with few layers and a small vocabulary: the
# kernels run at the head size, group, widths and K lengths they serve in production.
REAL = {
    "8B": dict(
        config=_cfg(num_hidden_layers=2, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                    head_dim=128, intermediate_size=12288, vocab_size=2003, rope_theta=1e6,
                    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=1024),
        seed=3, linear_std=0.02, norm_std=0.1, page_size=64),
    "0.6B": dict(
        config=_cfg(num_hidden_layers=2, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
                    head_dim=128, intermediate_size=3072, vocab_size=1777, rope_theta=1e6,
                    rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=1024),
        seed=6, linear_std=0.03, norm_std=0.1, page_size=64),
    "4B": dict(
        config=_cfg(num_hidden_layers=1, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
                    head_dim=128, intermediate_size=9728, vocab_size=1601, rope_theta=1e6,
                    rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=1024),
        seed=7, linear_std=0.02, norm_std=0.1, page_size=64),
    "14B": dict(
        config=_cfg(num_hidden_layers=1, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                    head_dim=128, intermediate_size=17408, vocab_size=1409, rope_theta=1e6,
                    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=1024),
        seed=8, linear_std=0.02, norm_std=0.1, page_size=64),
    "32B": dict(
        config=_cfg(num_hidden_layers=1, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                    head_dim=128, intermediate_size=25600, vocab_size=1501, rope_theta=1e6,
                    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=1024),
        seed=4, linear_std=0.02, norm_std=0.1, page_size=64),
}


# Long contexts: Qwen3-0.6B widths, two layers, 8,192 positions.  `sharpen` multiplies every
# q_norm weight: scores then have a standard deviation of about 1.5 instead of 1, so that some
# hundred of some thousand keys carry a row's softmax.  More would make a dropped or misplaced key
# show more, but bfloat16's rounding of q and k grows with the scores too (measured on 3,000 tokens:
# worst error 1.1% of the largest logit at 1, 1.4% at 1.5, 2.0% at 2, 2.8% at 3); float32 shows a
# single dropped key at any sharpness.
LONG = dict(
    config=_cfg(num_hidden_layers=2, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
                head_dim=128, intermediate_size=3072, vocab_size=1201, rope_theta=1e6,
                rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=8192),
    seed=9, linear_std=0.03, norm_std=0.1, page_size=64, sharpen=1.5)
