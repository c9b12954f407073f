"""Tiny configurations of the architecture for the tests.  A and B differ in
every size and option (layers, width, heads and groups, head size, inner size,
vocabulary, rope theta, norm eps, tied or untied head, positions); C has a
head_dim key that does not equal hidden_size / heads, grouped heads 3:1 and
weights stored in 32-bit.  None of the sizes is a power of two where it need
not be."""


def llama(**overrides):
    config = {
        "architectures": ["LlamaForCausalLM"],
        "model_type": "llama",
        "hidden_act": "silu",
    }
    config.update(overrides)
    return config


TINY_A = llama(
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
    intermediate_size=176, vocab_size=512, rope_theta=10000.0, rms_norm_eps=1e-5,
    tie_word_embeddings=True, max_position_embeddings=256, torch_dtype="bfloat16", eos_token_id=2,
)
TINY_B = llama(
    num_hidden_layers=3, hidden_size=96, num_attention_heads=3, num_key_value_heads=1,
    intermediate_size=256, vocab_size=1000, rope_theta=100000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=False, max_position_embeddings=512, torch_dtype="bfloat16",
)
TINY_C = llama(
    num_hidden_layers=2, hidden_size=160, num_attention_heads=6, num_key_value_heads=2, head_dim=64,
    intermediate_size=336, vocab_size=777, rope_theta=50000.0, rms_norm_eps=3e-6,
    tie_word_embeddings=False, max_position_embeddings=384, torch_dtype="float32", eos_token_id=[5, 9],
)

# name -> (config, weight seed)
TINY_CONFIGS = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2)}
