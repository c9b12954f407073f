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

# The layer sizes of the models the library is measured on, with two layers and a
# small vocabulary so that the plain implementation stays quick: grouped heads 3:1
# with a width that is no power of two; one key/value head per query head; groups of 8;
# and a fourth shape that is measured beside BASELINE's three: groups of 4 heads of 128
# channels, a width of 4,096 and an inner size of 14,336.
SHAPE_CONFIGS = {
    "smollm2-135m": (llama(
        num_hidden_layers=2, hidden_size=576, num_attention_heads=9, num_key_value_heads=3, intermediate_size=1536,
        vocab_size=3001, rope_theta=100000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
        max_position_embeddings=2048, torch_dtype="bfloat16"), 11),
    "smollm2-1.7b": (llama(
        num_hidden_layers=2, hidden_size=2048, num_attention_heads=32, num_key_value_heads=32, intermediate_size=8192,
        vocab_size=3001, rope_theta=130000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
        max_position_embeddings=2048, torch_dtype="bfloat16"), 12),
    "tinyllama-1.1b": (llama(
        num_hidden_layers=2, hidden_size=2048, num_attention_heads=32, num_key_value_heads=4, intermediate_size=5632,
        vocab_size=3001, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
        max_position_embeddings=2048, torch_dtype="bfloat16"), 13),
    "llama-8b": (llama(
        num_hidden_layers=2, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=14336,
        vocab_size=3001, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
        max_position_embeddings=2048, torch_dtype="bfloat16"), 14),
}
