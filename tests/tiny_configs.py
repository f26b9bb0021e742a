"""Tiny configurations (config.json dictionaries) used by the tests.

TINY_LLAMA and TINY_MISTRAL differ in every size and option: head counts and
groups, head size, width and hidden width that are no powers of two, number of
layers, vocabulary, eps, theta, window, tied / untied head; TINY_WIDE_HEADS and what is made from it
have the reference's other activation (gelu)."""
import copy

TINY_LLAMA = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 64,
    "intermediate_size": 176,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 16,
    "vocab_size": 256,
    "max_position_embeddings": 128,
    "rope_theta": 10000.0,
    "rms_norm_eps": 1e-5,
    "hidden_act": "silu",
    "tie_word_embeddings": True,
    "bos_token_id": 1,
    "eos_token_id": 2,
}

TINY_MISTRAL = {
    "architectures": ["MistralForCausalLM"],
    "hidden_size": 96,
    "intermediate_size": 256,
    "num_hidden_layers": 3,
    "num_attention_heads": 3,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "vocab_size": 320,
    "max_position_embeddings": 64,
    "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6,
    "hidden_act": "silu",
    "sliding_window": 16,
    "tie_word_embeddings": False,
    "bos_token_id": 1,
    "eos_token_id": 2,
}

# llama3 rope scaling with a small original length, so that all three frequency
# regimes occur inside 128 positions; vocabulary that is no multiple of 16.
TINY_LLAMA3 = copy.deepcopy(TINY_LLAMA)
TINY_LLAMA3.update({
    "vocab_size": 250,
    "head_dim": 32,
    "num_attention_heads": 2,
    "num_key_value_heads": 2,
    "rope_theta": 500.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 32},
    "max_position_embeddings": 256,
})

# heads * head_dim != hidden_size (the reference silently assumes equality,
# model.cpp:289); a longer context with a window in the middle of it.
TINY_WIDE_HEADS = copy.deepcopy(TINY_MISTRAL)
TINY_WIDE_HEADS.update({
    "hidden_size": 80,
    "intermediate_size": 208,
    "num_attention_heads": 6,
    "num_key_value_heads": 3,
    "head_dim": 48,
    "vocab_size": 311,
    "num_hidden_layers": 2,
    "sliding_window": 100,
    "max_position_embeddings": 512,
    "rms_norm_eps": 3e-6,
    "hidden_act": "gelu",
})

# a long context without a window: many pages of the cache, far keys
TINY_LONG = copy.deepcopy(TINY_LLAMA)
TINY_LONG.update({
    "max_position_embeddings": 1024,
    "num_hidden_layers": 2,
    "head_dim": 64,
    "hidden_size": 128,
    "num_attention_heads": 4,
    "num_key_value_heads": 1,
    "intermediate_size": 144,
    "vocab_size": 200,
    "tie_word_embeddings": False,
})

# the head size of the big models (128) with a window that prompts and decoding cross:
# the matrix-core attention kernels over a ring of cache pages
SMALL_WINDOWED = copy.deepcopy(TINY_MISTRAL)
SMALL_WINDOWED.update({
    "hidden_size": 256,
    "intermediate_size": 640,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 128,
    "vocab_size": 512,
    "num_hidden_layers": 2,
    "sliding_window": 96,
    "max_position_embeddings": 512,
    "rms_norm_eps": 1e-5,
})

# attention sinks beside a window (what the reference's -T makes of a model): three sinks and a
# window of 37 keys, which prompts and decoding pass several times over; half of each head rotated
TINY_SINKS = copy.deepcopy(TINY_WIDE_HEADS)
TINY_SINKS.update({
    "sliding_window": 37,
    "attention_sinks": 3,
    "partial_rotary_factor": 0.5,
    "rope_theta": 300.0,
})

# the same at the head size of the matrix-core kernels, a context of 96 = 2 sinks + 94
SMALL_SINKS = copy.deepcopy(SMALL_WINDOWED)
SMALL_SINKS.update({
    "sliding_window": 94,
    "attention_sinks": 2,
    "rope_theta": 10000.0,
})

ALL = {
    "small_windowed": SMALL_WINDOWED,
    "small_sinks": SMALL_SINKS,
    "tiny_sinks": TINY_SINKS,
    "tiny_llama": TINY_LLAMA,
    "tiny_mistral": TINY_MISTRAL,
    "tiny_llama3": TINY_LLAMA3,
    "tiny_wide_heads": TINY_WIDE_HEADS,
    "tiny_long": TINY_LONG,
}
