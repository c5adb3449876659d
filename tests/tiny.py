"""The tiny configurations of the tests.  A and B differ in every size and option: layers, width,
heads and groups, head size, feed-forward width (no powers of two), vocabulary, rotary base and
scaling, norm eps, tied or untied output matrix, position limit."""
import os

TINY_A = {
    "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 160, "vocab_size": 256,
    "rope_theta": 10000.0, "rope_scaling": None, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": True, "max_position_embeddings": 128, "hidden_act": "silu",
    "eos_token_id": 2, "bos_token_id": 1,
}

TINY_B = {
    "model_type": "llama", "num_hidden_layers": 3, "hidden_size": 192, "num_attention_heads": 6,
    "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 512, "vocab_size": 1000,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 256,
    "hidden_act": "silu", "eos_token_id": [7, 9], "bos_token_id": 0,
}

# head_dim differs from hidden_size / heads, three kv groups, qkv bias, odd-ish sizes
TINY_C = {
    "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 96, "num_attention_heads": 6,
    "num_key_value_heads": 3, "head_dim": 48, "intermediate_size": 208, "vocab_size": 517,
    "rope_theta": 10000.0, "rope_scaling": {"rope_type": "linear", "factor": 2.0},
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 512,
    "attention_bias": True, "hidden_act": "silu", "eos_token_id": 3,
}


# The middle band at the parameters of the released 1B and 3B models (factor 32, original window
# 8,192, base 500,000, head size 64) and of Tiny B, worked out apart from the code under test with
# 50 decimal digits: pair j has frequency f = base^(-2j/hd) and wavelength 2 pi / f; with
# s = (window / wavelength - low) / (high - low), linear in the quotient of the frequencies, the
# scaled frequency is (1 - s) f / factor + s f.  A blend that is linear in the wavelength instead
# keeps the bands, their bounds and the continuity at both edges, and gives 42 % to 158 % more at
# these pairs.  Parity with the table that the reference's exporter stores
# (tools/llama_exporter.py:54-62 takes it from an external rotary module) is not pinned by any file
# of the reference: these numbers hold the published rule.
LLAMA3_MIDDLE_BAND = [
    ((32.0, 1.0, 4.0, 8192, 500000.0, 64), {14: 0.003211445994752591, 15: 0.0012905479282092638,
                                           16: 0.0004295567965593682, 17: 9.708287802627673e-05,
                                           18: 1.9461638184831125e-05}),
    ((8.0, 1.0, 4.0, 64, 500000.0, 32), {1: 0.44036660267178046, 2: 0.0794030091792082, 3: 0.010674637535720701}),
]


def make_model(tmpdir, cfg_dict, seed=0, std=0.08, norm_std=0.2, name="model", stored="bfloat16"):
    """Writes a model folder through the library's random-weights mode.  The spread of the
    weights is wider than the usual 0.02 so that attention is far from uniform, and norm scales
    are jittered so that a missing scale shows.  ``stored``: the float type the file holds
    ("float32": full significands, which no 16-bit type can carry)."""
    import torch
    from libllm_amd.config import config_from_dict
    from libllm_amd.weights import write_random_model
    path = os.path.join(str(tmpdir), name)
    write_random_model(path, config_from_dict(cfg_dict), seed=seed, std=std, norm_std=norm_std,
                       dtype=getattr(torch, stored))
    return path
