"""Helpers shared by the tests: the tiny configurations, model folders made in a
temporary directory, and the comparison of engine logits with the plain implementation."""
import os
import random

import torch

import plain_llama as plain

# Two tiny configurations that differ in every size and option: heads and groups, head
# size, widths that are no power of two, layers, vocabulary, eps, rope base and scaling.
TINY_A = {   # Llama-2 style, MHA, no scaling
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4,
    "num_key_value_heads": 4, "intermediate_size": 176, "vocab_size": 256,
    "max_position_embeddings": 64, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "rope_scaling": None, "tie_word_embeddings": False,
}
TINY_B = {   # Llama-3.1 style, GQA 6:2, llama3 scaling whose three branches all occur
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 192, "num_hidden_layers": 3, "num_attention_heads": 6,
    "num_key_value_heads": 2, "intermediate_size": 512, "vocab_size": 384,
    "max_position_embeddings": 128, "rope_theta": 500000.0, "rms_norm_eps": 1e-6,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 32},
    "tie_word_embeddings": False,
}
TINY_C = {   # odd sizes: head_dim given and != hidden/heads, GQA 5:1... width 200, vocab 1000
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 200, "num_hidden_layers": 2, "num_attention_heads": 10,
    "num_key_value_heads": 5, "head_dim": 48, "intermediate_size": 328, "vocab_size": 1000,
    "max_position_embeddings": 512, "rope_theta": 50000.0, "rms_norm_eps": 3e-6,
    "rope_scaling": None, "tie_word_embeddings": True,
}
TINY_D = {   # sizes the fast kernels refuse: width 100 (no multiple of 8), head size 20, vocab 131
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 100, "num_hidden_layers": 2, "num_attention_heads": 5,
    "num_key_value_heads": 1, "intermediate_size": 52, "vocab_size": 131,
    "max_position_embeddings": 256, "rope_theta": 1000.0, "rms_norm_eps": 1e-5,
    "rope_scaling": None, "tie_word_embeddings": False,
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}


def make_folder(tmp, name, seed=0, dtype="float32", std=0.05):
    """A model folder with random weights, written by the library's random-weights mode.
    std 0.05 rather than 0.02 so that logits of these tiny models are not all near zero."""
    import gpt_fast_amd as gfa
    arch = gfa.config.registry.architecture_of(TINY[name])
    cfg = arch.read_config(TINY[name])
    folder = os.path.join(str(tmp), f"tiny_{name}_{dtype}_{seed}")
    if not os.path.isdir(folder):
        gfa.write_random_model(folder, arch, cfg, seed=seed, dtype=dtype, std=std)
    return folder


def random_tokens(vocab, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def plain_logits(folder, tokens, dtype=torch.float32):
    cfg, w = plain.load_folder(folder, dtype)
    return plain.forward(w, cfg, tokens)


def rel_err(a, b):
    """Largest difference relative to the largest magnitude of the reference."""
    a = a.double().cpu()
    b = b.double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


# Tolerances, stated once.  float32: the engine and the plain implementation do the same
# arithmetic in different orders.  bfloat16: weights are bfloat16 in both; the engine
# also rounds activations to bfloat16 between kernels.
TOL_F32 = 2e-5
TOL_BF16 = 4e-2


def mixed_step_case(V):
    """Five sequences; one step brings three of them one token each, one a chunk of 40
    tokens at position 70, one a fresh prompt of 130 tokens."""
    seqs = {"d0": random_tokens(V, 9, 31), "d1": random_tokens(V, 66, 32),
            "d2": random_tokens(V, 130, 33), "c": random_tokens(V, 112, 34),
            "p": random_tokens(V, 131, 35)}
    before = {"d0": 8, "d1": 65, "d2": 129, "c": 70}            # fed by the earlier step
    mixed = {"d0": 1, "d1": 1, "d2": 1, "c": 40, "p": 130}      # fed by the mixed step
    return seqs, before, mixed


# The order of a cache page's elements, written down from its description in csrc/common.h
# (not shared with the kernels: the kernel tests build and read pages through these).
def key_places(hd):
    """[64, hd] -> place of element (key, d) inside a (page, kv head) region of keys."""
    key = torch.arange(64)[:, None].expand(64, hd)
    d = torch.arange(hd)[None, :].expand(64, hd)
    if hd % 8:
        return key * hd + d
    kk = key % 32                                   # key 8 a + 4 t + b of a block -> slot 16 t + 4 a + b
    slot = ((kk // 4) % 2) * 16 + (kk // 8) * 4 + kk % 4
    return (key // 32) * 32 * hd + (d // 8) * 256 + slot * 8 + d % 8


def value_places(hd):
    """[hd, 64] -> place of element (d, key) inside a (page, kv head) region of values."""
    d = torch.arange(hd)[:, None].expand(hd, 64)
    key = torch.arange(64)[None, :].expand(hd, 64)
    if hd % 16:
        return d * 64 + key
    return (d // 16) * 1024 + (key // 32) * 512 + ((key // 8) % 4) * 128 + (d % 16) * 8 + key % 8


def to_cache_order(k_rows, v_cols):
    """Pages given as keys [n, G, 64, hd] and values [n, G, hd, 64] -> the same shapes with the
    elements where the kernels keep them."""
    n, G, _, hd = k_rows.shape
    k = torch.empty_like(k_rows).view(n, G, -1)
    v = torch.empty_like(v_cols).view(n, G, -1)
    k[..., key_places(hd).reshape(-1)] = k_rows.reshape(n, G, -1)
    v[..., value_places(hd).reshape(-1)] = v_cols.reshape(n, G, -1)
    return k.view_as(k_rows), v.view_as(v_cols)


def from_cache_order(k_pages, v_pages):
    """The inverse: what the kernels keep -> keys [n, G, 64, hd], values [n, G, hd, 64]."""
    n, G, _, hd = k_pages.shape
    k = k_pages.reshape(n, G, -1)[..., key_places(hd).reshape(-1)].view(n, G, 64, hd)
    v = v_pages.reshape(n, G, -1)[..., value_places(hd).reshape(-1)].view(n, G, hd, 64)
    return k, v


# The sampler's noise, written again from its description (gpt_fast_amd/sampling): a request's
# draw at sequence position ``pos`` compares p_i / q_i with q_i = -log(u_i), u_i = (n_i + 1/2) /
# 2^23, n_i the upper 23 bits of word i % 4 of Philox4x32-10 (Salmon et al., "Parallel random
# numbers: as easy as 1, 2, 3") with counter (i // 4, pos, request key, 0) and key (seed's low
# word, seed's high word).
def philox4x32_10(c0, c1, c2, c3, k0, k1):
    import numpy as np
    c0, c1, c2, c3 = (np.asarray(c, dtype=np.uint64) for c in (c0, c1, c2, c3))
    mask = np.uint64(0xFFFFFFFF)
    k0, k1 = np.uint64(k0), np.uint64(k1)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c0
        p1 = np.uint64(0xCD9E8D57) * c2
        c0, c1, c2, c3 = (p1 >> np.uint64(32)) ^ c1 ^ k0, p1 & mask, (p0 >> np.uint64(32)) ^ c3 ^ k1, p0 & mask
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    return c0, c1, c2, c3


def sampler_noise(vocab, seed, key, pos):
    """float64 [vocab]: the q_i of one draw."""
    import numpy as np
    blocks = np.arange((vocab + 3) // 4, dtype=np.uint64)
    same = np.zeros_like(blocks)
    words = philox4x32_10(blocks, same + np.uint64(pos), same + np.uint64(key), same,
                          seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)
    n = np.stack(words, axis=1).reshape(-1)[:vocab] >> np.uint64(9)
    return torch.from_numpy(-np.log((n.astype(np.float64) + 0.5) / 8388608.0))
