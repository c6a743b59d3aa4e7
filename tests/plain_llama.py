"""A plain, slow implementation of the Llama 2/3 dense decoder.

Whole sequences, no cache, one function for each part, float32 (or float64) on the
CPU.  It is written from the formulas of the reference's source text and shares no
code with the package under test: it reads ``config.json`` and the safetensors file
with its own few lines, and every function below names the reference lines it
follows (paths relative to the reference checkout).
"""
import json
import math
import os

import torch

# --------------------------------------------------------------------------- config


def find_multiple(n, k):
    """model.py:16-19 : round n up to a multiple of k."""
    return n if n % k == 0 else n + k - (n % k)


def read_config(folder):
    """The sizes of model.py:21-42 under a checkpoint folder's config.json keys."""
    with open(os.path.join(folder, "config.json")) as f:
        c = json.load(f)
    return config_from_dict(c)


def config_from_dict(c):
    dim = c["hidden_size"]
    n_head = c["num_attention_heads"]
    n_kv = c.get("num_key_value_heads") or n_head          # model.py:36-37
    inter = c.get("intermediate_size")
    if inter is None:                                       # model.py:38-41
        inter = find_multiple(int(2 * (4 * dim) / 3), 256)
    head_dim = c.get("head_dim") or dim // n_head           # model.py:42
    scaling = c.get("rope_scaling")
    if scaling is not None:
        kind = scaling.get("rope_type", scaling.get("type"))
        if kind in (None, "default"):
            scaling = None
        else:
            assert kind == "llama3", kind
    return dict(
        dim=dim, n_layer=c["num_hidden_layers"], n_head=n_head, n_kv=n_kv,
        head_dim=head_dim, inter=inter, vocab=c["vocab_size"],
        rope_base=float(c.get("rope_theta", 10000.0)),
        eps=float(c.get("rms_norm_eps", 1e-5)),
        rope_scaling=scaling,
        tie=bool(c.get("tie_word_embeddings", False)),
    )


# --------------------------------------------------------------------------- weights


def read_safetensors(path):
    """Own reader: 8-byte little-endian header length, JSON header, raw data.  Values come
    back as float32 (integers as stored); the file is mapped, not read whole."""
    import numpy as np
    mm = np.memmap(path, dtype=np.uint8, mode="r")
    n = int.from_bytes(mm[:8].tobytes(), "little")
    header = json.loads(mm[8:8 + n].tobytes().decode("utf-8"))
    base = 8 + n
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        buf = mm[base + lo:base + hi]
        dt = meta["dtype"]
        shape = meta["shape"]
        if dt == "F32":
            t = torch.from_numpy(np.array(buf.view("<f4")))
        elif dt == "BF16":                      # a bfloat16 is the upper half of a float32
            u = np.empty(buf.size // 2, dtype=np.uint32)
            u[:] = buf.view("<u2")
            u <<= 16
            t = torch.from_numpy(u.view(np.float32))
        elif dt == "F16":
            t = torch.from_numpy(np.array(buf.view("<f2"))).float()
        elif dt == "F64":
            t = torch.from_numpy(np.array(buf.view("<f8")))
        elif dt in ("I32", "I64"):
            t = torch.from_numpy(np.array(buf.view("<i4" if dt == "I32" else "<i8")))
        else:
            raise ValueError(f"{name}: dtype {dt}")
        out[name] = t.reshape(shape)
    return out


def permute_rows(w, n_head, head_dim):
    """scripts/convert_hf_checkpoint.py:75-81 : within each head, row h*hd/2+i of the
    half-split layout goes to row 2i+h of the interleaved layout."""
    cols = w.shape[1]
    return (w.view(n_head, 2, head_dim // 2, cols).transpose(1, 2)
             .reshape(n_head * head_dim, cols))


def internal_weights(hf, cfg, dtype=torch.float32):
    """scripts/convert_hf_checkpoint.py:58-72 (names), :105-115 (permute q and k, fuse
    q,k,v into wqkv).  Returns the reference's state-dict names (model.py:107-110,
    :158-159, :172-175, :222-224)."""
    w = {}
    g = lambda k: hf[k].to(dtype)
    w["tok_embeddings.weight"] = g("model.embed_tokens.weight")
    w["norm.weight"] = g("model.norm.weight")
    w["output.weight"] = (g("lm_head.weight") if "lm_head.weight" in hf
                          else w["tok_embeddings.weight"])
    for i in range(cfg["n_layer"]):
        p = f"model.layers.{i}."
        q = permute_rows(g(p + "self_attn.q_proj.weight"), cfg["n_head"], cfg["head_dim"])
        k = permute_rows(g(p + "self_attn.k_proj.weight"), cfg["n_kv"], cfg["head_dim"])
        v = g(p + "self_attn.v_proj.weight")
        o = f"layers.{i}."
        w[o + "attention.wqkv.weight"] = torch.cat([q, k, v])
        w[o + "attention.wo.weight"] = g(p + "self_attn.o_proj.weight")
        w[o + "feed_forward.w1.weight"] = g(p + "mlp.gate_proj.weight")
        w[o + "feed_forward.w3.weight"] = g(p + "mlp.up_proj.weight")
        w[o + "feed_forward.w2.weight"] = g(p + "mlp.down_proj.weight")
        w[o + "attention_norm.weight"] = g(p + "input_layernorm.weight")
        w[o + "ffn_norm.weight"] = g(p + "post_attention_layernorm.weight")
    return w


def load_folder(folder, dtype=torch.float32):
    cfg = read_config(folder)
    hf = read_safetensors(os.path.join(folder, "model.safetensors"))
    return cfg, internal_weights(hf, cfg, dtype)


# --------------------------------------------------------------------------- parts


def rms_norm(x, weight, eps):
    """model.py:236-241 : x * rsqrt(mean(x*x, -1) + eps), then times weight."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(ms + eps) * weight


def rope_frequencies(head_dim, base):
    """model.py:271 : f_i = 1 / base^(2i/hd), float32 arithmetic."""
    return 1.0 / (base ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))


def scale_frequencies(freqs, scaling):
    """model.py:244-263 : Llama-3.1 rescale of each frequency by its wavelength."""
    factor = scaling["factor"]
    low = scaling["low_freq_factor"]
    high = scaling["high_freq_factor"]
    old_len = scaling["original_max_position_embeddings"]
    low_wavelen = old_len / low
    high_wavelen = old_len / high
    out = []
    for f in freqs:
        wavelen = 2 * math.pi / f
        if wavelen < high_wavelen:
            out.append(f)
        elif wavelen > low_wavelen:
            out.append(f / factor)
        else:
            smooth = (old_len / wavelen - low) / (high - low)
            out.append((1 - smooth) * f / factor + smooth * f)
    return torch.tensor([float(v) for v in out], dtype=freqs.dtype)


def rope_table(positions, head_dim, base, scaling=None, dtype=torch.float32):
    """model.py:266-278 : angle[p,i] = p * f_i ; returns cos, sin of [P, hd/2]."""
    freqs = rope_frequencies(head_dim, base)
    if scaling is not None:
        freqs = scale_frequencies(freqs, scaling)
    ang = torch.outer(torch.as_tensor(positions).to(freqs.dtype), freqs)  # float32 product
    return torch.cos(ang).to(dtype), torch.sin(ang).to(dtype)


def apply_rope(x, cos, sin):
    """model.py:281-293 : pairs (x[2i], x[2i+1]) rotated by the angle of (position, i).
    x: [S, heads, hd]; cos, sin: [S, hd/2]."""
    S, nh, hd = x.shape
    xs = x.reshape(S, nh, hd // 2, 2)
    a, b = xs[..., 0], xs[..., 1]
    c, s = cos[:, None, :], sin[:, None, :]
    out = torch.stack([a * c - b * s, b * c + a * s], dim=-1)
    return out.reshape(S, nh, hd)


def causal_attention(q, k, v):
    """model.py:209-211 with the mask of model.py:134,138 : query head h reads kv head
    h // (H/Hkv) (repeat_interleave); scores / sqrt(hd); keys j <= i kept; softmax; PV.
    q: [S, H, hd]; k, v: [S, Hkv, hd] -> [S, H, hd]."""
    S, H, hd = q.shape
    Hkv = k.shape[1]
    rep = H // Hkv
    out = torch.empty_like(q)
    keep = torch.tril(torch.ones(S, S, dtype=torch.bool))
    for h in range(H):
        g = h // rep
        scores = (q[:, h, :] @ k[:, g, :].T) / math.sqrt(hd)
        scores = scores.masked_fill(~keep, float("-inf"))
        p = torch.softmax(scores, dim=-1)
        out[:, h, :] = p @ v[:, g, :]
    return out


def attention(x, wqkv, wo, cfg, positions):
    """model.py:191-216 : fused projection, split, rotate q and k, attend, project."""
    S = x.shape[0]
    H, Hkv, hd = cfg["n_head"], cfg["n_kv"], cfg["head_dim"]
    qkv = x @ wqkv.T
    q, k, v = qkv.split([H * hd, Hkv * hd, Hkv * hd], dim=-1)
    q = q.reshape(S, H, hd)
    k = k.reshape(S, Hkv, hd)
    v = v.reshape(S, Hkv, hd)
    cos, sin = rope_table(positions, hd, cfg["rope_base"], cfg["rope_scaling"], x.dtype)
    q = apply_rope(q, cos, sin)
    k = apply_rope(k, cos, sin)
    y = causal_attention(q, k, v).reshape(S, H * hd)
    return y @ wo.T


def feed_forward(x, w1, w3, w2):
    """model.py:226-227 : w2( silu(w1 x) * (w3 x) )."""
    a = x @ w1.T
    return ((a * torch.sigmoid(a)) * (x @ w3.T)) @ w2.T


def block(x, w, i, cfg, positions):
    """model.py:161-164 : h = x + attn(norm(x)); out = h + ffn(norm(h))."""
    p = f"layers.{i}."
    h = x + attention(rms_norm(x, w[p + "attention_norm.weight"], cfg["eps"]),
                      w[p + "attention.wqkv.weight"], w[p + "attention.wo.weight"],
                      cfg, positions)
    return h + feed_forward(rms_norm(h, w[p + "ffn_norm.weight"], cfg["eps"]),
                            w[p + "feed_forward.w1.weight"],
                            w[p + "feed_forward.w3.weight"],
                            w[p + "feed_forward.w2.weight"])


def forward(w, cfg, tokens, first_position=0):
    """model.py:136-146 : embed, blocks, final norm, output head; logits of every
    position of one whole sequence, [S, V]."""
    idx = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(first_position, first_position + idx.numel())
    x = w["tok_embeddings.weight"][idx]
    for i in range(cfg["n_layer"]):
        x = block(x, w, i, cfg, positions)
    x = rms_norm(x, w["norm.weight"], cfg["eps"])
    return x @ w["output.weight"].T


# --------------------------------------------------------------------------- sampling


def logits_to_probs(logits, temperature=1.0, top_k=None):
    """generate.py:44-52 : divide by max(T, 1e-5); keep values >= the k-th largest;
    softmax."""
    logits = logits / max(temperature, 1e-5)
    if top_k is not None:
        v, _ = torch.topk(logits, min(top_k, logits.size(-1)))
        pivot = v[..., -1:]
        logits = torch.where(logits < pivot, torch.full_like(logits, float("-inf")), logits)
    return torch.softmax(logits, dim=-1)


def sample_with_noise(probs, noise):
    """generate.py:40-42 : argmax(probs / q), q ~ Exp(1) given by the caller."""
    return torch.argmax(probs / noise, dim=-1)


def greedy_generate(w, cfg, prompt, max_new_tokens, stop_tokens=()):
    """generate.py:59-83, 139-211 with argmax in place of sampling: the whole sequence
    is run again for every new token."""
    seq = list(prompt)
    new = []
    for _ in range(max_new_tokens):
        logits = forward(w, cfg, seq)
        t = int(torch.argmax(logits[-1]))
        seq.append(t)
        new.append(t)
        if t in stop_tokens:
            break
    return new
