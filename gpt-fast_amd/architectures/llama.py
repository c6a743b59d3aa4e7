"""The Llama 2/3 dense decoder as data: its plan and its checkpoint layout.

Plan: every layer is a pre-norm block of grouped-query attention with interleaved
rotary pairs and a SwiGLU feed-forward (reference model.py:102-227); layers run once
each, in order, each with a cache of its own.

Checkpoint layout: the names of a checkpoint folder map to the reference's state-dict
names as in scripts/convert_hf_checkpoint.py:58-72; the rows of q and k are permuted
from the half-split to the interleaved pair layout (:75-81, 110-111) and q, k, v are
fused into ``wqkv`` (:112).  The gate and up projections are kept as one matrix ``w13``
(rows of w1, then rows of w3), a private layout for the fused gate kernel.
"""
import torch

from ..config.llama import LlamaConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import (AttentionSpec, GatedFeedForwardSpec, LayerSpec, ModelPlan,
                           NormSpec, PositionSpec, Run)
from ..weights.bindings import Binding, CheckpointLayout, Source


def llama_plan(c: LlamaConfig) -> ModelPlan:
    position = PositionSpec(kind="rope", rotary_dim=c.head_dim, base=c.rope_theta,
                            layout="interleaved", scaling=c.rope_scaling)
    layers = []
    for i in range(c.num_hidden_layers):
        layers.append(LayerSpec(
            name=f"layers.{i}",
            arrangement="pre_norm",
            mixer=AttentionSpec(dim=c.hidden_size, n_heads=c.num_attention_heads,
                                n_kv_heads=c.num_key_value_heads, head_dim=c.head_dim,
                                position=position),
            mixer_norm=NormSpec(c.hidden_size, c.rms_norm_eps),
            feed_forward=GatedFeedForwardSpec(c.hidden_size, c.intermediate_size, "silu"),
            feed_forward_norm=NormSpec(c.hidden_size, c.rms_norm_eps),
            mixer_name="attention", mixer_norm_name="attention_norm",
            feed_forward_name="feed_forward", feed_forward_norm_name="ffn_norm"))
    plan = ModelPlan(
        dim=c.hidden_size, vocab_size=c.vocab_size, layers=layers,
        order=[Run(i) for i in range(c.num_hidden_layers)],
        final_norm=NormSpec(c.hidden_size, c.rms_norm_eps),
        tie_embeddings=c.tie_word_embeddings,
        max_positions=c.max_position_embeddings,
        stop_tokens=tuple(c.eos_token_id))
    plan.validate()
    return plan


def interleave_rotary_rows(w: torch.Tensor, n_heads: int, head_dim: int) -> torch.Tensor:
    """Row ``h*hd/2 + i`` of each head (half-split pairs) becomes row ``2i + h``
    (interleaved pairs): scripts/convert_hf_checkpoint.py:75-81."""
    cols = w.shape[1]
    return (w.view(n_heads, 2, head_dim // 2, cols).transpose(1, 2)
             .reshape(n_heads * head_dim, cols))


def llama_bindings(c: LlamaConfig) -> CheckpointLayout:
    D, H, G, hd = c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim
    I, V = c.intermediate_size, c.vocab_size

    def fuse_qkv(parts):
        q, k, v = parts
        return torch.cat([interleave_rotary_rows(q, H, hd),
                          interleave_rotary_rows(k, G, hd), v])

    b = [Binding("tok_embeddings.weight", (Source("model.embed_tokens.weight", (V, D)),))]
    for i in range(c.num_hidden_layers):
        src, dst = f"model.layers.{i}.", f"layers.{i}."
        b += [
            Binding(dst + "attention_norm.weight",
                    (Source(src + "input_layernorm.weight", (D,), "norm"),), role="vector"),
            Binding(dst + "attention.wqkv",
                    (Source(src + "self_attn.q_proj.weight", (H * hd, D)),
                     Source(src + "self_attn.k_proj.weight", (G * hd, D)),
                     Source(src + "self_attn.v_proj.weight", (G * hd, D))),
                    combine=fuse_qkv),
            Binding(dst + "attention.wo",
                    (Source(src + "self_attn.o_proj.weight", (D, H * hd)),)),
            Binding(dst + "ffn_norm.weight",
                    (Source(src + "post_attention_layernorm.weight", (D,), "norm"),),
                    role="vector"),
            Binding(dst + "feed_forward.w13",
                    (Source(src + "mlp.gate_proj.weight", (I, D)),
                     Source(src + "mlp.up_proj.weight", (I, D))),
                    combine=torch.cat),
            Binding(dst + "feed_forward.w2",
                    (Source(src + "mlp.down_proj.weight", (D, I)),)),
        ]
    b.append(Binding("norm.weight", (Source("model.norm.weight", (D,), "norm"),),
                     role="vector"))
    b.append(Binding("output.weight", (Source("lm_head.weight", (V, D)),),
                     alias_of="tok_embeddings.weight" if c.tie_word_embeddings else None))
    # the converter drops rotary_emb.inv_freq (scripts/convert_hf_checkpoint.py:64,97-98)
    return CheckpointLayout(tuple(b), ignored=(r"\.rotary_emb\.inv_freq$",))


def llama_native_layouts(c: LlamaConfig):
    """The reference's own tensor names, as its state dict has them after conversion
    (model.py:107-110, 158-159, 172-175, 222-224): rows already interleaved, the three
    projections fused as ``wqkv`` - or still apart as ``wq``, ``wk``, ``wv``, which the
    reference joins without a permutation when it loads (model.py:184-189)."""
    D, H, G, hd = c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim
    I, V = c.intermediate_size, c.vocab_size

    def layout(fused: bool) -> CheckpointLayout:
        b = [Binding("tok_embeddings.weight", (Source("tok_embeddings.weight", (V, D)),))]
        for i in range(c.num_hidden_layers):
            p = f"layers.{i}."
            if fused:
                qkv = Binding(p + "attention.wqkv",
                              (Source(p + "attention.wqkv.weight", ((H + 2 * G) * hd, D)),))
            else:
                qkv = Binding(p + "attention.wqkv",
                              (Source(p + "attention.wq.weight", (H * hd, D)),
                               Source(p + "attention.wk.weight", (G * hd, D)),
                               Source(p + "attention.wv.weight", (G * hd, D))),
                              combine=torch.cat)
            b += [
                Binding(p + "attention_norm.weight",
                        (Source(p + "attention_norm.weight", (D,), "norm"),), role="vector"),
                qkv,
                Binding(p + "attention.wo", (Source(p + "attention.wo.weight", (D, H * hd)),)),
                Binding(p + "ffn_norm.weight",
                        (Source(p + "ffn_norm.weight", (D,), "norm"),), role="vector"),
                Binding(p + "feed_forward.w13",
                        (Source(p + "feed_forward.w1.weight", (I, D)),
                         Source(p + "feed_forward.w3.weight", (I, D))),
                        combine=torch.cat),
                Binding(p + "feed_forward.w2", (Source(p + "feed_forward.w2.weight", (D, I)),)),
            ]
        b.append(Binding("norm.weight", (Source("norm.weight", (D,), "norm"),), role="vector"))
        b.append(Binding("output.weight", (Source("output.weight", (V, D)),),
                         alias_of="tok_embeddings.weight" if c.tie_word_embeddings else None))
        # buffers of a run that a saved state dict may carry (model.py:87-89, 133-134)
        return CheckpointLayout(tuple(b), ignored=(r"\.kv_cache\.", r"^freqs_cis$",
                                                   r"^causal_mask$", r"^rope\.freqs$"))

    return (layout(True), layout(False))


def llama_sizes(c: LlamaConfig) -> dict:
    """Every size and constant of the configuration, flat, under the reference's names
    (model.py:21-34)."""
    rs = dict(c.rope_scaling) if c.rope_scaling else None
    scaling = "none" if not rs else " ".join(
        [str(rs.get("rope_type", rs.get("type", "")))] + [f"{k} {rs[k]:g}" for k in
         ("factor", "low_freq_factor", "high_freq_factor", "original_max_position_embeddings")
         if k in rs])
    return {"n_layer": c.num_hidden_layers, "dim": c.hidden_size, "n_head": c.num_attention_heads,
            "n_kv_heads": c.num_key_value_heads, "head_dim": c.head_dim,
            "intermediate_size": c.intermediate_size, "vocab_size": c.vocab_size,
            "rope_base": c.rope_theta, "rope_scaling": scaling, "norm_eps": c.rms_norm_eps}


LLAMA = register_architecture(Architecture(
    names=("LlamaForCausalLM", "llama"),
    read_config=LlamaConfig.from_dict,
    plan=llama_plan,
    bindings=llama_bindings,
    config_dict=LlamaConfig.to_dict,
    presets=LlamaConfig.from_name,
    other_layouts=llama_native_layouts,
    describe=llama_sizes,
))
