"""Parts defined in the tests, registered and stepped without a change to the library: a
feed-forward with routing and a position encoding that is no rotation.  They show that the
plan, the registries, the cache and the step function do not depend on the parts the
library ships; they are toys, not models of anything.

Each is compared with a plain computation written here from whole sequences (float32, CPU),
for a whole prompt, for the prompt cut into steps, and next to another sequence."""
import dataclasses
import math

import pytest
import torch

import plain_llama as plain
import util
from util import TOL_F32, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _random_parameters(model, seed):
    g = torch.Generator().manual_seed(seed)
    params = {}
    for name, p in model.parameters().items():
        t = torch.randn(p.shape, generator=g) * 0.08
        params[name] = 1 + t if p.init == "norm" else t
    return params


def _steps_equal_whole(eng, toks, want, vocab, tol):
    """Whole prompt; then prompt + single tokens beside another sequence in used slots."""
    from gpt_fast_amd import Entry
    n = len(toks)
    slot = eng.start_sequence()
    whole = eng.step([Entry(slot, toks, want=list(range(n)))]).cpu()
    eng.end_sequence(slot)
    assert rel_err(whole, want) < tol
    a, b = eng.start_sequence(), eng.start_sequence()
    other = util.random_tokens(vocab, 50, 77)
    cut = n // 2
    got = [eng.step([Entry(b, other[:30]), Entry(a, toks[:cut], want=list(range(cut)))]).cpu()]
    for i in range(cut, n):
        entries = [Entry(a, [toks[i]], want=[0])]
        if i - cut < 20:
            entries.insert(0, Entry(b, [other[30 + i - cut]]))
        got.append(eng.step(entries).cpu())
    eng.end_sequence(a)
    eng.end_sequence(b)
    assert rel_err(torch.cat(got), want) < tol


def _plain_attention_block(x, w, prefix, cfg, q_scale=None, k_scale=None, rotate=True,
                           kv_of=None):
    """x + wo(attention(norm(x))) from the plain parts; optional per-position scales on q, k.
    ``kv_of``: rows whose (normed, projected, rotated) keys and values are used instead of
    x's own - the input of an earlier run of this layer whose cache is borrowed."""
    S = x.shape[0]
    H, G, hd = cfg["n_head"], cfg["n_kv"], cfg["head_dim"]
    xn = plain.rms_norm(x, w[prefix + "attention_norm.weight"], cfg["eps"])
    qkv = xn @ w[prefix + "attention.wqkv"].T
    q, k, v = qkv.split([H * hd, G * hd, G * hd], dim=-1)
    q, k, v = q.reshape(S, H, hd), k.reshape(S, G, hd), v.reshape(S, G, hd)
    if kv_of is not None:
        other = plain.rms_norm(kv_of, w[prefix + "attention_norm.weight"], cfg["eps"])
        _, k, v = (other @ w[prefix + "attention.wqkv"].T).split([H * hd, G * hd, G * hd], dim=-1)
        k, v = k.reshape(S, G, hd), v.reshape(S, G, hd)
    if rotate:
        cos, sin = plain.rope_table(torch.arange(S), hd, cfg["rope_base"], cfg["rope_scaling"])
        q, k = plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin)
    if q_scale is not None:
        q, k = q * q_scale[:, None, None], k * k_scale[:, None, None]
    keep = torch.tril(torch.ones(S, S, dtype=torch.bool))
    y = torch.empty(S, H, hd)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) / math.sqrt(hd)
        y[:, h] = torch.softmax(s.masked_fill(~keep, float("-inf")), -1) @ v[:, g]
    return x + y.reshape(S, H * hd) @ w[prefix + "attention.wo"].T


def _plain_dense_ffn(x, w, prefix, cfg):
    xn = plain.rms_norm(x, w[prefix + "ffn_norm.weight"], cfg["eps"])
    w13 = w[prefix + "feed_forward.w13"]
    I = w13.shape[0] // 2
    return x + plain.feed_forward(xn, w13[:I], w13[I:], w[prefix + "feed_forward.w2"])


def test_toy_feed_forward_with_routing():
    """Each token goes to the expert with the largest router logit (of three gated
    feed-forwards) and the result is weighted by that expert's softmax probability."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.config.spec import LayerSpec, ModelPlan, Run
    from gpt_fast_amd.ops import linear as L
    from gpt_fast_amd.parts import Param, Part, Runtime, register_feed_forward
    from gpt_fast_amd.parts.model import DecoderModel

    @dataclasses.dataclass(frozen=True)
    class RoutedSpec:
        dim: int
        hidden: int
        experts: int
        kind: str = "toy_routed"

    class Routed(Part):
        def __init__(self, spec, rt):
            self.spec = spec

        def parameters(self):
            s = self.spec
            out = {"router": Param((s.experts, s.dim))}
            for e in range(s.experts):
                out[f"experts.{e}.w13"] = Param((2 * s.hidden, s.dim))
                out[f"experts.{e}.w2"] = Param((s.dim, s.hidden))
            return out

        def bind(self, tensors):
            self.t = tensors

        def forward(self, x, batch, residual):
            logits = L.linear(x, self.t["router"])                     # float32 engine
            prob = torch.softmax(logits.float(), -1)
            choice = prob.argmax(-1)
            for e in range(self.spec.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                h = L.gated_linear(x.index_select(0, rows).contiguous(), self.t[f"experts.{e}.w13"])
                y = L.linear(h, self.t[f"experts.{e}.w2"]).float() * prob[rows, e][:, None]
                residual.index_add_(0, rows, y)

    register_feed_forward("toy_routed", Routed)

    arch = gfa.architecture("llama")
    cfg = arch.read_config(util.TINY_B)
    base = arch.plan(cfg)
    D = cfg.hidden_size
    routed = dataclasses.replace(base.layers[1], feed_forward=RoutedSpec(D, 40, 3))
    plan = ModelPlan(dim=D, vocab_size=cfg.vocab_size, layers=[base.layers[0], routed],
                     order=[Run(0), Run(1)], final_norm=base.final_norm)
    model = DecoderModel(plan, Runtime(torch.float32, DEV))
    w = _random_parameters(model, 21)
    eng = gfa.Engine.from_plan(plan, {k: v.to(DEV) for k, v in w.items()}, "float32", DEV,
                               max_tokens=1024)
    pcfg = plain.config_from_dict(util.TINY_B)
    toks = util.random_tokens(cfg.vocab_size, 75, 5)

    x = w["tok_embeddings.weight"][torch.tensor(toks)]
    x = _plain_attention_block(x, w, "layers.0.", pcfg)
    x = _plain_dense_ffn(x, w, "layers.0.", pcfg)
    x = _plain_attention_block(x, w, "layers.1.", pcfg)
    xn = plain.rms_norm(x, w["layers.1.ffn_norm.weight"], pcfg["eps"])
    prob = torch.softmax(xn @ w["layers.1.feed_forward.router"].T, -1)
    choice = prob.argmax(-1)
    assert len(set(choice.tolist())) > 1                     # the routing routes
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        e = int(choice[t])
        w13 = w[f"layers.1.feed_forward.experts.{e}.w13"]
        y[t] = prob[t, e] * plain.feed_forward(xn[t:t + 1], w13[:40], w13[40:],
                                               w[f"layers.1.feed_forward.experts.{e}.w2"])[0]
    x = x + y
    want = plain.rms_norm(x, w["norm.weight"], pcfg["eps"]) @ w["output.weight"].T
    _steps_equal_whole(eng, toks, want, cfg.vocab_size, TOL_F32)


def test_toy_position_encoding_that_is_no_rotation():
    """Queries are scaled by gamma^-position and keys by gamma^position, so a score is
    damped by gamma^distance: only distances count, and nothing is rotated."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.config.spec import ModelPlan, Run
    from gpt_fast_amd.ops import kernels as K
    from gpt_fast_amd.parts import Part, Runtime, register_position
    from gpt_fast_amd.parts.model import DecoderModel

    @dataclasses.dataclass(frozen=True)
    class DecaySpec:
        gamma: float
        kind: str = "toy_decay"

    class Decay(Part):
        def __init__(self, spec, rt):
            self.spec = spec

        def rotate_and_store(self, qkv, batch, entry, n_heads, n_kv_heads, head_dim):
            n = qkv.shape[0]
            pos = batch.tok_pos[:n].float()
            up = torch.pow(torch.full_like(pos, self.spec.gamma), pos)[:, None]
            q_w, k_w = n_heads * head_dim, n_kv_heads * head_dim
            scaled = torch.cat([qkv[:, :q_w] / up, qkv[:, q_w:q_w + k_w] * up, qkv[:, q_w + k_w:]], 1)
            write = entry is not None and entry.writes
            return K.rope_cache_write(
                scaled.contiguous(), None, batch.tok_seq, batch.tok_pos, batch.table(entry.group_id),
                entry.k_pages if write else None, entry.v_pages if write else None,
                n_heads, n_kv_heads, head_dim, 0, 0)

    register_position("toy_decay", Decay)

    arch = gfa.architecture("llama")
    cfg = arch.read_config(util.TINY_A)
    base = arch.plan(cfg)
    gamma = 0.97
    layers = [dataclasses.replace(l, mixer=dataclasses.replace(l.mixer, position=DecaySpec(gamma)))
              if i == 0 else l for i, l in enumerate(base.layers)]
    plan = ModelPlan(dim=cfg.hidden_size, vocab_size=cfg.vocab_size, layers=layers,
                     order=[Run(i) for i in range(len(layers))], final_norm=base.final_norm)
    model = DecoderModel(plan, Runtime(torch.float32, DEV))
    w = _random_parameters(model, 22)
    eng = gfa.Engine.from_plan(plan, {k: v.to(DEV) for k, v in w.items()}, "float32", DEV,
                               max_tokens=1024)
    pcfg = plain.config_from_dict(util.TINY_A)
    toks = util.random_tokens(cfg.vocab_size, 130, 6)
    S = len(toks)
    x = w["tok_embeddings.weight"][torch.tensor(toks)]
    for i in range(len(layers)):
        p = f"layers.{i}."
        if i == 0:
            up = gamma ** torch.arange(S, dtype=torch.float32)
            x = _plain_attention_block(x, w, p, pcfg, q_scale=1 / up, k_scale=up, rotate=False)
        else:
            x = _plain_attention_block(x, w, p, pcfg)
        x = _plain_dense_ffn(x, w, p, pcfg)
    want = plain.rms_norm(x, w["norm.weight"], pcfg["eps"]) @ w["output.weight"].T
    _steps_equal_whole(eng, toks, want, cfg.vocab_size, TOL_F32)


def test_run_order_is_data_a_layer_twice_and_a_borrowed_cache():
    """order = layer 0, layer 1, layer 1 again (same weights, a cache entry of its own),
    layer 0 again reading the keys and values its first run wrote (and writing none):
    compared with the same computation from the plain parts over the whole sequence."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.config.spec import ModelPlan, Run
    from gpt_fast_amd.parts import Runtime
    from gpt_fast_amd.parts.model import DecoderModel

    arch = gfa.architecture("llama")
    cfg = arch.read_config(util.TINY_B)
    base = arch.plan(cfg)
    plan = ModelPlan(dim=cfg.hidden_size, vocab_size=cfg.vocab_size, layers=list(base.layers[:2]),
                     order=[Run(0), Run(1), Run(1), Run(0, cache_from=0)], final_norm=base.final_norm)
    model = DecoderModel(plan, Runtime(torch.float32, DEV))
    w = _random_parameters(model, 23)
    eng = gfa.Engine.from_plan(plan, {k: v.to(DEV) for k, v in w.items()}, "float32", DEV,
                               max_tokens=1024)
    pcfg = plain.config_from_dict(util.TINY_B)
    toks = util.random_tokens(cfg.vocab_size, 100, 8)
    x0 = w["tok_embeddings.weight"][torch.tensor(toks)]
    x = _plain_dense_ffn(_plain_attention_block(x0, w, "layers.0.", pcfg), w, "layers.0.", pcfg)
    for _ in range(2):
        x = _plain_dense_ffn(_plain_attention_block(x, w, "layers.1.", pcfg), w, "layers.1.", pcfg)
    x = _plain_attention_block(x, w, "layers.0.", pcfg, kv_of=x0)
    x = _plain_dense_ffn(x, w, "layers.0.", pcfg)
    want = plain.rms_norm(x, w["norm.weight"], pcfg["eps"]) @ w["output.weight"].T
    _steps_equal_whole(eng, toks, want, cfg.vocab_size, TOL_F32)
