"""A whole architecture defined in the test and registered without a change to the library:
its own config.json keys, typed configuration, plan, checkpoint tensor names, a norm of its
own kind (centred, with a bias), layers that differ from one another (window, inner size),
a rotation of part of each head in the half-split layout, a tied and capped head.  A model
folder is written from a configuration and a seed, loaded by ``config.json`` through the
registry, and stepped and decoded against a plain computation written here.  It is a toy: it
stands for no model of anyone's.
"""
import dataclasses
import json
import math
import os

import pytest
import torch

import plain_llama as plain
import util
from util import TOL_BF16, TOL_F32, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

TOY = {"architectures": ["ToyStack"], "model_type": "toy_stack", "width": 96, "blocks": 3,
       "heads": 6, "kv_heads": 3, "head_size": 16, "inner": [136, 72, 136],
       "windows": [None, 40, None], "rotary": 8, "rope_base": 777.0, "vocab": 211, "eps": 1e-3,
       "tie": True, "cap": 20.0, "max_len": 512}


@dataclasses.dataclass(frozen=True)
class ToyConfig:
    width: int
    blocks: int
    heads: int
    kv_heads: int
    head_size: int
    inner: tuple
    windows: tuple
    rotary: int
    rope_base: float
    vocab: int
    eps: float
    tie: bool
    cap: float
    max_len: int

    @staticmethod
    def from_dict(d):
        names = [f.name for f in dataclasses.fields(ToyConfig)]
        missing = [n for n in names if n not in d]
        if missing:
            raise KeyError(f"toy_stack config.json lacks {missing}")
        c = ToyConfig(**{n: (tuple(d[n]) if isinstance(d[n], list) else d[n]) for n in names})
        if len(c.inner) != c.blocks or len(c.windows) != c.blocks or c.heads % c.kv_heads:
            raise ValueError("toy_stack: one inner size and one window per block; heads in groups")
        return c

    def to_dict(self):
        d = {k: (list(v) if isinstance(v, tuple) else v) for k, v in dataclasses.asdict(self).items()}
        return {"architectures": ["ToyStack"], "model_type": "toy_stack", **d}


@dataclasses.dataclass(frozen=True)
class CentredNormSpec:
    dim: int
    eps: float
    kind: str = "toy_centred"


def _register():
    """Registered once per process; the library's files are not touched."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.config.registry import Architecture, register_architecture
    from gpt_fast_amd.config.spec import (AttentionSpec, GatedFeedForwardSpec, LayerSpec,
                                          ModelPlan, PositionSpec, Run)
    from gpt_fast_amd.parts import Param, Part, register_norm
    from gpt_fast_amd.weights.bindings import Binding, CheckpointLayout, Source

    class CentredNorm(Part):
        """(x - mean) / sqrt(var + eps) * g + b, in float32, by library tensor operations: a
        toy norm needs no kernel of its own to be a part."""
        replayable = True

        def __init__(self, spec, rt):
            self.spec, self.rt = spec, rt

        def parameters(self):
            return {"g": Param((self.spec.dim,), role="vector", init="norm"),
                    "b": Param((self.spec.dim,), role="vector", init="linear")}

        def bind(self, tensors):
            self.g, self.b = tensors["g"].float(), tensors["b"].float()

        def forward(self, residual, rows=None):
            x = residual if rows is None else residual.index_select(0, rows.long())
            x = x - x.mean(-1, keepdim=True)
            y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.spec.eps) * self.g + self.b
            return y.to(self.rt.dtype)

    register_norm("toy_centred", CentredNorm)

    def plan(c):
        pos = PositionSpec(kind="rope", rotary_dim=c.rotary, base=c.rope_base, layout="half")
        layers = [LayerSpec(
            name=f"blk.{i}", arrangement="pre_norm",
            mixer=AttentionSpec(dim=c.width, n_heads=c.heads, n_kv_heads=c.kv_heads,
                                head_dim=c.head_size, position=pos, window=c.windows[i]),
            mixer_norm=CentredNormSpec(c.width, c.eps),
            feed_forward=GatedFeedForwardSpec(c.width, c.inner[i], "silu"),
            feed_forward_norm=CentredNormSpec(c.width, c.eps),
            mixer_name="att", mixer_norm_name="n1", feed_forward_name="ff",
            feed_forward_norm_name="n2") for i in range(c.blocks)]
        p = ModelPlan(dim=c.width, vocab_size=c.vocab, layers=layers,
                      order=[Run(i) for i in range(c.blocks)],
                      final_norm=CentredNormSpec(c.width, c.eps), tie_embeddings=c.tie,
                      max_positions=c.max_len, embedding_name="emb", final_norm_name="out_norm",
                      head_name="head", logit_softcap=c.cap)
        p.validate()
        return p

    def bindings(c):
        D, H, G, hd, V = c.width, c.heads, c.kv_heads, c.head_size, c.vocab
        b = [Binding("emb", (Source("table", (V, D)),))]
        for i in range(c.blocks):
            s, t = f"stack.{i}.", f"blk.{i}."
            for n in ("n1", "n2"):
                b += [Binding(t + n + ".g", (Source(s + n + "_gain", (D,), "norm"),), role="vector"),
                      Binding(t + n + ".b", (Source(s + n + "_bias", (D,)),), role="vector")]
            b += [Binding(t + "att.wqkv", (Source(s + "qkv", ((H + 2 * G) * hd, D)),)),
                  Binding(t + "att.wo", (Source(s + "merge", (D, H * hd)),)),
                  Binding(t + "ff.w13", (Source(s + "gate", (c.inner[i], D)), Source(s + "up", (c.inner[i], D))),
                          combine=torch.cat),
                  Binding(t + "ff.w2", (Source(s + "down", (D, c.inner[i])),))]
        b += [Binding("out_norm.g", (Source("final_gain", (D,), "norm"),), role="vector"),
              Binding("out_norm.b", (Source("final_bias", (D,)),), role="vector"),
              Binding("head", (Source("unembed", (V, D)),), alias_of="emb" if c.tie else None)]
        return CheckpointLayout(tuple(b))

    register_architecture(Architecture(
        names=("ToyStack", "toy_stack"), read_config=ToyConfig.from_dict, plan=plan,
        bindings=bindings, config_dict=ToyConfig.to_dict,
        describe=lambda c: {"blocks": c.blocks, "width": c.width}, layer_count_key="blocks"))
    return gfa


def _centred(x, g, b, eps):
    x = x - x.mean(-1, keepdim=True)
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * g + b


def _plain_logits(t, c, toks):
    """The toy model on a whole sequence, from the checkpoint's own tensor names."""
    S, H, G, hd, rot = len(toks), c.heads, c.kv_heads, c.head_size, c.rotary
    x = t["table"][torch.tensor(toks)]
    pos = torch.arange(S, dtype=torch.float32)
    freqs = 1.0 / (c.rope_base ** (torch.arange(0, rot, 2).float() / rot))
    ang = pos[:, None] * freqs[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def rotate(u):                                   # half-split pairs (i, i + rot / 2) of the first rot dims
        a, b = u[..., :rot // 2], u[..., rot // 2:rot]
        return torch.cat([a * cos - b * sin, b * cos + a * sin, u[..., rot:]], -1)

    for i in range(c.blocks):
        s = f"stack.{i}."
        xn = _centred(x, t[s + "n1_gain"], t[s + "n1_bias"], c.eps)
        q, k, v = (xn @ t[s + "qkv"].T).split([H * hd, G * hd, G * hd], -1)
        q, k, v = rotate(q.reshape(S, H, hd)), rotate(k.reshape(S, G, hd)), v.reshape(S, G, hd)
        dist = pos[:, None] - pos[None, :]
        keep = dist >= 0
        if c.windows[i] is not None:
            keep &= dist < c.windows[i]
        y = torch.empty(S, H, hd)
        for h in range(H):
            g = h // (H // G)
            sc = (q[:, h] @ k[:, g].T) / math.sqrt(hd)
            y[:, h] = torch.softmax(sc.masked_fill(~keep, float("-inf")), -1) @ v[:, g]
        x = x + y.reshape(S, H * hd) @ t[s + "merge"].T
        xn = _centred(x, t[s + "n2_gain"], t[s + "n2_bias"], c.eps)
        x = x + plain.feed_forward(xn, t[s + "gate"], t[s + "up"], t[s + "down"])
    xn = _centred(x, t["final_gain"], t["final_bias"], c.eps)
    logits = xn @ t["table"].T                       # the head is the embedding table
    return c.cap * torch.tanh(logits / c.cap)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_architecture_from_its_own_config_json_to_tokens(dtype, tmp_path):
    gfa = _register()
    from gpt_fast_amd import Entry
    from gpt_fast_amd.config.registry import read_model_folder
    from gpt_fast_amd.engine.generate import generate
    folder = str(tmp_path / "toy")
    arch = gfa.architecture("toy_stack")
    cfg = arch.read_config(TOY)
    gfa.write_random_model(folder, arch, cfg, seed=5, dtype=dtype, std=0.08)
    with open(os.path.join(folder, "config.json")) as f:
        assert json.load(f)["windows"] == [None, 40, None]
    found, read = read_model_folder(folder)                      # by config.json, as everywhere
    assert found is arch and read == cfg
    t = {k: v.float() for k, v in plain.read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    assert "unembed" not in t and "stack.1.up" in t              # tied head; its own names
    eng = gfa.Engine.from_folder(folder, dtype=dtype, device=DEV, max_tokens=1024)
    tol = TOL_F32 if dtype == "float32" else TOL_BF16
    toks = util.random_tokens(cfg.vocab, 90, 3)
    want = _plain_logits(t, cfg, toks)
    # whole; then cut into a chunk, single tokens beside another sequence, in used slots
    slot = eng.start_sequence()
    whole = eng.step([Entry(slot, toks, want=list(range(len(toks))))]).cpu()
    eng.end_sequence(slot)
    assert rel_err(whole, want) < tol
    a, b = eng.start_sequence(), eng.start_sequence()
    other = util.random_tokens(cfg.vocab, 60, 4)
    got = [eng.step([Entry(b, other[:37]), Entry(a, toks[:50], want=list(range(50)))]).cpu()]
    for i in range(50, 90):
        got.append(eng.step([Entry(b, [other[37 + (i - 50) % 23]]), Entry(a, [toks[i]], want=[0])]).cpu()[-1:])
    eng.end_sequence(a)
    eng.end_sequence(b)
    assert rel_err(torch.cat(got), want) < tol
    # generation through the entry point: greedy tokens are the plain model's where it is sure
    prompts = [toks[:20], other[:7]]
    out = generate(eng, prompts, max_new_tokens=8, temperature=0.0, stop_tokens=())
    for p, new in zip(prompts, out.tokens):
        logits = _plain_logits(t, cfg, p + new[:-1])[len(p) - 1:]
        for i, tok in enumerate(new):
            assert float(logits[i][tok]) >= float(logits[i].max()) - tol * float(logits[i].abs().max())
    eng.cache.check()
    assert eng.cache.slots.held == 0
    # a checkpoint that does not fit says so by this architecture's own names
    from gpt_fast_amd.weights.bindings import WeightsError
    from gpt_fast_amd.weights.safetensors_io import write_safetensors
    raw = plain.read_safetensors(os.path.join(folder, "model.safetensors"))
    raw.pop("stack.2.down")
    raw["stack.9.down"] = raw["stack.0.down"]
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    with open(os.path.join(bad, "config.json"), "w") as f:
        json.dump(arch.config_dict(cfg), f)
    write_safetensors(os.path.join(bad, "model.safetensors"), {k: torch.as_tensor(v) for k, v in raw.items()})
    with pytest.raises(WeightsError) as e:
        gfa.Engine.from_folder(bad, dtype=dtype, device=DEV, max_tokens=256)
    assert e.value.missing == ["stack.2.down"] and e.value.unexpected == ["stack.9.down"]


def test_the_toy_architecture_through_the_replay_program(tmp_path):
    """bin/trace_run knows the architecture through a plugin module named in the environment:
    a prompt, then single tokens, from the toy folder, against the plain computation."""
    import subprocess
    import numpy as np
    gfa = _register()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = str(tmp_path / "toy")
    arch = gfa.architecture("toy_stack")
    cfg = arch.read_config(TOY)
    gfa.write_random_model(folder, arch, cfg, seed=6, dtype="bfloat16", std=0.08)
    t = {k: v.float() for k, v in plain.read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    (tmp_path / "toy_plugin.py").write_text("import test_toy_architecture_gpu as T\nT._register()\n")
    toks = util.random_tokens(cfg.vocab, 45, 8)
    steps = [{"step": 0, "entries": [{"id": "r", "tokens": toks[:30], "want": list(range(30))}], "end": []}]
    steps += [{"step": i - 29, "entries": [{"id": "r", "tokens": [toks[i]], "want": [0]}],
               "end": ["r"] if i == 44 else []} for i in range(30, 45)]
    env = dict(os.environ, GPT_FAST_AMD_PLUGINS="toy_plugin",
               PYTHONPATH=os.pathsep.join([str(tmp_path), os.path.join(root, "tests"), root,
                                           os.environ.get("PYTHONPATH", "")]))
    want = _plain_logits(t, cfg, toks)
    for dtype, tol in (("float32", TOL_F32), ("bfloat16", TOL_BF16)):
        out = str(tmp_path / dtype)
        proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                               "--out", out, "--max-tokens", "64"],
                              input="\n".join(json.dumps(s) for s in steps) + "\n",
                              capture_output=True, text=True, timeout=110, env=env)
        assert proc.returncode == 0, proc.stderr[-2000:]
        got = torch.cat([torch.from_numpy(np.fromfile(os.path.join(out, f"{s['step']}.f32"), dtype="<f4")
                                          .reshape(-1, cfg.vocab).copy()) for s in steps])
        assert rel_err(got, want) < tol, dtype
