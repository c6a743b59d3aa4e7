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


# --------------------------------------------------------------------------------------
# A mixer with fixed-size state of its own (no keys or values): a running mean of its
# inputs; state per sequence = [sum of inputs, count].  Two forms: one loops over the
# batch on the host (so its steps cannot be recorded), one works from the batch's device
# fields alone and says ``replayable``.
@dataclasses.dataclass(frozen=True)
class RunningMeanSpec:
    dim: int
    kind: str = "toy_running_mean"


def _running_mean_classes():
    from gpt_fast_amd.cache.store import StateNeed
    from gpt_fast_amd.parts import Param, Part

    class RunningMean(Part):
        def __init__(self, spec, rt):
            self.spec, self.rt = spec, rt

        def parameters(self):
            return {"mix": Param((self.spec.dim, self.spec.dim))}

        def bind(self, tensors):
            self.mix = tensors["mix"]

        def cache_need(self):
            return StateNeed((self.spec.dim + 1,), "float32")

        def forward(self, x, batch, entry, residual):
            state = entry.state                                   # [n_slots + 1, dim + 1]
            q_start = batch.host_field("q_start")
            slots = batch.host_field("slots")
            for b in range(batch.n_seqs):
                lo, hi = int(q_start[b]), int(q_start[b + 1])
                xs = x[lo:hi].float()
                s = state[int(slots[b])]
                sums = s[:-1] + torch.cumsum(xs, 0)
                counts = s[-1] + torch.arange(1, hi - lo + 1, device=x.device)
                residual[lo:hi] += (sums / counts[:, None]) @ self.mix.float().T
                s[:-1] = sums[-1]
                s[-1] = counts[-1]

    class RunningMeanOnDevice(RunningMean):
        """The same from device fields only: the same kernels whatever the batch holds."""
        replayable = True

        def forward(self, x, batch, entry, residual):
            state = entry.state
            n = x.shape[0]
            seq = batch.tok_seq.long()
            slot = batch.slots.long()[seq]                        # of every token
            idx = torch.arange(n, device=x.device)
            earlier = ((seq[:, None] == seq[None, :]) & (idx[:, None] >= idx[None, :])).float()
            old = state[slot]
            sums = earlier @ x.float() + old[:, :-1]
            counts = (earlier @ torch.ones(n, 1, device=x.device))[:, 0] + old[:, -1]
            residual += (sums / counts[:, None]) @ self.mix.float().T
            last = batch.q_start[1:].long() - 1                   # each sequence's last token
            state[batch.slots.long()] = torch.cat([sums[last], counts[last, None]], 1)

    return RunningMean, RunningMeanOnDevice


def _toy_state_model(on_device: bool):
    import gpt_fast_amd as gfa
    from gpt_fast_amd.config.spec import LayerSpec, ModelPlan, NormSpec, Run
    from gpt_fast_amd.parts import Runtime, register_mixer
    from gpt_fast_amd.parts.model import DecoderModel
    host_form, device_form = _running_mean_classes()
    register_mixer("toy_running_mean", device_form if on_device else host_form)
    arch = gfa.architecture("llama")
    cfg = arch.read_config(util.TINY_A)
    base = arch.plan(cfg)
    D = cfg.hidden_size
    toy_layer = LayerSpec(name="toy", mixer=RunningMeanSpec(D), mixer_norm=NormSpec(D, 1e-5),
                          feed_forward=base.layers[0].feed_forward,
                          feed_forward_norm=NormSpec(D, 1e-5))
    # attention, toy, attention, toy again (a state entry of its own), then the first layer
    # again with the first run's keys and values (borrowed)
    plan = ModelPlan(dim=D, vocab_size=cfg.vocab_size,
                     layers=[base.layers[0], toy_layer, base.layers[1]],
                     order=[Run(0), Run(1), Run(2), Run(1), Run(0, cache_from=0)],
                     final_norm=base.final_norm, max_positions=4096)
    model = DecoderModel(plan, Runtime(torch.float32, DEV))
    w = _random_parameters(model, 31)
    eng = gfa.Engine.from_plan(plan, {k: v.to(DEV) for k, v in w.items()}, "float32", DEV,
                               max_tokens=1024, max_sequences=6)
    return eng, w, plain.config_from_dict(util.TINY_A), cfg.vocab_size


def _plain_toy_state_logits(w, pcfg, toks):
    """The toy plan from whole sequences with the plain parts; the running mean is
    cumsum / count of the normed rows."""
    def toy_block(x):
        xn = plain.rms_norm(x, w["toy.mixer_norm.weight"], 1e-5)
        mean = torch.cumsum(xn, 0) / torch.arange(1, x.shape[0] + 1)[:, None]
        x = x + mean @ w["toy.mixer.mix"].T
        hn = plain.rms_norm(x, w["toy.feed_forward_norm.weight"], 1e-5)
        w13 = w["toy.feed_forward.w13"]
        I = w13.shape[0] // 2
        return x + plain.feed_forward(hn, w13[:I], w13[I:], w["toy.feed_forward.w2"])

    x0 = w["tok_embeddings.weight"][torch.tensor(toks)]
    x = _plain_dense_ffn(_plain_attention_block(x0, w, "layers.0.", pcfg), w, "layers.0.", pcfg)
    x = toy_block(x)
    x = _plain_dense_ffn(_plain_attention_block(x, w, "layers.1.", pcfg), w, "layers.1.", pcfg)
    x = toy_block(x)
    x = _plain_dense_ffn(_plain_attention_block(x, w, "layers.0.", pcfg, kv_of=x0), w, "layers.0.", pcfg)
    return plain.rms_norm(x, w["norm.weight"], pcfg["eps"]) @ w["output.weight"].T


@pytest.mark.parametrize("on_device", [False, True])
def test_toy_mixer_with_state_registers_and_steps(on_device):
    """A mixer defined here, with fixed-size state per sequence and no keys or values, is
    registered, built into a plan next to attention layers, and stepped: no file of the
    library changes.  Compared with the plain computation over the whole sequence: whole,
    cut into steps beside another sequence, in slots that were used before."""
    eng, w, pcfg, V = _toy_state_model(on_device)
    assert len(eng.cache.groups) == 2             # one KV group, one state group of two entries
    assert eng.model.replayable == on_device
    toks = util.random_tokens(V, 90, 3)
    want = _plain_toy_state_logits(w, pcfg, toks)
    _steps_equal_whole(eng, toks, want, V, TOL_F32)
    _steps_equal_whole(eng, toks, want, V, TOL_F32)          # again: slots and state reused
    assert eng.cache.slots.held == 0


@pytest.mark.parametrize("on_device", [False, True])
def test_toy_mixer_with_state_through_generate(on_device):
    """The same model through generate(): the decode session warms up before it records,
    which must not count a token twice into the state; rows that end at a stop token stay
    as fillers and must not write another sequence's state; the host-looping form is
    stepped without a recording although one is asked for.  Every token must be the best
    by the plain logits of the request's own sequence."""
    import gpt_fast_amd as gfa
    eng, w, pcfg, V = _toy_state_model(on_device)
    prompts = [util.random_tokens(V, n, 400 + n) for n in (5, 1, 17, 9)]
    free = gfa.generate(eng, prompts, max_new_tokens=14, temperature=0.0, use_graph=False).tokens
    stop = free[2][5]                              # request 2 ends after six tokens at the latest
    runs = {}
    for use_graph in (False, True):
        for _ in range(2):                         # the second time the recording is replayed
            res = gfa.generate(eng, prompts, max_new_tokens=14, temperature=0.0,
                               stop_tokens=[stop], use_graph=use_graph)
        runs[use_graph] = res.tokens
        assert eng.cache.slots.held == 0
    assert runs[True] == runs[False]
    assert len(runs[True][2]) <= 6 and runs[True][2][-1] == stop
    assert len(eng.recorded_steps) >= 1
    recorded = [s.graph is not None for s in eng.recorded_steps._steps.values()]
    assert any(recorded) == on_device
    for p, new in zip(prompts, runs[True]):
        logits = _plain_toy_state_logits(w, pcfg, p + new)
        for i, tok in enumerate(new):
            row = logits[len(p) - 1 + i]
            assert float(row[tok]) >= float(row.max()) - 1e-4 * float(row.abs().max()), (i, tok)


# --------------------------------------------------------------------------------------
# A mixer whose cache is of a kind of its own - a ring of its last SIZE inputs per sequence,
# registered from here with the class that stores it - and which asks for a field of its own
# in every step's description: the ring slot each token writes to.
@dataclasses.dataclass(frozen=True)
class RecentMeanSpec:
    dim: int
    size: int
    kind: str = "toy_recent_mean"


@dataclasses.dataclass(frozen=True)
class RingNeed:
    dim: int
    size: int


def _recent_mean_classes():
    from gpt_fast_amd.cache.store import Group, register_cache_need
    from gpt_fast_amd.engine.batch import StepField
    from gpt_fast_amd.parts import Param, Part

    class RingGroup(Group):
        """[entries, slots + 1, size + 1, dim]: the ring, and a row whose first element counts
        the inputs seen; the last slot belongs to no sequence."""

        def __init__(self, need, entries, geometry, dtype, device):
            self.need = need
            self.data = torch.zeros((entries, geometry.n_slots + 1, need.size + 1, need.dim),
                                    dtype=torch.float32, device=device)
            self.acquired = 0

        def acquire(self, slot):
            self.data[:, slot].zero_()
            self.acquired += 1

        def snapshot(self):
            saved = self.data.clone()
            return lambda: self.data.copy_(saved)

    register_cache_need(RingNeed, RingGroup)

    class RecentMean(Part):
        """residual += mix(mean of the last ``size`` normed inputs, this token's included)."""

        def __init__(self, spec, rt):
            self.spec = spec

        def parameters(self):
            return {"mix": Param((self.spec.dim, self.spec.dim))}

        def bind(self, tensors):
            self.mix = tensors["mix"]

        def cache_need(self):
            return RingNeed(self.spec.dim, self.spec.size)

        def step_fields(self):
            size = self.spec.size

            def fill(view, entries, starts, cache):
                n = 0
                for e, start in zip(entries, starts):
                    for i in range(len(e.tokens)):
                        view[n] = (start + i) % size
                        n += 1
            return [StepField("ring_slot", lambda n_tokens, n_seqs: n_tokens, fill)]

        def forward(self, x, batch, entry, residual):
            ring = entry.group.data[entry.index]                  # [slots + 1, size + 1, dim]
            q_start = batch.host_field("q_start")
            slots = batch.host_field("slots")
            ring_slot = batch.ring_slot.long()                    # the field, on the device
            for b in range(batch.n_seqs):
                r = ring[int(slots[b])]
                for n in range(int(q_start[b]), int(q_start[b + 1])):
                    r[ring_slot[n]] = x[n].float()
                    r[-1, 0] += 1
                    count = torch.clamp(r[-1, 0], max=self.spec.size)
                    residual[n] += (r[:-1].sum(0) / count) @ self.mix.float().T

    return RingGroup, RecentMean


def test_toy_mixer_with_a_cache_kind_and_a_step_field_of_its_own():
    """Neither the cache nor the step's description has to change for a mixer that needs
    another kind of storage and another per-step field: both are registered from here.
    Compared with the plain computation (a windowed mean over the whole sequence), whole and
    cut into steps beside another sequence, and through generate()."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.config.spec import LayerSpec, ModelPlan, NormSpec, Run
    from gpt_fast_amd.parts import Runtime, register_mixer
    from gpt_fast_amd.parts.model import DecoderModel
    RingGroup, RecentMean = _recent_mean_classes()
    register_mixer("toy_recent_mean", RecentMean)
    arch = gfa.architecture("llama")
    cfg = arch.read_config(util.TINY_A)
    base = arch.plan(cfg)
    D, SIZE = cfg.hidden_size, 5
    toy = LayerSpec(name="toy", mixer=RecentMeanSpec(D, SIZE), mixer_norm=NormSpec(D, 1e-5),
                    feed_forward=base.layers[0].feed_forward, feed_forward_norm=NormSpec(D, 1e-5))
    plan = ModelPlan(dim=D, vocab_size=cfg.vocab_size, layers=[base.layers[0], toy],
                     order=[Run(0), Run(1), Run(1)], final_norm=base.final_norm, max_positions=4096)
    model = DecoderModel(plan, Runtime(torch.float32, DEV))
    assert [f.name for f in model.step_fields()] == ["ring_slot"]      # asked for twice, kept once
    w = _random_parameters(model, 41)
    eng = gfa.Engine.from_plan(plan, {k: v.to(DEV) for k, v in w.items()}, "float32", DEV,
                               max_tokens=1024, max_sequences=4)
    ring_groups = [g for g in eng.cache.groups if isinstance(g, RingGroup)]
    assert len(ring_groups) == 1 and ring_groups[0].data.shape[:2] == (2, 5)   # two runs, 4 + 1 slots
    pcfg = plain.config_from_dict(util.TINY_A)

    def plain_logits(toks):
        def toy_block(x):
            xn = plain.rms_norm(x, w["toy.mixer_norm.weight"], 1e-5)
            mean = torch.stack([xn[max(0, t - SIZE + 1):t + 1].mean(0) for t in range(x.shape[0])])
            x = x + mean @ w["toy.mixer.mix"].T
            hn = plain.rms_norm(x, w["toy.feed_forward_norm.weight"], 1e-5)
            w13 = w["toy.feed_forward.w13"]
            I = w13.shape[0] // 2
            return x + plain.feed_forward(hn, w13[:I], w13[I:], w["toy.feed_forward.w2"])
        x = w["tok_embeddings.weight"][torch.tensor(toks)]
        x = _plain_dense_ffn(_plain_attention_block(x, w, "layers.0.", pcfg), w, "layers.0.", pcfg)
        x = toy_block(toy_block(x))
        return plain.rms_norm(x, w["norm.weight"], pcfg["eps"]) @ w["output.weight"].T

    V = cfg.vocab_size
    toks = util.random_tokens(V, 40, 9)
    want = plain_logits(toks)
    _steps_equal_whole(eng, toks, want, V, TOL_F32)
    _steps_equal_whole(eng, toks, want, V, TOL_F32)              # rings of used slots start empty
    prompts = [util.random_tokens(V, n, 500 + n) for n in (3, 11)]
    out = gfa.generate(eng, prompts, max_new_tokens=8, temperature=0.0).tokens
    for p, new in zip(prompts, out):
        logits = plain_logits(p + new)
        for i, tok in enumerate(new):
            row = logits[len(p) - 1 + i]
            assert float(row[tok]) >= float(row.max()) - 1e-4 * float(row.abs().max())
    assert eng.cache.slots.held == 0


def test_plan_level_steps_scale_position_and_cap():
    """What a plan may state around its layers, none of which Llama uses: a factor on the
    embedded rows, a position encoding added to them (a toy table of learned vectors,
    registered here), a factor and a soft cap on the logits."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.parts import Param, Part, register_position
    from gpt_fast_amd.parts import Runtime
    from gpt_fast_amd.parts.model import DecoderModel

    @dataclasses.dataclass(frozen=True)
    class LearnedTableSpec:
        dim: int
        positions: int
        kind: str = "toy_learned_table"

    class LearnedTable(Part):
        replayable = True

        def __init__(self, spec, rt):
            self.spec = spec

        def parameters(self):
            return {"table": Param((self.spec.positions, self.spec.dim))}

        def bind(self, tensors):
            self.table = tensors["table"]

        def add_to_stream(self, residual, batch):
            residual += self.table.float()[batch.tok_pos.long()]

    register_position("toy_learned_table", LearnedTable)
    arch = gfa.architecture("llama")
    cfg = arch.read_config(util.TINY_B)
    plan = arch.plan(cfg)
    plan.embedding_scale = 1.7
    plan.input_position = LearnedTableSpec(cfg.hidden_size, 200)
    plan.logit_scale = 3.0
    plan.logit_softcap = 2.5
    model = DecoderModel(plan, Runtime(torch.float32, DEV))
    w = _random_parameters(model, 41)
    assert "input_position.table" in w
    eng = gfa.Engine.from_plan(plan, {k: v.to(DEV) for k, v in w.items()}, "float32", DEV,
                               max_tokens=1024)
    pcfg = plain.config_from_dict(util.TINY_B)
    toks = util.random_tokens(cfg.vocab_size, 100, 12)
    x = w["tok_embeddings.weight"][torch.tensor(toks)] * 1.7 + w["input_position.table"][:100]
    for i in range(cfg.num_hidden_layers):
        x = _plain_dense_ffn(_plain_attention_block(x, w, f"layers.{i}.", pcfg), w, f"layers.{i}.", pcfg)
    logits = plain.rms_norm(x, w["norm.weight"], pcfg["eps"]) @ w["output.weight"].T
    want = 2.5 * torch.tanh(logits * 3.0 / 2.5)
    _steps_equal_whole(eng, toks, want, cfg.vocab_size, TOL_F32)
    # greedy generation through the recorded step agrees with stepping
    a = gfa.generate(eng, [toks[:10], toks[:3]], max_new_tokens=6, temperature=0.0).tokens
    b = gfa.generate(eng, [toks[:10], toks[:3]], max_new_tokens=6, temperature=0.0,
                     use_graph=False).tokens
    assert a == b
    # a position part without add_to_stream cannot stand there
    plan2 = arch.plan(cfg)
    plan2.input_position = plan2.layers[0].mixer.position
    with pytest.raises(TypeError, match="add_to_stream"):
        DecoderModel(plan2, Runtime(torch.float32, DEV))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_block_arrangement_of_its_own_reads_the_stream_and_keeps_the_fused_norms(dtype, monkeypatch):
    """A third arrangement, registered here: attention, then two gated feed-forwards, each
    behind a norm of its own.  Its ``forward`` reads the residual stream with
    ``stream.normed(norm, reader)`` and knows nothing else of how norms ride on the kernels
    that complete the stream - and still, in a few-row bfloat16 step, only the first norm of
    the step and the one before the head run as kernels of their own."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.config.spec import ModelPlan, Run
    from gpt_fast_amd.ops import kernels as KK
    from gpt_fast_amd.parts import Runtime, register_block
    from gpt_fast_amd.parts.base import FEED_FORWARDS, NORMS
    from gpt_fast_amd.parts.block import PreNormBlock
    from gpt_fast_amd.parts.model import DecoderModel

    class ThreeBranches(PreNormBlock):
        takes_stream = True

        def __init__(self, spec, rt):
            super().__init__(spec, rt)
            self.norm_b = NORMS.build(spec.feed_forward_norm, rt)
            self.feed_forward_b = FEED_FORWARDS.build(spec.feed_forward, rt)

        def children(self):
            return {**super().children(), "ffn_norm_b": self.norm_b, "feed_forward_b": self.feed_forward_b}

        def forward(self, stream, batch, entry):
            x = stream.normed(self.mixer_norm, reader=self.mixer)
            self.mixer.forward(x, batch, entry, stream)
            h = stream.normed(self.feed_forward_norm, reader=self.feed_forward)
            self.feed_forward.forward(h, batch, stream)
            g = stream.normed(self.norm_b, reader=self.feed_forward_b)
            self.feed_forward_b.forward(g, batch, stream)

    register_block("toy_three_branches", ThreeBranches)

    arch = gfa.architecture("llama")
    cfg = arch.read_config(util.TINY_A)
    base = arch.plan(cfg)
    layers = [dataclasses.replace(layer, arrangement="toy_three_branches") for layer in base.layers[:2]]
    plan = ModelPlan(dim=cfg.hidden_size, vocab_size=cfg.vocab_size, layers=layers,
                     order=[Run(0), Run(1)], final_norm=base.final_norm)
    compute = torch.float32 if dtype == "float32" else torch.bfloat16
    model = DecoderModel(plan, Runtime(compute, DEV))
    w = _random_parameters(model, 33)
    roles = {name: p.role for name, p in model.parameters().items()}
    w = {k: (v.to(compute).float() if roles[k] == "matrix" else v) for k, v in w.items()}   # as the engine holds them
    eng = gfa.Engine.from_plan(plan, {k: (v.to(compute) if roles[k] == "matrix" else v).to(DEV)
                                      for k, v in w.items()}, dtype, DEV, max_tokens=1024)
    pcfg = plain.config_from_dict(util.TINY_A)
    toks = util.random_tokens(cfg.vocab_size, 70, 9)

    x = w["tok_embeddings.weight"][torch.tensor(toks)]
    for n in range(2):
        p = f"layers.{n}."
        x = _plain_attention_block(x, w, p, pcfg)
        x = _plain_dense_ffn(x, w, p, pcfg)
        xn = plain.rms_norm(x, w[p + "ffn_norm_b.weight"], pcfg["eps"])
        w13 = w[p + "feed_forward_b.w13"]
        x = x + plain.feed_forward(xn, w13[:w13.shape[0] // 2], w13[w13.shape[0] // 2:], w[p + "feed_forward_b.w2"])
    want = plain.rms_norm(x, w["norm.weight"], pcfg["eps"]) @ w["output.weight"].T
    _steps_equal_whole(eng, toks, want, cfg.vocab_size, TOL_F32 if dtype == "float32" else util.TOL_BF16)

    if dtype == "bfloat16":
        from gpt_fast_amd import Entry
        calls = []
        real = KK.rmsnorm
        monkeypatch.setattr(KK, "rmsnorm", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
        slot = eng.start_sequence()
        eng.step([Entry(slot, toks[:40])])
        calls.clear()
        eng.step([Entry(slot, [toks[40]], want=[0])])
        eng.end_sequence(slot)
        assert len(calls) == 2, len(calls)     # of seven norms: the step's first and the head's
