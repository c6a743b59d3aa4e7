"""Generation through the entry points, trace replay as a program, parts alone, and a
toy mixer with state of its own that is registered from here."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as plain
import util
from util import TOL_BF16, TOL_F32, rel_err

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def engine_for(folder, dtype, **kw):
    import gpt_fast_amd as gfa
    kw.setdefault("max_tokens", 4096)
    return gfa.Engine.from_folder(folder, dtype=dtype, device="cuda:0", **kw)


@pytest.mark.parametrize("name,prompt_lens,new", [("A", [7, 3, 12], 8), ("B", [1, 5, 17, 33], 16)])
def test_greedy_generation_equals_plain(tmp_path_factory, name, prompt_lens, new):
    import gpt_fast_amd as gfa
    folder = util.make_folder(tmp_path_factory.getbasetemp(), name)
    cfg, w = plain.load_folder(folder)
    prompts = [util.random_tokens(cfg["vocab"], n, 40 + n) for n in prompt_lens]
    want = [plain.greedy_generate(w, cfg, p, new) for p in prompts]
    eng = engine_for(folder, "float32")
    res = gfa.generate(eng, prompts, max_new_tokens=new, temperature=0.0)
    assert res.tokens == want
    assert res.finish_reasons == ["length"] * len(prompts)
    assert eng.cache.slots.held == 0
    # one request alone gives the same tokens as in the batch; so do smaller batches
    alone = gfa.generate(eng, prompts[1:2], max_new_tokens=new, temperature=0.0)
    assert alone.tokens == want[1:2]
    two = gfa.generate(eng, prompts, max_new_tokens=new, temperature=0.0, batch_size=2)
    assert two.tokens == want
    # bfloat16: tokens agree wherever the float32 decision was not close
    eb = engine_for(folder, "bfloat16")
    got = gfa.generate(eb, prompts, max_new_tokens=new, temperature=0.0).tokens
    for p, g, wnt in zip(prompts, got, want):
        for i, (a, b) in enumerate(zip(g, wnt)):
            if a != b:
                logits = plain.forward(w, cfg, p + wnt[:i])[-1]
                top = torch.topk(logits, 2).values
                assert float(top[0] - top[1]) < 0.05 * float(logits.abs().max()), (i, a, b)
                break


def test_stop_tokens_end_only_their_sequence(tmp_path_factory):
    import gpt_fast_amd as gfa
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "A")
    cfg, w = plain.load_folder(folder)
    prompts = [util.random_tokens(cfg["vocab"], n, 70 + n) for n in (4, 9, 6)]
    free = [plain.greedy_generate(w, cfg, p, 10) for p in prompts]
    stop = free[1][3]                          # the 4th token of request 1 becomes a stop token
    want = [plain.greedy_generate(w, cfg, p, 10, stop_tokens=(stop,)) for p in prompts]
    assert len(want[1]) <= 4
    eng = engine_for(folder, "float32")
    res = gfa.generate(eng, prompts, max_new_tokens=10, temperature=0.0, stop_tokens=[stop])
    assert res.tokens == want
    assert res.finish_reasons[1] == "stop" and res.tokens[1][-1] == stop
    assert eng.cache.slots.held == 0


def test_sampled_generation_is_seeded_and_batch_independent(tmp_path_factory):
    import gpt_fast_amd as gfa
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    cfg = plain.read_config(folder)
    prompts = [util.random_tokens(cfg["vocab"], n, 90 + n) for n in (1, 5, 17, 33)]
    eng = engine_for(folder, "float32")
    kw = dict(max_new_tokens=16, temperature=0.8, top_k=50)
    a = gfa.generate(eng, prompts, seed=7, **kw).tokens
    b = gfa.generate(eng, prompts, seed=7, **kw).tokens
    c = gfa.generate(eng, prompts, seed=8, **kw).tokens
    assert a == b and a != c
    assert all(len(t) == 16 for t in a)
    # the same requests in batches of two draw the same tokens (noise is per request)
    d = gfa.generate(eng, prompts, seed=7, batch_size=2, **kw).tokens
    assert d == a
    # every token is the one the reference's law draws (generate.py:40-57) from the plain
    # logits of the request's own sequence with the sampler's stated noise: argmax(p / q),
    # p = softmax(top-50(logits / 0.8)).  A sampler that read another row's logits, another
    # position's or request's noise, or forgot the temperature would draw other tokens.
    _, w = plain.load_folder(folder)
    for key, (p, new) in enumerate(zip(prompts, a)):
        logits = plain.forward(w, cfg, p + new[:-1]).double()
        for j, tok in enumerate(new):
            pos = len(p) + j                               # the place of the token being drawn
            probs = plain.logits_to_probs(logits[pos - 1], temperature=0.8, top_k=50)
            assert int((probs > 0).sum()) == 50 and probs[tok] > 0
            race = probs / util.sampler_noise(cfg["vocab"], 7, key, pos)
            best = int(plain.sample_with_noise(probs, util.sampler_noise(cfg["vocab"], 7, key, pos)))
            # float32 logits and logf differ from these float64 ones in the last bits: on a
            # near tie of the race the other contender may win
            assert tok == best or float(race[tok]) > float(race[best]) * (1 - 1e-4), (key, j, tok, best)


def test_long_decoding_and_first_tokens(tmp_path_factory):
    """300 tokens decoded one by one from a one-token prompt: the first tokens of a
    sequence, page edges at 64, 128, 192, 256, and a long run, float32 and bfloat16."""
    from gpt_fast_amd import Entry
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    cfg, w = plain.load_folder(folder)
    tokens = util.random_tokens(cfg["vocab"], 300, 5)
    want = plain.forward(w, cfg, tokens)
    for dtype, tol in (("float32", TOL_F32), ("bfloat16", TOL_BF16)):
        eng = engine_for(folder, dtype)
        slot = eng.start_sequence()
        got = torch.cat([eng.step([Entry(slot, [t], want=[0])]).cpu() for t in tokens])
        eng.end_sequence(slot)
        assert rel_err(got[:4], want[:4]) < tol
        assert rel_err(got, want) < tol


def test_long_context(tmp_path_factory):
    """A prompt of 9000 tokens beside a short one, then tokens one by one: 141 pages per
    sequence, the prompt kernel's last tiles over thousands of keys, and single-token steps
    whose context is split over 32 workgroups per kv head, float32 and bfloat16."""
    from gpt_fast_amd import Entry
    util.TINY["B_long"] = dict(util.TINY_B, max_position_embeddings=16384)
    S, tail, new = 9000, 50, 24
    for dtype, tol in (("float32", TOL_F32), ("bfloat16", TOL_BF16)):
        folder = util.make_folder(tmp_path_factory.getbasetemp(), "B_long", seed=3, dtype=dtype)
        cfg, w = plain.load_folder(folder)
        tokens = util.random_tokens(cfg["vocab"], S + new, 9)
        other = util.random_tokens(cfg["vocab"], 300, 10)
        want = plain.forward(w, cfg, tokens)[S - tail:]
        eng = engine_for(folder, dtype, max_tokens=64 * 160 * 2)
        a, b = eng.start_sequence(), eng.start_sequence()
        got = [eng.step([Entry(b, other[:200]),
                         Entry(a, tokens[:S], want=list(range(S - tail, S)))]).cpu()]
        for t in range(new):
            entries = [Entry(a, [tokens[S + t]], want=[0])]
            if t < 10:
                entries.insert(0, Entry(b, [other[200 + t]]))
            got.append(eng.step(entries).cpu())
        got = torch.cat(got)
        assert rel_err(got[:tail], want[:tail]) < tol
        assert rel_err(got[tail:], want[tail:]) < tol


def test_decode_session_with_graph_equals_stepping(tmp_path_factory):
    from gpt_fast_amd import Entry
    from gpt_fast_amd.engine.decode import DecodeSession
    from gpt_fast_amd.sampling import SamplingParams
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    cfg, w = plain.load_folder(folder)
    prompts = [util.random_tokens(cfg["vocab"], n, 20 + n) for n in (60, 3, 64)]
    want = [plain.greedy_generate(w, cfg, p, 12) for p in prompts]
    for use_graph in (False, True):
        eng = engine_for(folder, "float32")
        slots = [eng.start_sequence() for _ in prompts]
        logits = eng.step([Entry(s, p, want=[len(p) - 1]) for s, p in zip(slots, prompts)])
        first = logits.argmax(-1).to(torch.int32)
        sess = DecodeSession(eng, slots, [0, 1, 2], first, SamplingParams(temperature=0.0),
                             use_graph=use_graph, max_new_tokens=12)
        got = [first.cpu()]
        for _ in range(11):
            got.append(sess.advance().cpu().clone())       # crosses a page edge at 64
            torch.cuda.synchronize()
        got = torch.stack(got, 1).tolist()
        assert got == want, use_graph
        for s in slots:
            eng.end_sequence(s)


def _replay(folder, dtype, steps, out, max_tokens):
    lines = "\n".join(json.dumps(s) for s in steps) + "\n"
    env = dict(os.environ)
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", out, "--max-tokens", str(max_tokens)],
                          input=lines, capture_output=True, text=True, timeout=110, env=env)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == \
        [f"done {s['step']}" for s in steps]


def test_trace_run_program(tmp_path_factory, tmp_path):
    """bin/trace_run on a trace of two batches of unequal requests; the second batch reuses
    what the first gave back; max-tokens is exactly what the live requests hold."""
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "C")
    cfg, w = plain.load_folder(folder)
    V = cfg["vocab"]
    reqs = {"a": util.random_tokens(V, 70, 1), "b": util.random_tokens(V, 5, 2),
            "c": util.random_tokens(V, 130, 3), "d": util.random_tokens(V, 64, 4)}
    prompt = {"a": 66, "b": 2, "c": 128, "d": 60}
    steps = []
    where = {}                                  # request -> list of (step, first row, count)

    def batch(ids, n0):
        n = n0
        live = list(ids)
        steps.append({"step": n, "entries": [
            {"id": r, "tokens": reqs[r][:prompt[r]], "want": list(range(prompt[r]))} for r in live],
            "end": []})
        at = 0
        for r in live:
            where.setdefault(r, []).append((n, at, prompt[r]))
            at += prompt[r]
        t = 0
        while live:
            n += 1
            ending = [r for r in live if prompt[r] + t + 1 >= len(reqs[r])]
            steps.append({"step": n, "entries": [
                {"id": r, "tokens": [reqs[r][prompt[r] + t]], "want": [0]} for r in live],
                "end": ending})
            for row, r in enumerate(live):
                where[r].append((n, row, 1))
            live = [r for r in live if r not in ending]
            t += 1
        return n + 1

    n = batch(["a", "b"], 0)
    batch(["c", "d"], n)
    most = max(128 + 64, 192 + 64)              # a+b: 128+64; c+d: 192+64 tokens in pages
    for dtype, tol in (("float32", TOL_F32), ("bfloat16", TOL_BF16)):
        out = str(tmp_path / dtype)
        _replay(folder, dtype, steps, out, most)
        for r, toks in reqs.items():
            rows = []
            for step, row, count in where[r]:
                data = np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, V)
                rows.append(torch.from_numpy(data[row:row + count].copy()))
            got = torch.cat(rows)
            assert got.shape[0] == len(toks)
            assert rel_err(got, plain.forward(w, cfg, toks)) < tol, (dtype, r)


def test_parts_alone(tmp_path_factory):
    """Each part of a layer on its own against the plain function of the same part."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd import Entry
    from gpt_fast_amd.config.spec import GatedFeedForwardSpec, NormSpec
    from gpt_fast_amd.parts import FEED_FORWARDS, MIXERS, NORMS, Runtime
    from gpt_fast_amd.cache.store import Cache
    from gpt_fast_amd.engine.batch import BatchUploader
    rt = Runtime(torch.float32, "cuda:0")
    torch.manual_seed(0)
    D = 72
    x = torch.randn(9, D, device="cuda:0")
    # norm
    norm = NORMS.build(NormSpec(D, 1e-4), rt)
    wn = torch.randn(D, device="cuda:0")
    norm.bind({"weight": wn})
    assert rel_err(norm.forward(x), plain.rms_norm(x.cpu(), wn.cpu(), 1e-4)) < 1e-6
    # feed-forward adds into the residual stream
    ff = FEED_FORWARDS.build(GatedFeedForwardSpec(D, 104), rt)
    w13, w2 = torch.randn(208, D, device="cuda:0") * 0.1, torch.randn(D, 104, device="cuda:0") * 0.1
    ff.bind({"w13": w13, "w2": w2})
    res = torch.ones(9, D, device="cuda:0")
    ff.forward(x, None, res)
    want = 1 + plain.feed_forward(x.cpu(), w13[:104].cpu(), w13[104:].cpu(), w2.cpu())
    assert rel_err(res, want) < 1e-5
    # attention mixer over its own cache entry, prompt then one token
    arch = gfa.architecture("llama")
    plan = arch.plan(arch.read_config(util.TINY_B))
    spec = plan.layers[0].mixer
    att = MIXERS.build(spec, rt)
    Dm = spec.dim
    wqkv = torch.randn((spec.n_heads + 2 * spec.n_kv_heads) * spec.head_dim, Dm, device="cuda:0") * 0.1
    wo = torch.randn(Dm, spec.n_heads * spec.head_dim, device="cuda:0") * 0.1
    att.bind({"wqkv": wqkv, "wo": wo})
    cache = Cache([att.cache_need()], [None], max_tokens=128, max_sequences=2,
                  dtype=torch.float32, device="cuda:0")
    up = BatchUploader("cuda:0")
    xs = torch.randn(70, Dm, device="cuda:0")
    slot = cache.acquire()
    res = torch.zeros(70, Dm, device="cuda:0")
    starts = cache.extend_many([(slot, 69)])
    att.forward(xs[:69].contiguous(), up.build([Entry(slot, [0] * 69)], starts, cache),
                cache.entries[0], res[:69])
    starts = cache.extend_many([(slot, 1)])
    att.forward(xs[69:].contiguous(), up.build([Entry(slot, [0])], starts, cache),
                cache.entries[0], res[69:])
    pcfg = plain.config_from_dict(util.TINY_B)
    want = plain.attention(xs.cpu(), wqkv.cpu(), wo.cpu(), pcfg, torch.arange(70))
    assert rel_err(res, want) < 1e-5


@pytest.mark.parametrize("n_seqs", [5, 24, 40])
def test_graph_replays_equal_eager_steps_for_any_batch_size(tmp_path_factory, n_seqs):
    """The captured step is replayed many times with eager work and synchronisations in
    between; every replay must give the tokens of the uncaptured step.  24 rows go through
    the few-row kernels with two tiles of rows, 40 through the vendor library's products
    inside the graph."""
    from gpt_fast_amd import Entry
    from gpt_fast_amd.engine.decode import DecodeSession
    from gpt_fast_amd.sampling import SamplingParams
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    cfg = plain.read_config(folder)
    prompts = [util.random_tokens(cfg["vocab"], 1 + (7 * i) % 50, 300 + i) for i in range(n_seqs)]
    runs = {}
    for use_graph in (False, True):
        eng = engine_for(folder, "bfloat16", max_tokens=64 * 2 * n_seqs)
        slots = [eng.start_sequence() for _ in prompts]
        logits = eng.step([Entry(s, p, want=[len(p) - 1]) for s, p in zip(slots, prompts)])
        first = logits.argmax(-1).to(torch.int32)
        sess = DecodeSession(eng, slots, list(range(n_seqs)), first,
                             SamplingParams(temperature=0.7, top_k=20, seed=3),
                             use_graph=use_graph, max_new_tokens=24)
        got = []
        for step in range(20):
            got.append(sess.collect(sess.launch()))
            if step % 3 == 0:                       # eager work between replays
                torch.cuda.synchronize()
                _ = (torch.ones(1000, device="cuda:0") * 2).sum().item()
        runs[use_graph] = got
        for s in slots:
            eng.end_sequence(s)
    assert runs[True] == runs[False]


def _plain_forward_with_windows(w, cfg, tokens, windows):
    """The plain model with a window per layer (None: all keys): the causal mask of
    model.py:134 with keys at distance >= window masked as well."""
    import math
    idx = torch.as_tensor(tokens, dtype=torch.long)
    S = idx.numel()
    pos = torch.arange(S)
    x = w["tok_embeddings.weight"][idx]
    H, G, hd = cfg["n_head"], cfg["n_kv"], cfg["head_dim"]
    for i, win in enumerate(windows):
        p = f"layers.{i}."
        xn = plain.rms_norm(x, w[p + "attention_norm.weight"], cfg["eps"])
        qkv = xn @ w[p + "attention.wqkv.weight"].T
        q, k, v = qkv.split([H * hd, G * hd, G * hd], dim=-1)
        cos, sin = plain.rope_table(pos, hd, cfg["rope_base"], cfg["rope_scaling"])
        q = plain.apply_rope(q.reshape(S, H, hd), cos, sin)
        k = plain.apply_rope(k.reshape(S, G, hd), cos, sin)
        v = v.reshape(S, G, hd)
        keep = torch.tril(torch.ones(S, S, dtype=torch.bool))
        if win is not None:
            keep &= (pos[:, None] - pos[None, :]) < win
        y = torch.empty(S, H, hd)
        for h in range(H):
            g = h // (H // G)
            s = (q[:, h] @ k[:, g].T) / math.sqrt(hd)
            y[:, h] = torch.softmax(s.masked_fill(~keep, float("-inf")), -1) @ v[:, g]
        x = x + y.reshape(S, H * hd) @ w[p + "attention.wo.weight"].T
        x = x + plain.feed_forward(plain.rms_norm(x, w[p + "ffn_norm.weight"], cfg["eps"]),
                                   w[p + "feed_forward.w1.weight"], w[p + "feed_forward.w3.weight"],
                                   w[p + "feed_forward.w2.weight"])
    return plain.rms_norm(x, w["norm.weight"], cfg["eps"]) @ w["output.weight"].T


@pytest.mark.parametrize("dtype,tol", [("float32", TOL_F32), ("bfloat16", TOL_BF16)])
def test_layers_with_windows_have_storage_of_their_own(tmp_path_factory, dtype, tol):
    """A plan (made here, not an architecture of the library) whose layers differ: full
    attention, a window of 70 keys, a window of 20.  Each need gets its own cache group;
    the windowed groups give pages back while the sequence grows; logits equal the plain
    model with the same windows, whole, cut into steps, and next to another sequence."""
    import dataclasses
    import gpt_fast_amd as gfa
    from gpt_fast_amd import Entry
    from gpt_fast_amd.weights.bindings import load_parameters
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    arch, cfg = gfa.read_model_folder(folder)
    plan = arch.plan(cfg)
    windows = [None, 70, 20]
    plan.layers = [dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, window=win))
                   for layer, win in zip(plan.layers, windows)]
    params = load_parameters(folder, arch.bindings(cfg), dtype, torch.device("cuda:0"))
    eng = gfa.Engine.from_plan(plan, params, dtype, "cuda:0", max_tokens=64 * 12)
    assert len(eng.cache.kv_groups) == 3
    pcfg, w = plain.load_folder(folder)
    toks = util.random_tokens(pcfg["vocab"], 300, 9)
    want = _plain_forward_with_windows(w, pcfg, toks, windows)
    slot = eng.start_sequence()
    whole = eng.step([Entry(slot, toks, want=list(range(300)))]).cpu()
    assert rel_err(whole, want) < tol
    held = [g.pages.held for _, g in eng.cache.kv_groups]
    assert held == [5, 5, 5]                      # a whole prompt needs every page while it runs
    eng.end_sequence(slot)
    # prompt, then token by token, beside a second sequence: windowed groups let pages go
    a, b = eng.start_sequence(), eng.start_sequence()
    other = util.random_tokens(pcfg["vocab"], 80, 10)
    got = [eng.step([Entry(a, toks[:150], want=list(range(150))), Entry(b, other[:40])]).cpu()]
    for i in range(150, 300):
        entries = [Entry(a, [toks[i]], want=[0])]
        if i < 190:
            entries.append(Entry(b, [other[i - 110]]))
        got.append(eng.step(entries).cpu())
    assert rel_err(torch.cat(got), want) < tol
    held = {g.need.window: len([p for p in eng.cache.page_list(gid, a) if p >= 0])
            for gid, g in eng.cache.kv_groups}
    assert held[None] == 5 and held[70] == 2 and held[20] == 1
    eng.cache.check()
    eng.end_sequence(a)
    eng.end_sequence(b)
    assert all(g.pages.held == 0 for _, g in eng.cache.kv_groups)


def test_trace_run_chunks_and_a_mixed_step(tmp_path_factory, tmp_path):
    """bin/trace_run on steps the generation loop never makes: a request fed as chunks of 37,
    29, 1 and 33 tokens, and one step that holds single tokens, a 40-token chunk at position
    70 and a fresh 130-token prompt.  float32 logits are bit-equal to the whole sequences'."""
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    cfg, w = plain.load_folder(folder)
    V = cfg["vocab"]
    seqs, before, mixed = util.mixed_step_case(V)
    seqs["k"] = util.random_tokens(V, 100, 21)
    steps, where = [], {r: [] for r in seqs}

    def add(parts, end=()):
        n = len(steps)
        at = 0
        entries = []
        for r, lo, count in parts:
            entries.append({"id": r, "tokens": seqs[r][lo:lo + count], "want": list(range(count))})
            where[r].append((n, at, count))
            at += count
        steps.append({"step": n, "entries": entries, "end": list(end)})

    at = 0
    for n in (37, 29, 1, 33):
        add([("k", at, n)], end=["k"] if at + n == 100 else [])
        at += n
    add([(r, 0, before[r]) for r in ("d0", "d1", "d2", "c")])
    add([(r, before.get(r, 0), mixed[r]) for r in ("d0", "c", "d1", "p", "d2")],
        end=["d0", "d1", "d2"])
    add([("c", 110, 1), ("p", 130, 1)], end=["p"])
    add([("c", 111, 1)], end=["c"])
    most = 64 + 128 + 192 + 128 + 192           # d0, d1, d2, c, p live together, in pages
    for dtype, tol in (("float32", TOL_F32), ("bfloat16", TOL_BF16)):
        out = str(tmp_path / dtype)
        _replay(folder, dtype, steps, out, most)
        eng = engine_for(folder, dtype) if dtype == "float32" else None
        for r, toks in seqs.items():
            rows = []
            for step, row, count in where[r]:
                data = np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, V)
                rows.append(torch.from_numpy(data[row:row + count].copy()))
            got = torch.cat(rows)
            assert rel_err(got, plain.forward(w, cfg, toks)) < tol, (dtype, r)
            if eng is not None:
                from gpt_fast_amd import Entry
                slot = eng.start_sequence()
                whole = eng.step([Entry(slot, toks, want=list(range(len(toks))))]).cpu()
                eng.end_sequence(slot)
                assert torch.equal(got, whole), r


@pytest.mark.parametrize("batch,total", [(20, 24), (28, 32)])
def test_generation_in_bfloat16_with_rows_that_retire_mid_session(tmp_path_factory, batch, total):
    """Requests in a batch of 20 (28) and one of 4, bfloat16, a stop token that ends several
    requests at different steps: the recorded step is replayed with filler rows in place of
    the ended requests, over more than sixteen rows (20: the few-row kernels with two tiles of
    rows; 28: the vendor library's products inside the recording).  The tokens equal those of
    the same run without a recording."""
    import gpt_fast_amd as gfa
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    cfg = plain.read_config(folder)
    prompts = [util.random_tokens(cfg["vocab"], 1 + (5 * i) % 31, 500 + i) for i in range(total)]
    eng = engine_for(folder, "bfloat16", max_tokens=64 * batch)
    free = gfa.generate(eng, prompts, max_new_tokens=24, temperature=0.0, batch_size=batch,
                        use_graph=False).tokens
    # a token that some requests draw early and others late or never
    counts = {}
    for t in free:
        for tok in set(t[2:20]):
            counts[tok] = counts.get(tok, 0) + 1
    stop = max(counts, key=lambda k: (min(counts[k], total - counts[k]), k))
    runs = {}
    for use_graph in (False, True):
        res = gfa.generate(eng, prompts, max_new_tokens=24, temperature=0.0, batch_size=batch,
                           stop_tokens=[stop], use_graph=use_graph)
        runs[use_graph] = res
        assert eng.cache.slots.held == 0
        eng.cache.check()
    assert runs[True].tokens == runs[False].tokens
    assert runs[True].finish_reasons == runs[False].finish_reasons
    ended = [i for i, r in enumerate(runs[True].finish_reasons) if r == "stop"]
    assert 2 <= len(ended) < total
    assert len({len(runs[True].tokens[i]) for i in ended}) > 1      # at different steps
    for i in ended:
        assert runs[True].tokens[i][-1] == stop and stop not in runs[True].tokens[i][:-1]
    # sampled, with a seed: also the same with and without the recording
    kw = dict(max_new_tokens=12, temperature=0.9, top_k=30, batch_size=batch, stop_tokens=[stop])
    a = gfa.generate(eng, prompts, seed=5, use_graph=True, **kw).tokens
    b = gfa.generate(eng, prompts, seed=5, use_graph=False, **kw).tokens
    c = gfa.generate(eng, prompts, seed=6, use_graph=True, **kw).tokens
    assert a == b and a != c


def test_the_recorded_step_is_kept_across_calls(tmp_path_factory):
    """generate() records the one-token step once per shape and sampling law; later calls
    of that shape replay it (the reference compiles its decode step once for all samples,
    generate.py:338-345), also for another seed, which lives in the step's buffer."""
    import gpt_fast_amd as gfa
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "A")
    cfg, w = plain.load_folder(folder)
    prompts = [util.random_tokens(cfg["vocab"], n, 60 + n) for n in (7, 3, 12)]
    eng = engine_for(folder, "float32")
    want = [plain.greedy_generate(w, cfg, p, 8) for p in prompts]
    assert gfa.generate(eng, prompts, max_new_tokens=8, temperature=0.0).tokens == want
    assert len(eng.recorded_steps) == 1
    first = next(iter(eng.recorded_steps._steps.values()))
    graph = first.graph
    assert graph is not None and not first.busy
    # other prompts of the same lengths: the same recording, right tokens
    prompts2 = [util.random_tokens(cfg["vocab"], n, 80 + n) for n in (7, 3, 12)]
    want2 = [plain.greedy_generate(w, cfg, p, 8) for p in prompts2]
    assert gfa.generate(eng, prompts2, max_new_tokens=8, temperature=0.0).tokens == want2
    assert len(eng.recorded_steps) == 1 and first.graph is graph
    # sampling is another law (one more recording); seeds share it
    kw = dict(max_new_tokens=8, temperature=0.8, top_k=50)
    a = gfa.generate(eng, prompts, seed=1, **kw).tokens
    b = gfa.generate(eng, prompts, seed=2, **kw).tokens
    assert len(eng.recorded_steps) == 2
    assert a != b
    assert a == gfa.generate(eng, prompts, seed=1, use_graph=False, **kw).tokens
    assert b == gfa.generate(eng, prompts, seed=2, use_graph=False, **kw).tokens
    # two sessions of one shape open at once do not share buffers
    from gpt_fast_amd.engine.decode import DecodeSession
    from gpt_fast_amd.sampling import SamplingParams
    slots = [eng.start_sequence() for _ in range(2)]
    from gpt_fast_amd import Entry
    eng.step([Entry(s, [1, 2, 3]) for s in slots])
    tok = torch.tensor([4], dtype=torch.int32, device="cuda:0")
    s1 = DecodeSession(eng, slots[:1], [0], tok, SamplingParams(temperature=0.0), max_new_tokens=4)
    s2 = DecodeSession(eng, slots[1:], [1], tok, SamplingParams(temperature=0.0), max_new_tokens=4)
    assert s1.rec is not s2.rec
    t1, t2 = s1.collect(s1.launch()), s2.collect(s2.launch())
    assert t1 == t2                                  # equal sequences, equal tokens
    s1.close(), s2.close()
    for s in slots:
        eng.end_sequence(s)


def test_generate_checks_room_before_it_runs(tmp_path_factory):
    import gpt_fast_amd as gfa
    from gpt_fast_amd.cache.slots import CacheFull
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")           # 128 positions
    eng = engine_for(folder, "float32", max_tokens=64 * 3, max_sequences=3)
    with pytest.raises(ValueError, match="128 positions"):
        gfa.generate(eng, [[1] * 100], max_new_tokens=29, temperature=0.0)
    with pytest.raises(CacheFull):                   # 65 + 64 + 1 tokens: four pages
        gfa.generate(eng, [[1] * 60, [2] * 60, [3]], max_new_tokens=6, temperature=0.0)
    with pytest.raises(CacheFull):                   # four sequences, three slots
        gfa.generate(eng, [[1], [2], [3], [4]], max_new_tokens=2, temperature=0.0)
    assert eng.cache.slots.held == 0
    # the same requests in batches that fit
    out = gfa.generate(eng, [[1], [2], [3], [4]], max_new_tokens=2, temperature=0.0, batch_size=2)
    assert [len(t) for t in out.tokens] == [2, 2, 2, 2]


# --------------------------------------------------------------------------------------
# the command line, as a program (reference generate.py:272-437, 440-470)
def _cli(*args, timeout=110):
    proc = subprocess.run([sys.executable, "-m", "gpt_fast_amd", *map(str, args)], cwd=ROOT,
                          capture_output=True, text=True, timeout=timeout)
    return proc


def test_command_line_generates_the_plain_tokens(tmp_path_factory):
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    cfg, w = plain.load_folder(folder)
    prompt = util.random_tokens(cfg["vocab"], 9, 44)
    want = plain.greedy_generate(w, cfg, prompt, 8)
    proc = _cli("--checkpoint_path", folder, "--prompt_ids", ",".join(map(str, prompt)),
                "--temperature", 0, "--num_samples", 2, "--max_new_tokens", 8, "--dtype", "float32")
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.splitlines()
    shown = [l for l in lines if l.strip() and all(p.isdigit() for p in l.split())]
    assert len(shown) == 2                            # one line of ids per sample
    for l in shown:
        assert [int(t) for t in l.split()] == prompt + want
    for needle in ("Time for inference 1:", "Time for inference 2:", "Bandwidth achieved:",
                   "FLOPS achieved:", "Batch Size: 1", "Prompt Length: 9", "Generated tokens: 8",
                   "Average tokens/sec:", "Memory used:"):
        assert any(needle in l for l in lines), needle


def test_command_line_random_weights_and_a_batch(tmp_path):
    proc = _cli("--random", "tiny-llama-b", "--prompt", 5, "--batch_size", 3, "--num_samples", 2,
                "--max_new_tokens", 6, "--top_k", 40)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = proc.stdout
    assert "Only displaying the first generation of the batch" in out
    assert "Batch Size: 3" in out and "Prompt Length: 5" in out
    shown = [l for l in out.splitlines() if l.strip() and all(p.isdigit() for p in l.split())]
    assert len(shown) == 2 and all(len(l.split()) == 11 for l in shown)
    # the preset may also be a config.json file; the architecture comes from the file
    import json as _json
    path = tmp_path / "config.json"
    path.write_text(_json.dumps(util.TINY_C))
    proc = _cli("--random", path, "--prompt", 4, "--num_samples", 1, "--max_new_tokens", 3,
                "--dtype", "float32")
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Prompt Length: 4" in proc.stdout


def test_command_line_profile_writes_a_trace_of_the_last_sample(tmp_path):
    """--profile PATH (generate.py:380-385, 403-407): the last sample runs under the profiler
    and its trace is written to PATH.json; the trace names kernels of this library."""
    import json as _json
    trace = tmp_path / "trace"
    proc = _cli("--random", "tiny-llama-a", "--prompt", 6, "--num_samples", 2, "--max_new_tokens", 4,
                "--temperature", 0, "--profile", trace, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    path = tmp_path / "trace.json"
    assert path.is_file() and path.stat().st_size > 1000
    events = _json.loads(path.read_text())["traceEvents"]
    names = {e.get("name", "") for e in events}
    assert any("kernel" in n and ("skinny" in n or "attention" in n or "rmsnorm" in n or "embed" in n)
               for n in names), sorted(names)[:40]


def test_command_line_refusals(tmp_path_factory):
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "A")
    for args, needle in (
            (["--checkpoint_path", folder, "--interactive", "--prompt", 5], "interactive"),
            (["--checkpoint_path", folder, "--speculate_k", 4], "speculative"),
            (["--prompt", 4], "either --checkpoint_path"),
            (["--checkpoint_path", folder, "--random", "7B"], "either --checkpoint_path"),
            (["--checkpoint_path", folder, "--prompt", "some text"], "tokenizer"),
            (["--random", "no-such-model", "--prompt", 4], "preset"),
            (["--checkpoint_path", folder, "--prompt", 60, "--max_new_tokens", 10,
              "--num_samples", 1], "64 positions")):
        proc = _cli(*args)
        assert proc.returncode != 0, args
        assert needle in (proc.stderr + proc.stdout), (args, proc.stderr[-500:])


def test_command_line_text_prompt_starts_with_bos(tmp_path_factory, tmp_path):
    """A folder with only a tokenizer.json (the Llama-3 family's kind): the text prompt is
    encoded with the BOS id of config.json in front (generate.py:213-217)."""
    import json as _json
    import shutil
    from tokenizers import Tokenizer, models, pre_tokenizers
    src = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    folder = str(tmp_path / "with_tokenizer")
    shutil.copytree(src, folder)
    cfg_path = os.path.join(folder, "config.json")
    c = _json.load(open(cfg_path))
    c["bos_token_id"] = 7
    _json.dump(c, open(cfg_path, "w"))
    vocab = {f"w{i}": i for i in range(c["vocab_size"])}
    tk = Tokenizer(models.WordLevel(vocab, unk_token="w0"))
    tk.pre_tokenizer = pre_tokenizers.Whitespace()
    tk.save(os.path.join(folder, "tokenizer.json"))
    pcfg, w = plain.load_folder(folder)
    want = plain.greedy_generate(w, pcfg, [7, 21, 5, 300], 5)
    proc = _cli("--checkpoint_path", folder, "--prompt", "w21 w5 w300", "--temperature", 0,
                "--num_samples", 1, "--max_new_tokens", 5, "--dtype", "float32")
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Prompt Length: 4" in proc.stdout
    text = " ".join(f"w{t}" for t in [7, 21, 5, 300] + want)
    assert text in proc.stdout


def test_command_line_interactive_streams_the_answer(tmp_path_factory, tmp_path):
    """--interactive (generate.py:356-377, 404-407): the prompt is asked for, a folder with
    "chat" in its path wraps it in [INST] .. [/INST] (generate.py:298, 359), and the drawn
    tokens' text is written as it comes, each word with the space in front of it."""
    import json as _json
    import shutil
    from tokenizers import Tokenizer, models, pre_tokenizers
    src = util.make_folder(tmp_path_factory.getbasetemp(), "B")
    for name, wrap in (("plain_folder", False), ("tiny-chat-folder", True)):
        folder = str(tmp_path / name)
        shutil.copytree(src, folder)
        cfg_path = os.path.join(folder, "config.json")
        c = _json.load(open(cfg_path))
        c["bos_token_id"] = 7
        _json.dump(c, open(cfg_path, "w"))
        vocab = {f"w{i}": i for i in range(c["vocab_size"] - 3)}
        vocab.update({"[INST]": c["vocab_size"] - 3, "[/INST]": c["vocab_size"] - 2, ".": c["vocab_size"] - 1})
        tk = Tokenizer(models.WordLevel(vocab, unk_token="w0"))
        tk.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
        tk.save(os.path.join(folder, "tokenizer.json"))
        pcfg, w = plain.load_folder(folder)
        ids = [21, 5, 300]
        if wrap:
            ids = [vocab["[INST]"]] + ids + [vocab["[/INST]"]]
        want = plain.greedy_generate(w, pcfg, [7] + ids, 6)
        proc = subprocess.run([sys.executable, "-m", "gpt_fast_amd", "--checkpoint_path", folder,
                               "--interactive", "--temperature", "0", "--num_samples", "1",
                               "--max_new_tokens", "6", "--dtype", "float32", "--prompt", "w1 w2"],
                              cwd=ROOT, input="w21 w5 w300\n", capture_output=True, text=True, timeout=110)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert "What is your prompt? " in proc.stdout
        inv = {i: t for t, i in vocab.items()}
        assert "".join(" " + inv[t] for t in want) in proc.stdout, proc.stdout[-800:]
        assert f"Prompt Length: 3" in proc.stdout          # of the warm-up prompt, BOS included


def test_windowed_layers_at_twenty_rows(tmp_path_factory):
    """The same three kinds of layer with twenty sequences decoding at once: a step of twenty
    rows runs on the tiled-weight products and the attention kernel that adds the projection's
    slices itself, with windows, while windowed groups give pages back (their table entries
    turn -1).  bfloat16 against the plain model with the same windows."""
    import dataclasses
    import gpt_fast_amd as gfa
    from gpt_fast_amd import Entry
    from gpt_fast_amd.weights.bindings import load_parameters
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "B", dtype="bfloat16")
    arch, cfg = gfa.read_model_folder(folder)
    plan = arch.plan(cfg)
    windows = [None, 70, 20]
    plan.layers = [dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, window=win))
                   for layer, win in zip(plan.layers, windows)]
    params = load_parameters(folder, arch.bindings(cfg), "bfloat16", torch.device("cuda:0"))
    eng = gfa.Engine.from_plan(plan, params, "bfloat16", "cuda:0", max_tokens=64 * 20 * 4,
                               max_sequences=20)
    pcfg, w = plain.load_folder(folder)
    n_seq, new = 20, 40
    prompts = [60 + 7 * i for i in range(n_seq)]                       # 60 .. 193 tokens
    seqs = [util.random_tokens(pcfg["vocab"], prompts[i] + new, 40 + i) for i in range(n_seq)]
    slots = [eng.start_sequence() for _ in range(n_seq)]
    got = [[] for _ in range(n_seq)]
    for lo in range(0, n_seq, 5):                                      # prompts five at a time
        out = eng.step([Entry(slots[i], seqs[i][:prompts[i]], want=[prompts[i] - 1])
                        for i in range(lo, lo + 5)]).cpu()
        for j, i in enumerate(range(lo, lo + 5)):
            got[i].append(out[j])
    for t in range(new - 1):
        out = eng.step([Entry(slots[i], [seqs[i][prompts[i] + t]], want=[0]) for i in range(n_seq)]).cpu()
        for i in range(n_seq):
            got[i].append(out[i])
    for i in (0, 7, 13, 19):
        want = _plain_forward_with_windows(w, pcfg, seqs[i][:-1], windows)[prompts[i] - 1:]
        assert rel_err(torch.stack(got[i]), want) < TOL_BF16, i
    gone = [sum(1 for p in eng.cache.page_list(gid, slots[19]) if p < 0)
            for gid, g in eng.cache.kv_groups if g.need.window == 20]
    assert gone and gone[0] >= 2                                        # pages did go back
    eng.cache.check()
    for s in slots:
        eng.end_sequence(s)
