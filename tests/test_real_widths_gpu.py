"""The engine against the plain implementation at the layer widths of real checkpoints
(two layers of the Llama-3.1-8B shape; two of the Llama-2-7B shape), where the bfloat16
engine picks by shape the kernels that serving runs: two tiles of W per workgroup, tile
heights below 16, the own gate kernel at 25..64 rows, the sliced second feed-forward product,
the head-size-128 prompt kernel, single-token attention with four query heads per kv head
and a page row beyond 63 entries, the many-workgroup sampler.  The tiny configurations of
the other tests reach few of these.  The reference checks its numerics on the real model
only (eval.py:134-148); weights here are random, bfloat16, N(0, 0.02).
"""
import os

import pytest
import torch

import plain_llama as plain
import util
from util import TOL_BF16, TOL_F32, rel_err

pytestmark = pytest.mark.gpu

LLAMA31_SCALING = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                   "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
WIDE = {
    "8B": {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 4096,
           "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 8,
           "intermediate_size": 14336, "vocab_size": 128256, "max_position_embeddings": 8192,
           "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "rope_scaling": LLAMA31_SCALING,
           "tie_word_embeddings": False},
    "7B": {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 4096,
           "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 32,
           "intermediate_size": 11008, "vocab_size": 32000, "max_position_embeddings": 4096,
           "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "rope_scaling": None,
           "tie_word_embeddings": False},
}


class Wide:
    """A model folder of one of the shapes, and the plain implementation's view of it."""

    def __init__(self, tmp, name):
        import gpt_fast_amd as gfa
        arch = gfa.config.registry.architecture_of(WIDE[name])
        self.folder = os.path.join(str(tmp), f"wide_{name}")
        print(f"[real widths] writing {name} ...", flush=True)
        gfa.write_random_model(self.folder, arch, arch.read_config(WIDE[name]), seed=11,
                               dtype="bfloat16", std=0.02)
        self.cfg, self.w = plain.load_folder(self.folder)        # float32 copies of the bf16 values
        self.vocab = self.cfg["vocab"]

    def rows(self, tokens, rows):
        """Plain logits of ``tokens`` at the positions ``rows`` (the head on those rows only;
        everything before it is the whole sequence, model.py:136-146)."""
        idx = torch.as_tensor(tokens, dtype=torch.long)
        pos = torch.arange(idx.numel())
        x = self.w["tok_embeddings.weight"][idx]
        for i in range(self.cfg["n_layer"]):
            x = plain.block(x, self.w, i, self.cfg, pos)
        x = plain.rms_norm(x[torch.as_tensor(rows)], self.w["norm.weight"], self.cfg["eps"])
        return x @ self.w["output.weight"].T

    def engine(self, dtype, max_tokens):
        import gpt_fast_amd as gfa
        return gfa.Engine.from_folder(self.folder, dtype=dtype, device="cuda:0", max_tokens=max_tokens)


@pytest.fixture(scope="module", params=["8B", "7B"])
def wide(request, tmp_path_factory):
    model = Wide(tmp_path_factory.mktemp("wide"), request.param)
    yield model
    model.w = None
    os.remove(os.path.join(model.folder, "model.safetensors"))


def _all_rows(engine, tokens, cuts):
    """Logits of every position, the tokens fed in steps of the lengths ``cuts``."""
    from gpt_fast_amd import Entry
    slot = engine.start_sequence()
    out, at = [], 0
    for n in cuts:
        out.append(engine.step([Entry(slot, tokens[at:at + n], want=list(range(n)))]).cpu())
        at += n
    assert at == len(tokens)
    engine.end_sequence(slot)
    return torch.cat(out)


def test_a_prompt_whole_and_in_chunks(wide):
    tokens = util.random_tokens(wide.vocab, 300, 1)
    print("[real widths] plain forward of 300 tokens ...", flush=True)
    want = wide.rows(tokens, list(range(300)))
    eng = wide.engine("bfloat16", 1024)
    whole = _all_rows(eng, tokens, [300])
    assert rel_err(whole, want) < TOL_BF16
    cut = _all_rows(eng, tokens, [37, 29, 1, 233])
    assert rel_err(cut, want) < TOL_BF16
    # the two cuttings differ by the rounding of different kernels only
    assert rel_err(cut, whole) < TOL_BF16 / 2
    del eng
    torch.cuda.empty_cache()
    eng = wide.engine("float32", 1024)
    whole32 = _all_rows(eng, tokens, [300])
    assert rel_err(whole32, want) < TOL_F32
    assert torch.equal(_all_rows(eng, tokens, [37, 29, 1, 233]), whole32)


def test_single_token_steps_at_many_row_counts(wide):
    """Sequences of unequal contexts (one beyond 4,100 keys: its page row has more than 63
    entries and its context is split over workgroups) decode together, teacher-forced, while
    the batch shrinks through 64, 48, 32, 24, 20, 16, 12, 8 and 1 rows."""
    from gpt_fast_amd import Entry
    counts = [64, 48, 32, 24, 20, 16, 12, 8, 1] if wide.cfg["n_kv"] == 8 else [32, 8, 1]
    long_context = 4130 if wide.cfg["n_kv"] == 8 else 700
    n_seq = counts[0]
    steps_of = [sum(1 for c in counts if c > i) for i in range(n_seq)]   # row i lives while count > i
    lengths = [long_context] + [3 + (11 * i) % 37 for i in range(1, n_seq)]
    seqs = [util.random_tokens(wide.vocab, L + n, 50 + i)
            for i, (L, n) in enumerate(zip(lengths, steps_of))]
    eng = wide.engine("bfloat16", 64 * n_seq * 2 + long_context + 256)
    slots = [eng.start_sequence() for _ in seqs]
    got = [[] for _ in seqs]
    for first in range(0, n_seq, 16):                     # the prompts, sixteen to a step
        rows = list(range(first, min(first + 16, n_seq)))
        logits = eng.step([Entry(slots[i], seqs[i][:lengths[i]], want=[lengths[i] - 1])
                           for i in rows]).cpu()
        for r, i in enumerate(rows):
            got[i].append(logits[r:r + 1])
    for t, count in enumerate(counts):
        live = list(range(count))
        logits = eng.step([Entry(slots[i], [seqs[i][lengths[i] + t]], want=[0]) for i in live]).cpu()
        for r, i in enumerate(live):
            got[i].append(logits[r:r + 1])
        nxt = counts[t + 1] if t + 1 < len(counts) else 0
        for i in range(nxt, count):
            eng.end_sequence(slots[i])
    eng.cache.check()
    assert eng.cache.slots.held == 0
    print("[real widths] plain forwards of the decoded sequences ...", flush=True)
    for i, seq in enumerate(seqs):
        fed = seq[:lengths[i] + steps_of[i]]
        want = wide.rows(fed, list(range(lengths[i] - 1, len(fed))))
        assert rel_err(torch.cat(got[i]), want) < TOL_BF16, (i, lengths[i], steps_of[i])


def test_generation_with_the_recorded_step(wide):
    """generate() - prefill, then the one-token step replayed from its recording, argmax and
    the many-workgroup sampler on the device - draws tokens that the plain logits of its own
    sequences bear out: greedy tokens are the best within the bfloat16 tolerance, sampled ones
    lie within the top-k."""
    from gpt_fast_amd.engine.generate import generate
    eng = wide.engine("bfloat16", 8 * 256)
    prompts = [util.random_tokens(wide.vocab, n, 80 + n) for n in (5, 130, 17, 64, 1, 33, 90, 12)]
    new = 6
    for temperature, top_k in ((0.0, None), (0.8, 50)):
        out = generate(eng, prompts, max_new_tokens=new, temperature=temperature, top_k=top_k,
                       seed=7, stop_tokens=())
        assert [len(t) for t in out.tokens] == [new] * len(prompts)
        again = generate(eng, prompts, max_new_tokens=new, temperature=temperature, top_k=top_k,
                         seed=7, stop_tokens=(), use_graph=False)
        assert again.tokens == out.tokens                  # replayed and stepped: the same kernels
        for p, t in zip(prompts, out.tokens):
            logits = wide.rows(p + t[:-1], list(range(len(p) - 1, len(p) + new - 1)))
            for i, tok in enumerate(t):
                row = logits[i]
                slack = TOL_BF16 * float(row.abs().max())
                bound = float(row.max()) if top_k is None else float(torch.topk(row, top_k).values[-1])
                assert float(row[tok]) >= bound - slack, (temperature, len(p), i, tok)
    eng.cache.check()
    assert eng.cache.slots.held == 0


def test_generation_of_more_sequences_than_the_few_row_kernels_take(wide):
    """80 sequences at once: the one-token step has 80 rows, more than any hand-written
    product takes, so its products are the vendor library's - cut into slices of the inner
    size where the result has few tiles - recorded and replayed like the others."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.engine.generate import generate
    from gpt_fast_amd.ops import linear as L
    assert L._library_slices(80, wide.cfg["dim"], 11008, torch.device("cuda:0")) > 1      # a feed-forward's second product is cut
    eng = gfa.Engine.from_folder(wide.folder, dtype="bfloat16", device="cuda:0",
                                 max_tokens=80 * 64, max_sequences=80)
    prompts = [util.random_tokens(wide.vocab, 2 + (7 * i) % 23, 300 + i) for i in range(80)]
    new = 4
    out = generate(eng, prompts, max_new_tokens=new, temperature=0.0, seed=1, stop_tokens=())
    again = generate(eng, prompts, max_new_tokens=new, temperature=0.0, seed=1, stop_tokens=(),
                     use_graph=False)
    assert again.tokens == out.tokens
    for b in (0, 33, 79):
        p, t = prompts[b], out.tokens[b]
        logits = wide.rows(p + t[:-1], list(range(len(p) - 1, len(p) + new - 1)))
        for i, tok in enumerate(t):
            assert float(logits[i][tok]) >= float(logits[i].max()) - TOL_BF16 * float(logits[i].abs().max())
    eng.cache.check()
    assert eng.cache.slots.held == 0
