"""The engine against the plain implementation on the GPU: whole prompts, token by
token, unequal batches with slot reuse, float32 and bfloat16."""
import pytest
import torch

import util
from util import TOL_BF16, TOL_F32, rel_err

pytestmark = pytest.mark.gpu

DTYPES = [("float32", TOL_F32), ("bfloat16", TOL_BF16)]


def engine_for(folder, dtype, max_tokens=4096):
    import gpt_fast_amd as gfa
    return gfa.Engine.from_folder(folder, dtype=dtype, device="cuda:0", max_tokens=max_tokens)


def whole(engine, tokens):
    from gpt_fast_amd import Entry
    slot = engine.start_sequence()
    logits = engine.step([Entry(slot, tokens, want=list(range(len(tokens))))])
    engine.end_sequence(slot)
    return logits.cpu()


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_whole_prompt(tmp_path_factory, name, dtype, tol):
    folder = util.make_folder(tmp_path_factory.getbasetemp(), name, dtype="float32")
    eng = engine_for(folder, dtype)
    V = util.TINY[name]["vocab_size"]
    for n, seed in ((1, 1), (7, 2), (64, 3), (65, 4), (150, 5)):
        tokens = util.random_tokens(V, n, seed)
        want = util.plain_logits(folder, tokens)
        got = whole(eng, tokens)
        assert got.shape == want.shape
        assert rel_err(got, want) < tol, (name, dtype, n)


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_last_32_one_by_one(tmp_path_factory, name, dtype, tol):
    from gpt_fast_amd import Entry
    folder = util.make_folder(tmp_path_factory.getbasetemp(), name, dtype="float32")
    eng = engine_for(folder, dtype)
    V = util.TINY[name]["vocab_size"]
    tokens = util.random_tokens(V, 100, 11)
    want = util.plain_logits(folder, tokens)
    slot = eng.start_sequence()
    head = tokens[:-32]
    got = [eng.step([Entry(slot, head, want=list(range(len(head))))]).cpu()]
    for t in tokens[-32:]:
        got.append(eng.step([Entry(slot, [t], want=[0])]).cpu())
    eng.end_sequence(slot)
    got = torch.cat(got)
    assert rel_err(got, want) < tol
    if dtype == "float32":
        # a float32 result does not depend on the cutting at all
        assert torch.equal(got, whole(eng, tokens))


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_unequal_batches_reuse_slots(tmp_path_factory, name, dtype, tol):
    from gpt_fast_amd import Entry
    folder = util.make_folder(tmp_path_factory.getbasetemp(), name, dtype="float32")
    eng = engine_for(folder, dtype, max_tokens=64 * 12)
    V = util.TINY[name]["vocab_size"]
    for round_, lengths in enumerate(([7, 3, 12], [1, 5, 17, 33], [70, 2, 130, 64], [40, 90])):
        new = [9, 4, 14, 6][:len(lengths)]
        seqs = [util.random_tokens(V, L + n, 100 * round_ + i)
                for i, (L, n) in enumerate(zip(lengths, new))]
        slots = [eng.start_sequence() for _ in seqs]
        got = [[] for _ in seqs]
        # all prompts in one step
        logits = eng.step([Entry(s, q[:L], want=list(range(L)))
                           for s, q, L in zip(slots, seqs, lengths)]).cpu()
        at = 0
        for i, L in enumerate(lengths):
            got[i].append(logits[at:at + L])
            at += L
        # then one token each; shorter requests end earlier
        live = list(range(len(seqs)))
        t = 0
        while live:
            logits = eng.step([Entry(slots[i], [seqs[i][lengths[i] + t]], want=[0])
                               for i in live]).cpu()
            for row, i in enumerate(live):
                got[i].append(logits[row:row + 1])
            t += 1
            for i in [i for i in live if t >= new[i]]:
                eng.end_sequence(slots[i])
                live.remove(i)
        for i, q in enumerate(seqs):
            want = util.plain_logits(folder, q)
            assert rel_err(torch.cat(got[i]), want) < tol, (name, dtype, round_, i)
        eng.cache.check()
    assert eng.cache.slots.held == 0


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_batch_of_forty_shrinking_to_one(tmp_path_factory, name, dtype, tol):
    """Forty sequences decode together and end one after another: single-token steps of 40
    down to 1 rows, which go through the many-row, the few-row and the one-row products."""
    from gpt_fast_amd import Entry
    folder = util.make_folder(tmp_path_factory.getbasetemp(), name, dtype="float32")
    eng = engine_for(folder, dtype, max_tokens=64 * 2 * 40)
    V = util.TINY[name]["vocab_size"]
    n_seq = 40
    lengths = [1 + (7 * i) % 23 for i in range(n_seq)]
    new = [2 + i for i in range(n_seq)]                    # sequence i decodes 2 + i tokens
    seqs = [util.random_tokens(V, L + n, 300 + i) for i, (L, n) in enumerate(zip(lengths, new))]
    slots = [eng.start_sequence() for _ in seqs]
    got = [[] for _ in seqs]
    logits = eng.step([Entry(s, q[:L], want=[L - 1]) for s, q, L in zip(slots, seqs, lengths)]).cpu()
    for i in range(n_seq):
        got[i].append(logits[i:i + 1])
    live = list(range(n_seq))
    t = 0
    while live:
        logits = eng.step([Entry(slots[i], [seqs[i][lengths[i] + t]], want=[0]) for i in live]).cpu()
        for row, i in enumerate(live):
            got[i].append(logits[row:row + 1])
        t += 1
        for i in [i for i in live if t >= new[i]]:
            eng.end_sequence(slots[i])
            live.remove(i)
    for i, q in enumerate(seqs):
        want = util.plain_logits(folder, q)[lengths[i] - 1:]
        assert rel_err(torch.cat(got[i]), want) < tol, (name, dtype, i)
    eng.cache.check()
    assert eng.cache.slots.held == 0


# --------------------------------------------------------------------------------------
# Steps of several tokens at a position other than 0 (the reference runs such a step when it
# verifies a draft, generate.py:104-108, and its mask row is chosen by input_pos,
# model.py:138), and steps that hold rows of every kind at once.
def _chunked(eng, tokens, cuts):
    """Feed ``tokens`` of one sequence as chunks of the given sizes; logits of every row."""
    from gpt_fast_amd import Entry
    assert sum(cuts) == len(tokens)
    slot = eng.start_sequence()
    got, at = [], 0
    for n in cuts:
        got.append(eng.step([Entry(slot, tokens[at:at + n], want=list(range(n)))]).cpu())
        at += n
    eng.end_sequence(slot)
    return torch.cat(got)


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_chunks_at_offsets_off_the_page_edges(tmp_path_factory, name, dtype, tol):
    """100 tokens as chunks of 37 + 29 + 1 + 33: every chunk after the first starts at a
    position that is neither 0 nor a multiple of the page size, and the second ends inside
    the second page."""
    folder = util.make_folder(tmp_path_factory.getbasetemp(), name, dtype="float32")
    eng = engine_for(folder, dtype)
    V = util.TINY[name]["vocab_size"]
    tokens = util.random_tokens(V, 100, 21)
    want = util.plain_logits(folder, tokens)
    got = _chunked(eng, tokens, [37, 29, 1, 33])
    assert rel_err(got, want) < tol
    if dtype == "float32":
        assert torch.equal(got, whole(eng, tokens))
    # other cuts, among them chunks that end exactly on a page edge and one-token chunks
    for cuts in ([64, 36], [63, 1, 36], [1, 1, 62, 36], [5, 95]):
        g2 = _chunked(eng, tokens, cuts)
        assert rel_err(g2, want) < tol, cuts
        if dtype == "float32":
            assert torch.equal(g2, got), cuts
    eng.cache.check()
    assert eng.cache.slots.held == 0


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_one_step_with_decode_rows_a_chunk_and_a_fresh_prompt(tmp_path_factory, name, dtype, tol):
    from gpt_fast_amd import Entry
    folder = util.make_folder(tmp_path_factory.getbasetemp(), name, dtype="float32")
    eng = engine_for(folder, dtype)
    V = util.TINY[name]["vocab_size"]
    seqs, before, mixed = util.mixed_step_case(V)
    slots = {r: eng.start_sequence() for r in seqs}
    got = {r: [] for r in seqs}
    order = ["d0", "d1", "d2", "c"]
    logits = eng.step([Entry(slots[r], seqs[r][:before[r]], want=list(range(before[r])))
                       for r in order]).cpu()
    at = 0
    for r in order:
        got[r].append(logits[at:at + before[r]])
        at += before[r]
    # the mixed step, rows in an order that puts the chunk between single tokens
    order = ["d0", "c", "d1", "p", "d2"]
    fed = {r: before.get(r, 0) for r in order}
    logits = eng.step([Entry(slots[r], seqs[r][fed[r]:fed[r] + mixed[r]],
                             want=list(range(mixed[r]))) for r in order]).cpu()
    at = 0
    for r in order:
        got[r].append(logits[at:at + mixed[r]])
        at += mixed[r]
        fed[r] += mixed[r]
    # the rest of the chunked sequence and of the prompt, one token each, together
    for r in ("c", "p"):
        while fed[r] < len(seqs[r]):
            got[r].append(eng.step([Entry(slots[r], [seqs[r][fed[r]]], want=[0])]).cpu())
            fed[r] += 1
    for r, toks in seqs.items():
        want = util.plain_logits(folder, toks)
        g = torch.cat(got[r])
        assert g.shape == want.shape
        assert rel_err(g, want) < tol, (name, dtype, r)
        if dtype == "float32":
            assert torch.equal(g, whole(eng, toks)), (name, r)
        eng.end_sequence(slots[r])
    eng.cache.check()
    assert eng.cache.slots.held == 0


def test_a_step_refuses_rows_without_a_slot(tmp_path_factory):
    from gpt_fast_amd import Entry
    folder = util.make_folder(tmp_path_factory.getbasetemp(), "A", dtype="float32")
    eng = engine_for(folder, "float32")
    with pytest.raises(ValueError, match="filler"):
        eng.step([Entry(None, [1, 2], want=[1])])
    assert eng.cache.slots.held == 0
