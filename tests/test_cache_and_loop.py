"""The cache's bookkeeping and the generation loop's decisions.  No GPU: the cache is
built on CPU tensors and the loop is driven by a scripted stepper."""
import random

import pytest
import torch

from gpt_fast_amd.cache.slots import CacheFull, FreeList
from gpt_fast_amd.cache.store import Cache, KVNeed, StateNeed
from gpt_fast_amd.engine.batch import BatchLayout, Entry, fill_host
from gpt_fast_amd.engine.generate import BatchRun, generate, split_batches

import numpy as np


def test_free_list_never_loses_or_doubles():
    f = FreeList(5, "thing")
    got = [f.take() for _ in range(5)]
    assert got == [0, 1, 2, 3, 4] and f.free == 0
    with pytest.raises(CacheFull):
        f.take()
    f.give(3)
    f.give(1)
    with pytest.raises(ValueError, match="not held"):
        f.give(3)                                   # freed twice
    with pytest.raises(ValueError):
        f.give(9)
    assert f.take() == 1 and f.take() == 3          # lowest first: slots are used again
    f.check()
    rng = random.Random(0)
    held = set(range(5))
    for _ in range(500):
        if held and rng.random() < 0.5:
            i = rng.choice(sorted(held))
            f.give(i)
            held.remove(i)
        elif f.free:
            i = f.take()
            assert i not in held
            held.add(i)
        f.check()
        assert f.held == len(held)


def make_cache(max_tokens=64 * 6, max_sequences=4, window=None):
    needs = [KVNeed(2, 8, None), KVNeed(2, 8, window), KVNeed(2, 8, None), StateNeed((3,))]
    return Cache(needs, [None, None, None, None], max_tokens=max_tokens,
                 max_sequences=max_sequences, dtype=torch.float32, device="cpu")


def test_groups_by_need():
    c = make_cache(window=32)
    # runs 0 and 2 share a group (equal needs), the windowed run and the state run have their own
    assert len(c.groups) == 3
    assert c.entries[0].group_id == c.entries[2].group_id != c.entries[1].group_id
    assert (c.entries[0].index, c.entries[2].index) == (0, 1)
    assert c.groups[c.entries[0].group_id].k.shape == (2, 7, 2, 64, 8)       # 6 pages and the spare one
    assert c.groups[c.entries[0].group_id].v.shape == (2, 7, 2, 8, 64)
    assert c.entries[3].state.shape == (5, 3)                  # 4 slots and the spare one
    assert c.spare_slot == 4
    # a borrowed entry reads the lender's storage and does not write
    b = Cache([KVNeed(1, 8), KVNeed(1, 8)], [None, 0], max_tokens=64, max_sequences=1,
              dtype=torch.float32, device="cpu")
    assert b.entries[1].index == b.entries[0].index and not b.entries[1].writes
    assert b.groups[0].entries == 1


def test_pages_follow_lengths_and_come_back():
    c = make_cache()
    a, b = c.acquire(), c.acquire()
    assert c.extend(a, 70) == 0 and c.length(a) == 70
    assert len(c.page_list(0, a)) == 2
    assert c.extend(b, 1) == 0
    assert c.extend(a, 58) == 70 and len(c.page_list(0, a)) == 2      # 128 tokens: still 2 pages
    assert c.extend(a, 1) == 128 and len(c.page_list(0, a)) == 3
    assert c.tokens_held() == 192 + 64
    c.check()
    # all-or-nothing: 6 pages in the pool, 4 held; this step would need 3 more
    with pytest.raises(CacheFull):
        c.extend_many([(a, 64), (b, 128)])
    assert c.length(a) == 129 and c.length(b) == 1
    c.check()
    pages_a = list(c.page_list(0, a))
    c.release(a)
    with pytest.raises(ValueError, match="not held"):
        c.release(a)
    with pytest.raises(ValueError):
        c.extend(a, 1)
    d = c.acquire()
    assert d == a and c.length(d) == 0                # the slot is used again
    c.extend(d, 64 * 3)
    assert set(c.page_list(0, d)) == set(pages_a)     # and so are its pages
    c.check()
    c.release(b)
    c.release(d)
    c.check()
    assert c.slots.held == 0 and all(g.pages.held == 0 for _, g in c.kv_groups)


def test_same_slot_twice_in_a_step_is_refused():
    c = make_cache()
    a = c.acquire()
    with pytest.raises(ValueError, match="twice"):
        c.extend_many([(a, 1), (a, 1)])
    with pytest.raises(ValueError):
        c.extend(a, 0)


def test_window_gives_pages_back():
    c = make_cache(max_tokens=64 * 8, window=70)
    wg = c.entries[1].group_id
    a = c.acquire()
    c.extend(a, 64 * 4)
    assert c.groups[wg].pages.held == 4
    c.extend(a, 1)            # start = 256: keys below 256 - 70 + 1 = 187 are out of reach
    assert c.page_list(wg, a)[:2] == [-1, -1] and c.page_list(wg, a)[2] >= 0
    assert c.groups[wg].pages.held == 3
    assert c.groups[c.entries[0].group_id].pages.held == 5      # the full group keeps all
    c.check()
    c.release(a)
    c.check()


def test_state_is_zeroed_at_acquire():
    c = make_cache()
    a = c.acquire()
    c.entries[3].state[a] += 5.0
    c.release(a)
    assert c.acquire() == a
    assert float(c.entries[3].state[a].abs().sum()) == 0.0


def test_batch_description_layout():
    c = make_cache()
    a, b = c.acquire(), c.acquire()
    starts = c.extend_many([(a, 3), (b, 70)])
    entries = [Entry(a, [5, 6, 7], want=[0, 2], key=11), Entry(b, list(range(70)), want=[69], key=12)]
    widths = {gid: 2 for gid, _ in c.kv_groups}
    lay = BatchLayout(73, 2, 3, widths)
    host = np.zeros(lay.size, dtype=np.int32)
    fill_host(lay, host, entries, starts, c)
    f = lambda name: host[lay.fields[name][0]: lay.fields[name][0] + lay.fields[name][1]]
    assert list(f("tokens")[:4]) == [5, 6, 7, 0]
    assert list(f("tok_seq")[:4]) == [0, 0, 0, 1] and list(f("tok_pos")[:5]) == [0, 1, 2, 0, 1]
    assert list(f("q_start")) == [0, 3, 73] and list(f("want_rows")) == [0, 2, 72]
    assert list(f("row_keys")) == [11, 12]
    assert list(f("want_pos")) == [0, 2, 69] and list(f("slots")) == [a, b]
    assert list(f("seed")) == [0, 0]
    off, n = lay.tables[0]
    table = host[off:off + n].reshape(2, 2)
    assert table[0, 0] == c.page_list(0, a)[0] and table[0, 1] == -1
    assert list(table[1]) == c.page_list(0, b)
    with pytest.raises(ValueError):
        fill_host(lay, host, [Entry(a, [1, 2, 3], want=[3]), entries[1]], starts, c)


def test_filler_rows_point_at_the_spare_page_and_slot_and_the_seed_is_two_words():
    c = make_cache()
    a = c.acquire()
    starts = c.extend_many([(a, 1)]) + [0]
    entries = [Entry(a, [5], want=[0], key=1), Entry(None, [0], want=[0], key=2)]
    lay = BatchLayout(2, 2, 2, {gid: 3 for gid, _ in c.kv_groups})
    host = np.zeros(lay.size, dtype=np.int32)
    fill_host(lay, host, entries, starts, c, seed=(5 << 32) | 0xFFFFFFFE)
    f = lambda name: host[lay.fields[name][0]: lay.fields[name][0] + lay.fields[name][1]]
    assert list(f("slots")) == [a, c.spare_slot] and c.spare_slot == c.max_sequences
    assert list(f("seed")) == [-2, 5]                 # low word 0xFFFFFFFE as int32, high word
    for gid, g in c.kv_groups:
        off, n = lay.tables[gid]
        table = host[off:off + n].reshape(2, 3)
        assert list(table[1]) == [g.spare_page] * 3 and table[0, 0] == c.page_list(gid, a)[0]
    # the spare slot's state is nobody's: acquiring every slot never hands it out
    held = [a] + [c.acquire() for _ in range(c.max_sequences - 1)]
    assert c.spare_slot not in held
    with pytest.raises(CacheFull):
        c.acquire()


def test_room_is_checked_for_whole_batches():
    c = make_cache(max_tokens=64 * 6, max_sequences=4)
    c.require_room([64, 64, 128, 100])                # 1 + 1 + 2 + 2 pages
    with pytest.raises(CacheFull, match="tokens"):
        c.require_room([65, 64, 128, 100])
    with pytest.raises(CacheFull, match="slots"):
        c.require_room([1, 1, 1, 1, 1])


def test_generate_refuses_before_it_starts():
    """Too long for the model's positions, or too much for the cache: an error before any
    slot is taken or any step runs."""
    class Plan:
        stop_tokens = ()
        max_positions = 50

    class Model:
        plan = Plan

    class Eng:
        model = Model
        cache = make_cache(max_tokens=64 * 2, max_sequences=2)

    st = ScriptedStepper(lambda key, fed: 1)
    with pytest.raises(ValueError, match="50 positions"):
        generate(Eng, [[1] * 45], 6, temperature=0.0, stepper=st)
    Plan.max_positions = 200
    with pytest.raises(CacheFull):
        generate(Eng, [[1] * 30, [2] * 30, [3]], 5, temperature=0.0, stepper=st)
    with pytest.raises(CacheFull):                    # 70 tokens each: two pages each
        generate(Eng, [[1] * 40] * 2, 31, temperature=0.0, stepper=st, batch_size=2)
    assert st.calls == [] and st.slots.held == 0
    # the last token drawn is never fed: 60 + 5 - 1 = 64 tokens are one page each
    Plan.max_positions = 65
    out = generate(Eng, [[1] * 60, [2] * 60], 5, temperature=0.0, stepper=st)
    assert [len(t) for t in out.tokens] == [5, 5]


class ScriptedStepper:
    """Hands out slots, checks what the loop asks for, answers from a script:
    the token for (request key, number of tokens fed so far)."""

    def __init__(self, script, n_slots=8):
        self.script = script
        self.slots = FreeList(n_slots, "slot")
        self.fed = {}
        self.calls = []

    def start_sequence(self):
        s = self.slots.take()
        self.fed[s] = []
        return s

    def end_sequence(self, slot):
        self.slots.give(slot)
        del self.fed[slot]

    def next_tokens(self, entries):
        out = []
        self.calls.append([(e.key, list(e.tokens)) for e in entries])
        for e in entries:
            assert list(e.want) == [len(e.tokens) - 1]
            self.fed[e.slot] += list(e.tokens)
            out.append(self.script(e.key, self.fed[e.slot]))
        return out


def test_loop_unequal_prompts_stop_tokens_and_early_ends():
    # every request echoes (last token + 1); token 50 is the stop token
    st = ScriptedStepper(lambda key, fed: fed[-1] + 1)
    prompts = [[10, 11], [47], [30, 31, 32], [49]]
    run = BatchRun(st, prompts, keys=[0, 1, 2, 3], max_new_tokens=5, stop_tokens=[50])
    new, why = run.run()
    assert new == [[12, 13, 14, 15, 16], [48, 49, 50], [33, 34, 35, 36, 37], [50]]
    assert why == ["length", "stop", "length", "stop"]
    # the prompts go in one step, then one token per live request; ended ones drop out
    assert st.calls[0] == [(0, [10, 11]), (1, [47]), (2, [30, 31, 32]), (3, [49])]
    assert st.calls[1] == [(0, [12]), (1, [48]), (2, [33])]
    assert st.calls[3] == [(0, [14]), (2, [35])]
    assert len(st.calls) == 5 and run.steps == 5      # reference: max_new_tokens model calls
    assert st.slots.held == 0


def test_loop_gives_slots_back_on_errors():
    def script(key, fed):
        if len(fed) > 3:
            raise RuntimeError("boom")
        return 1
    st = ScriptedStepper(script)
    with pytest.raises(RuntimeError):
        BatchRun(st, [[1], [2, 3]], [0, 1], 9).run()
    assert st.slots.held == 0
    with pytest.raises(ValueError):
        BatchRun(st, [[]], [0], 3)
    with pytest.raises(ValueError):
        BatchRun(st, [[1]], [0], 0)


def test_batches_one_after_another_reuse_slots():
    assert split_batches(5, 2) == [[0, 1], [2, 3], [4]]
    assert split_batches(3, None) == [[0, 1, 2]] and split_batches(0, 4) == []
    st = ScriptedStepper(lambda key, fed: key, n_slots=2)

    class FakeEngine:
        class model:
            class plan:
                stop_tokens = ()
    seen = []
    res = generate(FakeEngine, [[1], [2, 2], [3], [4, 4, 4], [5]], 3, temperature=0.0,
                   batch_size=2, stepper=st, callback=lambda rows, toks: seen.append((rows, toks)))
    assert res.tokens == [[0] * 3, [1] * 3, [2] * 3, [3] * 3, [4] * 3]
    assert res.finish_reasons == ["length"] * 5 and res.stats["steps"] == 9
    assert seen[0] == ([0, 1], [0, 1]) and seen[3] == ([2, 3], [2, 3]) and seen[-1] == ([4], [4])
    assert st.slots.held == 0


class SessionStepper(ScriptedStepper):
    """A scripted stepper that also offers decode sessions, answering one step late like
    the device session does."""

    def open_session(self, slots, keys, last_tokens, max_new_tokens):
        outer = self

        class Session:
            def __init__(self):
                self.slots = list(slots)
                self.keys = list(keys)
                self.last = list(last_tokens)
                self.launches = 0

            def retire(self, row):
                assert self.slots[row] is not None
                self.slots[row] = None

            def launch(self):
                self.launches += 1
                out = []
                for r, s in enumerate(self.slots):
                    if s is None:
                        out.append(-777)               # junk of a filler row
                        continue
                    outer.fed[s].append(self.last[r])
                    self.last[r] = outer.script(self.keys[r], outer.fed[s])
                    out.append(self.last[r])
                return out

            def collect(self, handle):
                return handle

            def close(self):
                self.closed = True
        self.session = Session()
        return self.session


def test_loop_with_a_session_notices_stops_one_step_late():
    st = SessionStepper(lambda key, fed: fed[-1] + 1)
    prompts = [[10, 11], [47], [30, 31, 32], [49]]
    run = BatchRun(st, prompts, keys=[0, 1, 2, 3], max_new_tokens=5, stop_tokens=[50])
    new, why = run.run()
    # the same tokens and reasons as the synchronous loop
    assert new == [[12, 13, 14, 15, 16], [48, 49, 50], [33, 34, 35, 36, 37], [50]]
    assert why == ["length", "stop", "length", "stop"]
    assert st.slots.held == 0
    # request 3 ended in the prefill and never entered the session; requests 0 and 2 end
    # by length and are not launched beyond it: 4 decode steps in all
    assert len(st.session.slots) == 3 and st.session.launches == 4
    assert st.session.closed
    # request 1's filler row was retired after its stop token was seen
    assert st.session.slots == [0, None, 2] or st.session.slots[1] is None


def test_loop_with_a_session_single_token_budget():
    st = SessionStepper(lambda key, fed: 7)
    new, why = BatchRun(st, [[1, 2], [3]], [0, 1], max_new_tokens=1).run()
    assert new == [[7], [7]] and why == ["length", "length"]
    assert not hasattr(st, "session")                 # nothing left to decode


def test_bench_refuses_more_than_one_gpu_in_one_line():
    """bench.py measures one GPU: for N > 1 it prints one line that says so and exits with 2,
    before anything touches a device."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "4"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1 and "one GPU" in r.stdout


def test_attention_plan_for_single_token_steps():
    """How a single-token step is cut over waves: pure arithmetic, no kernel.  More sequences
    mean fewer context splits; a split leaves a wave two 32-key blocks of the table's capacity
    at least, there are never more than 32, and short contexts are not split at all."""
    import functools
    from gpt_fast_amd.ops import attention_bf16 as A
    MAX_SPLITS, plan = A.MAX_SPLITS, functools.partial(A.plan, units=256)   # the chip it was tuned on
    H, G, hd = 32, 8, 128
    for n_seqs in (1, 3, 8, 16, 64, 300):
        last = MAX_SPLITS
        for width in (1, 4, 12, 17, 65, 257, 2048):
            rt, nw, tiles, splits = plan(n_seqs, 1, H, G, hd, width)
            assert rt == 1 and tiles == 1 and nw == 4
            assert 1 <= splits <= MAX_SPLITS
            assert splits == 1 or splits * nw * 64 <= width * 64 + nw * 64
        for n_more in (n_seqs, 2 * n_seqs, 5 * n_seqs):
            now = plan(n_more, 1, H, G, hd, 257)[3]
            assert now <= last
            last = now
    assert plan(1, 1, H, G, hd, 4)[3] == 1 and plan(8, 1, H, G, hd, 12)[3] == 1
    assert plan(1, 1, H, G, hd, 33)[3] == 9 and plan(1, 1, H, G, hd, 65)[3] == 17
    assert plan(1, 1, H, G, hd, 257)[3] == 32
    assert plan(8, 1, H, G, hd, 65)[3] == 4 and plan(4, 1, H, G, hd, 65)[3] == 8
    assert plan(16, 1, H, G, hd, 65)[3] == 1 and plan(16, 1, H, G, hd, 129)[3] == 2
    assert plan(64, 1, H, G, hd, 2048)[3] == 1
    # 32 query heads on one kv head: two row tiles per token; wide heads: two waves
    assert plan(2, 1, 32, 1, 64, 8)[2] == 2
    assert plan(2, 1, 4, 2, 256, 8)[1] == 2


def test_cache_page_order_is_a_permutation():
    """The order in which a page's keys and values lie (the kernel tests build and read pages
    through util.key_places / value_places): every element has one place, for head sizes that
    take the operand order and for those that fall back to rows; and in the operand order the
    sixteen keys of a score tile and a 16-byte chunk of dims are 256 consecutive bytes."""
    import torch
    import util
    for hd in (16, 20, 24, 48, 64, 128, 256):
        kp, vp = util.key_places(hd), util.value_places(hd)
        assert sorted(kp.reshape(-1).tolist()) == list(range(64 * hd))
        assert sorted(vp.reshape(-1).tolist()) == list(range(64 * hd))
        k = torch.arange(2 * 3 * 64 * hd, dtype=torch.float32).view(2, 3, 64, hd)
        v = -torch.arange(2 * 3 * 64 * hd, dtype=torch.float32).view(2, 3, hd, 64)
        a, b = util.to_cache_order(k, v)
        k2, v2 = util.from_cache_order(a, b)
        assert torch.equal(k, k2) and torch.equal(v, v2)
    kp = util.key_places(128)
    # tile t of a 32-key block: keys 8 a + 4 t + b; their chunk c lies at slots 16 t .. 16 t + 15
    for t in (0, 1):
        keys = [8 * a + 4 * t + b for a in range(4) for b in range(4)]
        for c in (0, 5, 15):
            places = [int(kp[32 + k, 8 * c]) for k in keys]
            assert places == list(range(places[0], places[0] + 128, 8))
    vp = util.value_places(128)
    # a value tile: dims 16 j .. 16 j + 15, eight consecutive keys each: 16 bytes per dim, dims side by side
    assert [int(vp[16 + i, 40]) for i in range(16)] == list(range(int(vp[16, 40]), int(vp[16, 40]) + 128, 8))
    assert [int(vp[16, 40 + e]) for e in range(8)] == list(range(int(vp[16, 40]), int(vp[16, 40]) + 8))


def test_a_cache_need_of_another_kind_and_values_of_another_width():
    """Needs are an open table: a kind registered here gets a group of its class, takes part
    in acquire / extend / release with the others, and can refuse a step as a whole.  Keys
    and values of a KV need may have different widths."""
    from dataclasses import dataclass

    from gpt_fast_amd.cache.slots import CacheFull
    from gpt_fast_amd.cache.store import Group, register_cache_need

    @dataclass(frozen=True)
    class BudgetNeed:
        tokens: int

    log = []

    class BudgetGroup(Group):
        """Takes at most ``need.tokens`` tokens per sequence."""

        def __init__(self, need, entries, geometry, dtype, device):
            self.need, self.entries, self.geometry = need, entries, geometry

        def acquire(self, slot):
            log.append(("acquire", slot))

        def release(self, slot):
            log.append(("release", slot))

        def plan_extend(self, items, lengths):
            for slot, n_new in items:
                if lengths[slot] + n_new > self.need.tokens:
                    raise CacheFull(f"slot {slot} would exceed {self.need.tokens} tokens")
            return lambda: log.append(("extend", tuple(items)))

    register_cache_need(BudgetNeed, BudgetGroup)
    c = Cache([KVNeed(2, 8, None, value_dim=24), BudgetNeed(100), BudgetNeed(100), None],
              [None, None, None, None], max_tokens=64 * 8, max_sequences=3,
              dtype=torch.float32, device="cpu")
    kv, budget = c.groups
    assert isinstance(budget, BudgetGroup) and budget.entries == 2 and budget.geometry.n_slots == 3
    assert kv.k.shape == (1, 9, 2, 64, 8) and kv.v.shape == (1, 9, 2, 24, 64)
    assert kv.bytes_per_token() == 2 * (8 + 24) * 4
    assert [g for _, g in c.paged_groups] == [kv]
    a, b = c.acquire(), c.acquire()
    c.extend_many([(a, 90), (b, 10)])
    held = kv.pages.held
    with pytest.raises(CacheFull, match="exceed 100"):
        c.extend_many([(b, 70), (a, 11)])               # the budget refuses: nothing changes,
    assert kv.pages.held == held and c.length(a) == 90 and c.length(b) == 10   # not even pages
    c.extend_many([(b, 70)])
    c.release(a)
    c.release(b)
    c.check()
    assert [e[0] for e in log] == ["acquire", "acquire", "extend", "extend", "release", "release"]
    with pytest.raises(TypeError, match="registered kind"):
        Cache([object()], [None], max_tokens=64, max_sequences=1, dtype=torch.float32, device="cpu")


def test_a_part_can_ask_for_a_field_of_its_own_in_the_steps_description():
    """BatchLayout takes further fields; fill_host has each written by its own function, for
    live rows and for rows that only fill a recorded batch's shape."""
    from gpt_fast_amd.engine.batch import StepField

    def fill(view, entries, starts, cache):
        for b, (e, start) in enumerate(zip(entries, starts)):
            view[b] = -1 if e.slot is None else start + len(e.tokens)

    field = StepField("new_len", lambda n_tokens, n_seqs: n_seqs, fill)
    c = Cache([KVNeed(1, 8)], [None], max_tokens=256, max_sequences=2, dtype=torch.float32, device="cpu")
    a = c.acquire()
    starts = c.extend_many([(a, 3)])
    entries = [Entry(a, [1, 2, 3], want=[2]), Entry(None, [0], want=[0])]
    lay = BatchLayout(4, 2, 2, {0: 2}, extra=[field])
    host = np.zeros(lay.size, dtype=np.int32)
    fill_host(lay, host, entries, [starts[0], 0], c)
    off, count = lay.fields["new_len"]
    assert count == 2 and list(host[off:off + 2]) == [3, -1]
    assert off % 4 == 0 and lay.key() != BatchLayout(4, 2, 2, {0: 2}).key()
    with pytest.raises(ValueError, match="tokens"):
        BatchLayout(1, 1, 1, {}, extra=[StepField("tokens", lambda n, b: 1, fill)])


def test_dispatch_thresholds_follow_the_number_of_compute_units():
    """Decisions that depend on the chip take its number of compute units as an argument:
    the context splits of single-token attention (never more workgroups than compute units,
    none where every second unit has one and the chain is short) and the slices of a
    many-row library product (as many as bring the result tiles to about 2.5 per unit)."""
    from gpt_fast_amd.ops import attention_bf16 as A
    from gpt_fast_amd.ops import linear as L
    # one sequence, 8 kv heads, 4,096 keys: 8 workgroups without a split, 32 blocks per wave
    assert A.plan(1, 1, 32, 8, 128, 64, units=256)[3] == 16        # two blocks per wave at least
    assert A.plan(1, 1, 32, 8, 128, 64, units=64)[3] == 8          # 8 x 8 = 64 workgroups
    assert A.plan(1, 1, 32, 8, 128, 64, units=8)[3] == 1           # already one per unit
    assert A.plan(16, 1, 32, 8, 128, 64, units=256)[3] == 1        # 128 workgroups stream
    assert A.plan(16, 1, 32, 8, 128, 512, units=256)[3] == 2       # ... unless the chain is long
    assert A.plan(1, 1, 32, 8, 128, 3, units=256)[3] == 1          # a short context: no split
    L._units["fake256"], L._units["fake64"] = 256, 64
    try:
        assert L._library_slices(512, 4096, 14336, "fake256") == 4
        assert L._library_slices(200, 4096, 14336, "fake256") == 8
        assert L._library_slices(2048, 4096, 14336, "fake256") == 2
        assert L._library_slices(2048, 4096, 4096, "fake256") == 1
        assert L._library_slices(2048, 4096, 14336, "fake64") == 1
        assert L._library_slices(512, 4096, 4096, "fake256") == 4
        assert L._library_slices(300, 200, 96, "fake256") == 1     # a short inner size is never cut
    finally:
        del L._units["fake256"], L._units["fake64"]


def test_residual_stream_runs_what_was_put_off_before_any_read():
    """The stream holds at most one part's last kernels back; every read - the rows of a norm
    or the tensor itself - runs them first, telling them the norm that reads (only if all
    rows are read) and whether its reader takes the norm in halves."""
    from gpt_fast_amd.parts.base import ResidualStream, add_late
    log = []

    class Norm:
        def forward(self, residual, rows=None):
            log.append(("norm", rows))
            return residual * 2

    class Reader:
        takes_prepared = 3          # halves from three rows on

    def finish(tag, give=None):
        def run(rows, then_norm, takes_halves):
            log.append((tag, then_norm, takes_halves))
            rows += 1
            return give
        return run

    norm = Norm()
    s = ResidualStream(torch.zeros(4, 2))
    s.defer(finish("a"))
    s.defer(finish("b"))                                  # a second part: the first runs now, plainly
    assert log == [("a", None, False)]
    out = s.normed(norm, reader=Reader())
    assert log[1] == ("b", norm, True) and log[2] == ("norm", None)      # no rows handed over: own kernel
    assert torch.equal(out, torch.full((4, 2), 4.0))
    s.defer(finish("c", give="handed over"))
    assert s.normed(norm, reader=None) == "handed over" and log[-1] == ("c", norm, False)
    s.defer(finish("d", give="ignored"))
    s.normed(norm, rows=torch.tensor([1]))                # some rows only: no fused norm is asked for
    assert log[-2] == ("d", None, False) and log[-1][0] == "norm"
    s.defer(finish("e"))
    assert float(s.tensor.sum()) == 5 * 8 and log[-1] == ("e", None, False)
    two = ResidualStream(torch.zeros(2, 2))
    two.defer(finish("f"))
    two.normed(norm, reader=Reader())
    assert ("f", norm, False) in log                      # two rows: below the reader's least
    plain = torch.zeros(1, 2)
    add_late(plain, finish("g"))                          # a plain tensor: at once
    assert log[-1] == ("g", None, False) and float(plain.sum()) == 2
