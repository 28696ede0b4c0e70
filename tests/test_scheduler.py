"""The scheduler's decisions, with a stand-in for the engine (the cache manager is the real
one): admission, portions under the token budget, decode, finish and free, and what happens
when pages run out."""
import numpy as np
import pytest
import torch

from zinfer_amd.cache import CacheManager
from zinfer_amd.engine.scheduler import Scheduler
from zinfer_amd.parts import KVNeed
from zinfer_amd.sampling import SamplingParams

V = 50


class FakeEngine:
    """Keeps the real cache manager; logits put all weight on (last token + 1) % V, so that
    generation is predictable and does not depend on the batch."""

    class _Spec:
        vocab_size = V
        max_positions = 1000
        eos_token_ids = ()

    class _Model:
        pass

    def __init__(self, num_pages, page_size=4, max_requests=8):
        self.cache = CacheManager([KVNeed(1, 4)], [None], page_size, num_pages, max_requests,
                                  torch.float32, "cpu")
        self.model = self._Model()
        self.model.spec = self._Spec()
        self.log = []

    def step(self, entries, end=()):
        self.log.append([(e.request_id, len(e.tokens), list(e.want)) for e in entries])
        rows = []
        for e in entries:
            if not self.cache.has_request(e.request_id):
                self.cache.add_request(e.request_id)
            new_len = self.cache.length(e.request_id) + len(e.tokens)
            self.cache.reserve(e.request_id, new_len)
            self.cache.commit(e.request_id, new_len)
            for w in e.want:
                row = np.zeros(V, np.float32)
                row[(e.tokens[w] + 1) % V] = 10.0
                rows.append(row)
        self.cache.check()
        return torch.from_numpy(np.stack(rows)) if rows else torch.zeros((0, V))

    def argmax(self, logits):
        return torch.argmax(logits, dim=-1).tolist()


GREEDY = dict(temperature=0.0, ignore_eos=True)


def test_whole_prompt_then_decode_no_wasted_forward():
    eng = FakeEngine(num_pages=16)
    s = Scheduler(eng, max_step_tokens=64)
    rid = s.add_request([3, 4, 5], SamplingParams(max_new_tokens=4, **GREEDY))
    out = s.run()
    assert out[rid].generated == [6, 7, 8, 9] and out[rid].finish_reason == "length"
    # one prefill step and three decode steps: the fourth token needs no forward of its own
    assert [len(st) for st in eng.log] == [1, 1, 1, 1] and eng.log[0][0][1] == 3
    assert eng.cache.num_free_pages() == [16] and not eng.cache.requests


def test_portions_under_the_token_budget_and_mixed_steps():
    eng = FakeEngine(num_pages=64)
    s = Scheduler(eng, max_step_tokens=10, chunk_size=6)
    a = s.add_request(list(range(1, 15)), SamplingParams(max_new_tokens=3, **GREEDY))   # 14 tokens
    b = s.add_request([7, 8], SamplingParams(max_new_tokens=5, **GREEDY))
    s.run()
    # step 0: a gets a portion of 6, b its 2 tokens (budget 10); b samples, a does not
    assert eng.log[0] == [(a, 6, []), (b, 2, [1])]
    # step 1: b decodes (1 token, first), a's next portion of 6 beside it
    assert eng.log[1] == [(b, 1, [0]), (a, 6, [])]
    # step 2: a's last 2 prompt tokens reach the end of its prompt -> it samples
    assert eng.log[2] == [(b, 1, [0]), (a, 2, [1])]
    for st in eng.log:
        assert sum(n for _, n, _ in st) <= 10
    assert s.finished[a].generated == [15, 16, 17] and s.finished[b].generated == [9, 10, 11, 12, 13]


def test_first_come_first_served_and_max_seqs():
    eng = FakeEngine(num_pages=64)
    s = Scheduler(eng, max_step_tokens=100, max_seqs=2)
    ids = [s.add_request([i + 1], SamplingParams(max_new_tokens=2, **GREEDY)) for i in range(4)]
    s.step()
    assert [r.id for r in s.running] == ids[:2] and [r.id for r in s.waiting] == ids[2:]
    s.run()
    order = [rid for st in eng.log for rid, _, _ in st]
    assert order.index(ids[2]) > order.index(ids[1])
    assert all(s.finished[i].generated == [i + 2, i + 3] for i in range(4))


def test_eos_is_neither_stored_nor_counted():
    eng = FakeEngine(num_pages=16)
    s = Scheduler(eng, max_step_tokens=32, eos_token_ids=(8,))
    a = s.add_request([5], SamplingParams(temperature=0.0, max_new_tokens=10))
    b = s.add_request([5], SamplingParams(temperature=0.0, max_new_tokens=10, ignore_eos=True))
    c = s.add_request([5], SamplingParams(temperature=0.0, max_new_tokens=10, stop_token_ids=(7,)))
    s.run()
    assert s.finished[a].generated == [6, 7] and s.finished[a].finish_reason == "eos"
    assert len(s.finished[b].generated) == 10
    assert s.finished[c].generated == [6]


def test_admission_waits_for_pages():
    eng = FakeEngine(num_pages=4, page_size=4)          # 16 tokens of cache
    s = Scheduler(eng, max_step_tokens=64)
    a = s.add_request(list(range(1, 11)), SamplingParams(max_new_tokens=2, **GREEDY))  # 3 pages
    b = s.add_request(list(range(1, 9)), SamplingParams(max_new_tokens=2, **GREEDY))   # 2 pages
    s.step()
    assert [r.id for r in s.running] == [a] and [r.id for r in s.waiting] == [b]
    s.run()
    assert s.n_preemptions == 0
    assert s.finished[a].generated == [11, 12] and s.finished[b].generated == [9, 10]


def test_out_of_pages_preempts_the_newest_and_recomputes():
    eng = FakeEngine(num_pages=4, page_size=4)
    s = Scheduler(eng, max_step_tokens=64)
    a = s.add_request([1, 2, 3, 4, 5, 6, 7], SamplingParams(max_new_tokens=6, **GREEDY))
    b = s.add_request([21, 22, 23, 24, 25, 26, 27], SamplingParams(max_new_tokens=6, **GREEDY))
    s.run()
    assert s.n_preemptions >= 1 and s.finished[b].preemptions >= 1 and s.finished[a].preemptions == 0
    assert s.finished[a].generated == [8, 9, 10, 11, 12, 13]
    assert s.finished[b].generated == [28, 29, 30, 31, 32, 33]     # unchanged by the preemption
    # after the preemption b came back with prompt + generated as one portion
    recompute = [st for st in eng.log if any(rid == b and n > 7 for rid, n, _ in st)]
    assert recompute, "b must have recomputed its prompt and generated tokens"
    assert eng.cache.num_free_pages() == [4]


def test_a_request_that_cannot_fit_alone():
    """A prompt larger than the whole pool is rejected when it is added; a request that is
    alone and outgrows the pool while decoding ends with what it has."""
    eng = FakeEngine(num_pages=2, page_size=4)
    s = Scheduler(eng, max_step_tokens=64)
    rid = s.add_request(list(range(1, 12)), SamplingParams(max_new_tokens=2, **GREEDY))
    out = s.run()
    assert out[rid].finish_reason == "rejected" and "CacheFull" in out[rid].error
    assert out[rid].generated == [] and eng.log == []
    eng2 = FakeEngine(num_pages=2, page_size=4)
    s2 = Scheduler(eng2, max_step_tokens=64)
    rid = s2.add_request([1, 2, 3, 4, 5, 6, 7], SamplingParams(max_new_tokens=5, **GREEDY))
    out = s2.run()                                   # grows beyond the pool while decoding
    assert out[rid].finish_reason == "cache" and out[rid].generated == [8, 9]
    assert eng2.cache.num_free_pages() == [2] and not eng2.cache.requests
    eng2.cache.check()


def test_a_bad_request_among_good_ones_is_rejected_alone():
    """A token id beyond the vocabulary, a prompt beyond the position table, an empty prompt:
    each finishes as "rejected" when it is added, is handed back by the next step, and the
    requests around it run as if it had never come."""
    eng = FakeEngine(num_pages=64)
    eng.model.spec.max_positions = 40
    s = Scheduler(eng, max_step_tokens=16, chunk_size=8)
    good1 = s.add_request([3, 4, 5], SamplingParams(max_new_tokens=3, **GREEDY))
    bad_token = s.add_request([3, V, 5], SamplingParams(max_new_tokens=3, **GREEDY))
    negative = s.add_request([3, -1], SamplingParams(max_new_tokens=3, **GREEDY))
    too_long = s.add_request(list(range(1, 42)), SamplingParams(max_new_tokens=3, **GREEDY))
    empty = s.add_request([], SamplingParams(max_new_tokens=3, **GREEDY))
    good2 = s.add_request([20, 21], SamplingParams(max_new_tokens=2, **GREEDY))
    first = s.step()
    assert {r.id for r in first} >= {bad_token, negative, too_long, empty}
    out = s.run()
    assert out[good1].generated == [6, 7, 8] and out[good2].generated == [22, 23]
    for rid, needle in ((bad_token, "TokenIdOutOfBounds"), (negative, "TokenIdOutOfBounds"),
                        (too_long, "PositionOutOfBounds"), (empty, "EmptyPrompt")):
        assert out[rid].finish_reason == "rejected" and needle in out[rid].error
        assert out[rid].generated == []
    seen = {rid for st in eng.log for rid, _, _ in st}
    assert seen == {good1, good2}
    assert eng.cache.num_free_pages() == [64] and not eng.cache.requests


def test_a_request_id_in_use_is_refused():
    from zinfer_amd.errors import StepError
    eng = FakeEngine(num_pages=16)
    s = Scheduler(eng, max_step_tokens=16)
    s.add_request([1, 2], SamplingParams(max_new_tokens=2, **GREEDY), request_id="x")
    with pytest.raises(StepError, match="already in use"):
        s.add_request([3], request_id="x")                   # waiting
    s.step()
    with pytest.raises(StepError, match="already in use"):
        s.add_request([3], request_id="x")                   # running
    s.run()
    assert s.finished["x"].generated == [3, 4]
    # finished: the id is free again, the old record goes, nothing of it is carried over
    s.add_request([7], SamplingParams(max_new_tokens=3, **GREEDY), request_id="x")
    assert "x" not in s.finished
    s.run()
    assert s.finished["x"].prompt == [7] and s.finished["x"].generated == [8, 9, 10]
    # a rejected request is finished at once; until step() has handed it back its id is taken
    s.add_request([], request_id="y")
    with pytest.raises(StepError, match="already in use"):
        s.add_request([1], request_id="y")
    s.run()
    s.add_request([1], SamplingParams(max_new_tokens=1, **GREEDY), request_id="y")
    s.run()
    assert s.finished["y"].generated == [2]
    # the caller takes finished requests out; nothing is kept for ever
    assert s.pop_finished("x").generated == [8, 9, 10] and "x" not in s.finished
    assert set(s.pop_finished()) == {"y"} and s.finished == {}
    with pytest.raises(KeyError):
        s.pop_finished("x")
    eng.cache.check()


def test_sampled_output_does_not_depend_on_the_batch():
    def run(n_others):
        eng = FakeEngine(num_pages=64)
        # flat logits: the random stream alone decides
        eng.step_orig = eng.step

        def flat(entries, end=()):
            out = eng.step_orig(entries, end)
            return torch.zeros_like(out)
        eng.step = flat
        s = Scheduler(eng, max_step_tokens=64)
        rid = s.add_request([1, 2], SamplingParams(temperature=1.0, seed=9, max_new_tokens=8,
                                                   ignore_eos=True))
        for i in range(n_others):
            s.add_request([3 + i], SamplingParams(temperature=1.0, seed=9, max_new_tokens=5,
                                                  ignore_eos=True))
        return s.run()[rid].generated
    assert run(0) == run(3)
    assert len(set(run(0))) > 1


class FakeGraphEngine(FakeEngine):
    """A stand-in whose decode steps may run several in a row (as the engine's graph replays)."""
    use_graphs = True

    def __init__(self, *args, **kw):
        super().__init__(*args, **kw)
        self.runs = []

    def decode_steps(self, entries, n_steps, records=None):
        assert all(len(e.tokens) == 1 for e in entries)
        self.runs.append((len(entries), n_steps, records is not None))
        lens = [(e.request_id, self.cache.length(e.request_id) + n_steps) for e in entries]
        assert self.cache.can_reserve(lens)
        for rid, n in lens:
            self.cache.reserve(rid, n)
            self.cache.commit(rid, n)
        self.cache.check()
        cur = [e.tokens[0] for e in entries]
        out = []
        for _ in range(n_steps):
            cur = [(t + 1) % V for t in cur]
            out.append(cur)
        return out


def test_decode_steps_in_a_row_only_when_everyone_decodes_and_nobody_waits():
    eng = FakeGraphEngine(num_pages=64)
    s = Scheduler(eng, max_step_tokens=8, chunk_size=8, multi_step=4)
    a = s.add_request([1, 2, 3], SamplingParams(max_new_tokens=11, **GREEDY))
    b = s.add_request(list(range(10, 22)), SamplingParams(max_new_tokens=7, **GREEDY))
    out = s.run()
    assert out[a].generated == list(range(4, 15)) and out[b].generated == list(range(22, 29))
    # while b is still in its prompt every step goes through the host; afterwards runs of at
    # most 4, never beyond what a request may still generate
    assert eng.runs and all(n <= 4 for _, n, _ in eng.runs)
    assert not any(len(st) == 2 and all(n == 1 for _, n, _ in st) for st in eng.log[3:])
    assert eng.cache.num_free_pages() == [64] and not eng.cache.requests
    assert s.n_steps == len(eng.log) + sum(n for _, n, _ in eng.runs)


def test_decode_steps_in_a_row_stop_at_eos_and_discard_the_rest():
    eng = FakeGraphEngine(num_pages=64)
    s = Scheduler(eng, max_step_tokens=8, multi_step=8, eos_token_ids=(9,))
    a = s.add_request([3], SamplingParams(temperature=0.0, max_new_tokens=30))
    b = s.add_request([20], SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True))
    out = s.run()
    assert out[a].generated == [4, 5, 6, 7, 8] and out[a].finish_reason == "eos"
    assert out[b].generated == list(range(21, 33)) and out[b].finish_reason == "length"
    assert eng.cache.num_free_pages() == [64]


def test_decode_steps_in_a_row_shrink_to_the_free_pages_and_skip_penalties():
    eng = FakeGraphEngine(num_pages=4, page_size=4)
    s = Scheduler(eng, max_step_tokens=8, multi_step=8)
    a = s.add_request([1, 2], SamplingParams(max_new_tokens=14, **GREEDY))
    out = s.run()
    assert out[a].generated == list(range(3, 17))
    assert all(n <= 8 for _, n, _ in eng.runs) and s.n_preemptions == 0
    # penalties need the tokens on the host after every step
    eng = FakeGraphEngine(num_pages=16)
    s = Scheduler(eng, max_step_tokens=8, multi_step=8)
    s.add_request([1, 2], SamplingParams(temperature=0.0, repetition_penalty=1.2,
                                         max_new_tokens=6, ignore_eos=True))
    s.run()
    assert not eng.runs


def test_abort_gives_everything_back():
    eng = FakeEngine(num_pages=16)
    s = Scheduler(eng, max_step_tokens=8, max_seqs=1)
    a = s.add_request([1, 2, 3], SamplingParams(max_new_tokens=50, **GREEDY))
    b = s.add_request([7, 8], SamplingParams(max_new_tokens=4, **GREEDY))      # waits: one slot
    s.step(); s.step()
    assert s.request(a).generated == [4, 5] and s.request(b) in s.waiting
    s.abort(b, "stop")                       # from the waiting queue
    req = s.abort(a, "stop")                 # while running
    assert req.finished and req.finish_reason == "stop" and req.generated == [4, 5]
    assert not s.has_work() and eng.cache.num_free_pages() == [16] and not eng.cache.requests
    assert s.abort(a) is req                 # once more: nothing happens
    with pytest.raises(KeyError):
        s.request("nobody")
