"""The generation loop's decisions with a stand-in engine and sampler (no GPU), and the
host side of the sampler."""
import pytest
import torch

import plain_llama as pl
from bitnet_c_amd.engine.generate import Request, generate, plan_batches
from bitnet_c_amd.sampling import SamplingParams, SequenceSampler, XorShift64Star


class FakeCache:
    def __init__(self, n_pages):
        self.n_pages = n_pages


class FakeEngine:
    """Logits whose argmax is (last token + 1) % vocab; records every step."""

    def __init__(self, vocab=50, max_seq_len=1000, n_pages=64):
        self.vocab, self.max_seq_len, self.cache = vocab, max_seq_len, FakeCache(n_pages)
        self.free, self.live, self.steps, self.released = list(range(100)), {}, [], []

    def new_sequence(self):
        s = self.free.pop(0)
        self.live[s] = 0
        return s

    def release(self, s):
        assert s in self.live, "released twice"
        del self.live[s]
        self.released.append(s)
        self.free.insert(0, s)

    def step(self, entries):
        self.steps.append([(e.slot, list(e.tokens)) for e in entries])
        rows = []
        for e in entries:
            assert e.slot in self.live
            self.live[e.slot] += len(e.tokens)
            for w in e.want:
                lg = torch.zeros(self.vocab)
                lg[(e.tokens[w] + 1) % self.vocab] = 1.0
                rows.append(lg)
        return torch.stack(rows) if rows else torch.zeros(0, self.vocab)


def greedy(logits, samplers):
    return [int(t) for t in logits.argmax(dim=1)]


def test_unequal_prompts_stop_tokens_and_early_ends():
    eng = FakeEngine()
    reqs = [Request([1, 2, 3], 5), Request([10], 2), Request([20, 21], 10, stop_ids=(24,)), Request([30], 0)]
    res = generate(eng, reqs, greedy, batch_size=8)
    assert res[0].tokens == [4, 5, 6, 7, 8] and res[0].finish == "length"
    assert res[1].tokens == [11, 12] and res[1].finish == "length"
    assert res[2].tokens == [22, 23] and res[2].finish == "stop"          # the stop token is not emitted
    assert res[3].tokens == [] and res[3].finish == "length"              # -n 0: the prompt only
    # one step for all prompts, then one token each for the live ones
    assert [len(s) for s in eng.steps] == [4, 3, 2, 1, 1]
    assert eng.steps[1] == [(0, [4]), (1, [11]), (2, [22])]
    # after the budget is reached no further step runs for that sequence
    assert sum(len(t) for st in eng.steps[1:] for _, t in st) == (5 - 1) + (2 - 1) + 2
    assert not eng.live and sorted(eng.released) == [0, 1, 2, 3]


def test_batches_one_after_another_reuse_slots():
    eng = FakeEngine(vocab=1000)
    reqs = [Request([100 + 10 * i], 1 + i % 3) for i in range(7)]     # prompts are multiples of 10, new tokens never
    res = generate(eng, reqs, greedy, batch_size=3)
    assert [r.tokens for r in res] == [[101 + 10 * i + k for k in range(1 + i % 3)] for i in range(7)]
    prompts = [[t[0] for _, t in s] for s in eng.steps if s[0][1][0] % 10 == 0]
    assert prompts == [[100, 110, 120], [130, 140, 150], [160]]           # as many batches as the requests need
    # a batch starts only when the one before it has ended
    starts = [k for k, s in enumerate(eng.steps) if s[0][1][0] % 10 == 0]
    assert starts == [0, 3, 6]
    assert max(max(sl for sl, _ in s) for s in eng.steps) <= 2             # three slots serve seven requests
    assert not eng.live


def test_batch_planning_respects_the_cache():
    reqs = [Request([0] * 100, 28), Request([0] * 10, 10), Request([0] * 200, 0), Request([0] * 5000, 1),
            Request([], 3), Request([0] * 60, 600)]
    batches, errors = plan_batches(reqs, batch_size=8, max_tokens=64 * 5, max_seq_len=1024)
    # needs (rounded to pages): 128, 64, 256, -, -, 704 > 320
    assert batches == [[0, 1], [2]] and set(errors) == {3, 4, 5}
    assert "sequence limit" in errors[3] and "empty" in errors[4] and "cache holds" in errors[5]
    b2, _ = plan_batches([Request([1], 1)] * 5, batch_size=2, max_tokens=10 ** 6, max_seq_len=100)
    assert b2 == [[0, 1], [2, 3], [4]]


def test_sequence_limit_and_cancel():
    eng = FakeEngine(max_seq_len=6)
    res = generate(eng, [Request([1, 2, 3, 4], 10)], greedy)
    assert res[0].finish == "limit" and res[0].tokens == [5, 6, 7]         # positions 4, 5 fed; the 7th has no room
    eng = FakeEngine()
    seen = []
    res = generate(eng, [Request([1], 10), Request([5], 3)], greedy, on_token=lambda i, t: seen.append((i, t)) or i == 0)
    assert res[0].tokens == [2] and res[0].finish == "cancelled"           # the callback stops after one token
    assert res[1].tokens == [6, 7, 8]
    assert (0, 2) in seen and not eng.live


def test_an_error_in_a_step_gives_the_slots_back():
    class Broken(FakeEngine):
        def step(self, entries):
            if len(self.steps) == 2:
                raise RuntimeError("boom")
            return super().step(entries)
    eng = Broken()
    with pytest.raises(RuntimeError):
        generate(eng, [Request([1], 5), Request([2], 5)], greedy)
    assert not eng.live


class AheadEngine(FakeEngine):
    """A stand-in that takes a decode step's tokens from a tensor, as the engine takes them from the device."""
    takes_device_tokens = True

    def __init__(self, *a, fail_ahead_at=None, **kw):
        super().__init__(*a, **kw)
        self.ahead_steps, self.fail_ahead_at = 0, fail_ahead_at

    def step(self, entries, device_tokens=None):
        if device_tokens is not None:
            from bitnet_c_amd.engine.step import StepError
            self.ahead_steps += 1
            if self.fail_ahead_at == self.ahead_steps:
                raise StepError("no page left")
            assert all(list(e.tokens) == [0] for e in entries) and device_tokens.shape == (len(entries),)
            entries = [type(e)(e.slot, [int(t)], e.want) for e, t in zip(entries, device_tokens)]
        return super().step(entries)


class _Pending:
    def __init__(self, toks):
        self.device_tokens = toks

    def rows(self, idx):
        return self.device_tokens[list(idx)]

    def tokens(self):
        return [int(t) for t in self.device_tokens]


def _greedy_ahead():
    def fn(logits, samplers):
        return greedy(logits, samplers)
    fn.start = lambda logits, samplers: _Pending(logits.argmax(dim=1).to(torch.int32))
    return fn


def _mixed_requests():
    return [Request([1, 2, 3], 5), Request([10], 2), Request([20, 21], 10, stop_ids=(24,)), Request([30], 0),
            Request([40], 1), Request([41, 42], 7, stop_ids=(43,)), Request([7], 9, stop_ids=(12, 3))]


@pytest.mark.parametrize("batch_size", [8, 3, 1])
def test_steps_queued_ahead_decide_the_same(batch_size):
    """With tokens that stay on the device a step is queued before the host has seen them: tokens, finish reasons and
    the slots' fate are those of the plain loop; a sequence that its token has ended ran one step for nothing."""
    a, b = FakeEngine(), AheadEngine()
    want = generate(a, _mixed_requests(), greedy, batch_size=batch_size)
    got = generate(b, _mixed_requests(), _greedy_ahead(), batch_size=batch_size)
    assert [(r.tokens, r.finish) for r in got] == [(r.tokens, r.finish) for r in want]
    assert not b.live and sorted(b.released) == sorted(a.released)
    assert b.ahead_steps > 0
    # the steps differ only by the rows of sequences that a stop token ended: those ran once more
    fed = lambda eng: sorted((sl, t[0]) for st in eng.steps for sl, t in st if len(t) == 1)
    extra = [x for x in fed(b) if x not in fed(a)]
    stopped = sum(r.finish == "stop" for r in want)
    assert len(fed(b)) - len(fed(a)) == len(extra) <= stopped
    # nothing ran for a sequence at its budget or at the limit: those are counts, known without the token
    eng = AheadEngine(max_seq_len=6)
    res = generate(eng, [Request([1, 2, 3, 4], 10)], _greedy_ahead())
    assert res[0].finish == "limit" and res[0].tokens == [5, 6, 7] and [len(s) for s in eng.steps] == [1, 1, 1]


def test_a_cancelling_callback_and_a_refused_step_under_queued_steps():
    eng = AheadEngine()
    seen = []
    res = generate(eng, [Request([1], 10), Request([5], 3)], _greedy_ahead(),
                   on_token=lambda i, t: seen.append((i, t)) or i == 0)
    assert res[0].tokens == [2] and res[0].finish == "cancelled" and res[1].tokens == [6, 7, 8]
    assert seen == [(0, 2), (1, 6), (1, 7), (1, 8)] and not eng.live
    # a step that the engine refuses when it is queued ahead changes nothing: the loop decides with the tokens at hand
    # and asks again the plain way
    eng = AheadEngine(fail_ahead_at=2)
    res = generate(eng, [Request([1], 6), Request([9], 4)], _greedy_ahead())
    assert res[0].tokens == [2, 3, 4, 5, 6, 7] and res[1].tokens == [10, 11, 12, 13] and not eng.live


def test_a_sampler_that_needs_the_host_first_is_asked_the_plain_way():
    fn = _greedy_ahead()
    fn.start = lambda logits, samplers: None
    eng = AheadEngine()
    res = generate(eng, [Request([1], 3)], fn)
    assert res[0].tokens == [2, 3, 4] and eng.ahead_steps == 0


def test_sampling_that_needs_the_host_first_says_so():
    """A repetition penalty reads the host's ring of recent tokens before it can sample: tokens cannot stay on the device."""
    from bitnet_c_amd.sampling import start_sampling
    logits = torch.zeros(2, 10)
    with_penalty = [SequenceSampler(SamplingParams(repeat_penalty=1.3), [1, 2]), SequenceSampler(SamplingParams(), [3])]
    assert start_sampling(logits, with_penalty) is None


def test_host_rng_and_recent_ring_follow_the_plain_sampler():
    a, b = XorShift64Star(0), pl.XorShift64Star(42)
    assert [a.next_float() for _ in range(50)] == [b.next_float() for _ in range(50)]
    s = SequenceSampler(SamplingParams(repeat_penalty=1.1, repeat_window=4), prompt=[1, 2, 3, 4, 5])
    s.accept(6)
    assert s.recent == [3, 4, 5, 6]
    off = SequenceSampler(SamplingParams(), prompt=[1, 2, 3])
    off.accept(9)
    assert off.recent == []
    with pytest.raises(ValueError):
        SamplingParams(temperature=-1.0)


def test_same_seed_same_stream_whatever_the_batch():
    # every sequence owns its generator: the k-th draw of a sequence is the same alone or among others
    def draws(n_partners):
        ss = [SequenceSampler(SamplingParams(temperature=0.8, seed=42 + i)) for i in range(1 + n_partners)]
        out = []
        for _ in range(5):
            vals = [s.rng.next_float() for s in ss]
            out.append(vals[0])
        return out
    assert draws(0) == draws(3)


def test_prompt_tiles_are_paired_long_with_short_inside_a_sequence():
    # The prompt attention gives a workgroup two consecutive tiles of the list: every tile appears once, a pair
    # belongs to one sequence and carries about the same number of keys as every other pair of that sequence, the
    # longest sequence comes first, and the odd ones out are paired with each other at the end.
    from bitnet_c_amd.ops import pair_tiles
    import random
    rnd = random.Random(3)
    for lens in ([2048], [130], [32], [700, 64, 2048, 33], [rnd.randint(1, 3000) for _ in range(9)]):
        qt, rows, r = 32, [], 0
        for s, n in enumerate(lens):
            p0 = 64 * s                                    # some sequences continue a cached prefix
            rows += [(s, r + i, min(qt, n - i), p0 + i) for i in range(0, n, qt)]
            r += n
        out = pair_tiles(list(rows))
        assert sorted(out) == sorted(rows)
        keys = lambda t: t[3] + t[2]
        n_paired = sum(len([t for t in rows if t[0] == s]) // 2 * 2 for s in range(len(lens)))
        first_seq = [t[0] for t in out[:n_paired:2]]
        assert first_seq == sorted(first_seq, key=lambda s: -max(keys(t) for t in rows if t[0] == s))
        for a, b in zip(out[:n_paired:2], out[1:n_paired:2]):
            assert a[0] == b[0] and keys(a) >= keys(b)
            mine = [t for t in rows if t[0] == a[0]]
            total = max(keys(t) for t in mine) + min(keys(t) for t in mine)
            assert abs(keys(a) + keys(b) - total) <= qt    # long + short: the same sum for every pair
        rest = out[n_paired:]
        assert len({t[0] for t in rest}) == len(rest)       # one middle tile per sequence with an odd count


def test_streamed_copies_take_what_the_cache_leaves():
    """The rule by which a model takes streamed copies of its weight matrices when nobody says: what is free once the
    weights and the cache are in place, but for a tenth of the device's memory."""
    from bitnet_c_amd.engine.model import streamed_budget
    GB = 1 << 30
    assert streamed_budget(250 * GB, 288 * GB) >= 16 * GB              # an 8B model with a cache of 20 GB: all of it
    assert 60 * GB <= streamed_budget(100 * GB, 288 * GB) <= 75 * GB   # 70B with a cache of 46 GB: most feed-forwards
    assert streamed_budget(20 * GB, 288 * GB) == 0                     # a device that the cache fills
    assert streamed_budget(0, 0) == 0
