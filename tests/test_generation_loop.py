"""The generation loop's decisions, driven by a scripted model (no GPU)."""
import pytest

from picolm_amd.generation import GenerationLoop


class ScriptedStepper:
    """Logits are just (request key, position): the scripted sampler turns them into tokens."""

    def __init__(self, n_slots=4, capacity=1000, page_budget=10 ** 9):
        self.capacity = capacity
        self.n_slots = n_slots
        self.free = list(range(n_slots))
        self.length = {}
        self.first_token = {}
        self.log = []
        self.page_budget = page_budget

    def fits(self, lengths):
        return len(lengths) <= len(self.free) and sum(lengths) <= self.page_budget

    def begin(self, n):
        assert n <= len(self.free)
        out = [self.free.pop(0) for _ in range(n)]
        for s in out:
            self.length[s] = 0
        self.log.append(("begin", tuple(out)))
        return out

    def step(self, slots, tokens):
        assert len(set(slots)) == len(slots)
        rows = []
        for s, t in zip(slots, tokens):
            assert s in self.length, "a step on a slot that is not live"
            if self.length[s] == 0:
                self.first_token[s] = t[0]
            else:
                assert len(t) == 1, "after the prompt a sequence brings one token"
            self.length[s] += len(t)
            assert self.length[s] <= self.capacity
            rows.append((self.first_token[s], self.length[s]))
        self.log.append(("step", tuple(slots), tuple(len(t) for t in tokens)))
        return rows

    def release(self, slots):
        for s in slots:
            assert s in self.length, "released twice"
            del self.length[s]
            self.free.append(s)
        self.log.append(("release", tuple(slots)))


class ScriptedSampler:
    """Request with first prompt token f emits f*100 + position; emits `stop` at stop_at[f]."""

    def __init__(self, stop_at=None, stop=9):
        self.stop_at = stop_at or {}
        self.stop = stop
        self.calls = []

    def sample(self, logits, indices):
        self.calls.append(list(indices))
        out = []
        for f, pos in logits:
            out.append(self.stop if self.stop_at.get(f) == pos else f * 100 + pos)
        return out


def run(prompts, max_new, stop_at=None, **kw):
    st = ScriptedStepper(**{k: v for k, v in kw.items() if k in ("n_slots", "capacity", "page_budget")})
    sm = ScriptedSampler(stop_at)
    loop = GenerationLoop(st, lambda n: sm, stop_ids=[9], batch_size=kw.get("batch_size", 64))
    return loop.run(prompts, max_new), st, sm, loop


def test_exactly_max_new_tokens_and_prompt_in_one_step():
    res, st, sm, loop = run([[1, 5, 5], [2]], 4)
    assert [r.tokens for r in res] == [[103, 104, 105, 106], [201, 202, 203, 204]]
    assert [r.finish for r in res] == ["length", "length"]
    steps = [e for e in st.log if e[0] == "step"]
    assert steps[0][2] == (3, 1)                      # unequal prompts, one step, no padding
    assert all(e[2] == (1, 1) for e in steps[1:])     # then one token each
    assert len(steps) == 4                            # the last sampled token is not fed back
    assert loop.stats.generated_tokens == 8 and loop.stats.prompt_tokens == 4


def test_stop_token_is_recorded_and_ends_only_its_sequence():
    res, st, sm, _ = run([[1, 0], [2, 0, 0], [3]], 6, stop_at={2: 4})
    assert res[1].tokens == [203, 9] and res[1].finish == "stop"
    assert len(res[0].tokens) == 6 and len(res[2].tokens) == 6
    assert res[0].tokens == [102 + i for i in range(6)]          # the others are unchanged
    steps = [e for e in st.log if e[0] == "step"]
    assert [len(e[1]) for e in steps] == [3, 3, 2, 2, 2, 2]      # the ended sequence left the batch
    rel = [e for e in st.log if e[0] == "release"]
    assert rel[0] == ("release", (1,))                           # and gave its slot back at once
    assert st.length == {}                                       # nothing is left live


def test_batches_follow_each_other_and_slots_are_used_again():
    prompts = [[i + 1] * (i + 1) for i in range(5)]
    res, st, sm, loop = run(prompts, 2, n_slots=2, batch_size=2)
    assert [r.tokens for r in res] == [[(i + 1) * 100 + (i + 1), (i + 1) * 100 + (i + 2)] for i in range(5)]
    begins = [e for e in st.log if e[0] == "begin"]
    assert [len(e[1]) for e in begins] == [2, 2, 1] and loop.stats.batches == 3
    assert begins[1][1] == begins[0][1] or set(begins[1][1]) == set(begins[0][1])   # the same slots again
    assert sm.calls[0] == [0, 1] and sm.calls[2] == [2, 3]       # sampler streams follow the request, not the slot


def test_admission_by_room_in_the_cache():
    res, st, sm, loop = run([[1] * 10, [2] * 10, [3] * 10], 5, page_budget=32)
    assert loop.stats.batches == 2 and all(len(r.tokens) == 5 for r in res)
    with pytest.raises(ValueError, match="does not fit"):
        run([[1] * 10], 5, page_budget=8)


def test_capacity_ends_a_sequence():
    res, st, sm, _ = run([[1] * 6, [2] * 2], 10, capacity=8)
    assert res[0].finish == "capacity" and len(res[0].tokens) == 3      # tokens at positions 6, 7 fed; the third only sampled
    assert res[1].finish == "capacity" and len(res[1].tokens) == 7


def test_bad_requests():
    with pytest.raises(ValueError, match="empty prompt"):
        run([[1], []], 3)
    with pytest.raises(ValueError, match="prompt tokens"):
        run([[1] * 20], 3, capacity=8)
    res, st, _, _ = run([[1, 2]], 0)
    assert res[0].tokens == [] and res[0].finish == "length" and st.length == {}


def test_a_failing_step_releases_the_batch():
    st = ScriptedStepper()
    boom = RuntimeError("device fault")

    def bad_step(slots, tokens):
        raise boom
    st.step = bad_step
    loop = GenerationLoop(st, lambda n: ScriptedSampler(), batch_size=4)
    with pytest.raises(RuntimeError):
        loop.run([[1], [2]], 3)
    assert st.length == {} and len(st.free) == 4


# -- one step ahead ---------------------------------------------------------------------------
class AheadStepper(ScriptedStepper):
    """Also takes the tokens of a step before the host has looked at them."""

    def step_ahead(self, slots, tokens_on_device):
        assert len(tokens_on_device) == len(slots)
        return self.step(slots, [[t] for t in tokens_on_device])


class _Pending:
    def __init__(self, tokens, sampler):
        self.tokens, self.sampler, self.waited = tokens, sampler, False

    def on_device(self, rows=None):
        return list(self.tokens) if rows is None else [self.tokens[r] for r in rows]

    def wait(self):
        assert not self.waited
        self.waited = True
        self.sampler.unread -= 1
        return list(self.tokens)


class AheadSampler(ScriptedSampler):
    def launch(self, logits, indices):
        self.unread = getattr(self, "unread", 0) + 1
        assert self.unread <= 2, "more than two draws whose tokens the host has not read"
        return _Pending(self.sample(logits, indices), self)


@pytest.mark.parametrize("case", range(40))
def test_one_step_ahead_decides_as_the_plain_loop(case):
    """Random requests, stops, limits and a small capacity: the loop that launches the next step
    before it reads this step's tokens produces the same tokens and endings, uses slots the same
    way, and steps a sequence at most once beyond its stop token."""
    import random
    rnd = random.Random(case)
    n = rnd.randint(1, 7)
    prompts = [[10 + i] + [5] * rnd.randint(0, 6) for i in range(n)]
    max_new = rnd.randint(1, 9)
    capacity = rnd.choice([8, 10, 1000])
    stop_at = {10 + i: len(prompts[i]) + rnd.randint(0, 8) for i in range(n) if rnd.random() < 0.6}
    kw = dict(n_slots=rnd.randint(1, 4), capacity=capacity, batch_size=rnd.randint(1, 4))
    plain, st0, sm0, loop0 = run(prompts, max_new, stop_at, **kw)
    st = AheadStepper(n_slots=kw["n_slots"], capacity=capacity)
    sm = AheadSampler(stop_at)
    loop = GenerationLoop(st, lambda k: sm, stop_ids=[9], batch_size=kw["batch_size"])
    ahead = loop.run(prompts, max_new)
    assert [(r.tokens, r.finish) for r in ahead] == [(r.tokens, r.finish) for r in plain]
    assert not st.length and sorted(st.free) == list(range(kw["n_slots"]))
    assert loop.stats.generated_tokens == loop0.stats.generated_tokens
    stopped = sum(r.finish == "stop" for r in plain)
    assert loop0.stats.steps <= loop.stats.steps
    tokens_stepped = lambda s: sum(sum(e[2]) for e in s.log if e[0] == "step")
    assert tokens_stepped(st0) <= tokens_stepped(st) <= tokens_stepped(st0) + stopped


def test_prompts_are_cut_into_steps_within_the_token_budget():
    from picolm_amd.generation import prefill_steps
    assert prefill_steps([10, 20, 30], 100) == [[(0, 0, 10), (1, 0, 20), (2, 0, 30)]]      # they fit: one step
    lens = [300, 50, 1000, 64, 1]
    steps = prefill_steps(lens, 512)
    seen = [0] * len(lens)
    for st in steps:
        assert sum(c for _, _, c in st) <= 512
        assert len({i for i, _, _ in st}) == len(st)                     # a sequence is in a step once
        for i, first, count in st:
            assert first == seen[i] and count > 0                        # each goes on where it stopped
            assert first % 64 == 0                                       # in whole pages until its end
            seen[i] += count
    assert seen == lens
    assert len(prefill_steps([100] * 40, 64)) == 2                       # more sequences than the budget has pages: a page each
    # a model whose steps take no more than 256 tokens of a sequence: further steps, also within the budget
    assert prefill_steps([10, 300, 600], 4096, most=256) == [[(0, 0, 10), (1, 0, 256), (2, 0, 256)], [(1, 256, 44), (2, 256, 256)],
                                                             [(2, 512, 88)]]
    assert prefill_steps([10, 200], 4096, most=256) == [[(0, 0, 10), (1, 0, 200)]]
