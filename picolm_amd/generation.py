"""The generation loop: prompts in one step, then sample / record / stop? / one more token
(picolm/picolm.c:1502-1610), over batches of unequal prompts.

Differences from picolm's loop, all deliberate: exactly `max_new_tokens` tokens are produced
(picolm's bound runs one over, picolm/picolm.c:1496-1500, :1539); a stop token is recorded
and ends its sequence (picolm/picolm.c:1574); a sequence also ends at the cache's capacity;
sequences that end leave the batch and the others go on unchanged; when all of a batch have
ended its slots are released and the next batch starts in them.

The loop only decides; it never looks inside logits.  `stepper` needs begin(n) -> slots,
step(slots, tokens) -> logits rows, release(slots), `capacity` (longest sequence) and
fits(lengths) -> bool; `make_sampler(n)` returns an object with sample(logits, indices).

A stepper with step_ahead(slots, tokens on the device) and a sampler with launch(logits,
indices) -> pending tokens (on_device(rows), wait()) are driven one step ahead: the next step is
handed to the GPU before this step's tokens have reached the host, so that the GPU does not
stand still while the host decides.  The decisions and the tokens are the same; a sequence that
a stop token ends has by then been stepped once more, and that step's token is dropped.
"""
from __future__ import annotations

import os

import time
from dataclasses import dataclass, field

from .sampling.params import SamplingParams


@dataclass
class Generated:
    tokens: list = field(default_factory=list)
    finish: str = ""          # "stop", "length" or "capacity"


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    prefill_seconds: float = 0.0
    generated_tokens: int = 0
    decode_seconds: float = 0.0
    batches: int = 0
    steps: int = 0


class GenerationLoop:
    def __init__(self, stepper, make_sampler, stop_ids=(), batch_size: int = 64, clock=time.perf_counter,
                 sync=None):
        self.stepper = stepper
        self.make_sampler = make_sampler
        self.stop_ids = frozenset(int(s) for s in stop_ids)
        self.batch_size = max(1, int(batch_size))
        self.clock = clock
        self.sync = sync or (lambda: None)
        self.stats = GenerationStats()

    def _admit(self, prompts, first: int, max_new_tokens: int) -> int:
        """How many requests from `first` on form the next batch."""
        n = 0
        lengths = []
        while first + n < len(prompts) and n < self.batch_size:
            need = min(len(prompts[first + n]) + max_new_tokens, self.stepper.capacity)
            if not self.stepper.fits(lengths + [need]):
                break
            lengths.append(need)
            n += 1
        if n == 0:
            raise ValueError(f"request {first} ({len(prompts[first])} prompt tokens, {max_new_tokens} new) "
                             "does not fit the cache even alone")
        return n

    def run(self, prompts, max_new_tokens: int, on_token=None) -> list[Generated]:
        for i, p in enumerate(prompts):
            if len(p) == 0:
                raise ValueError(f"request {i} has an empty prompt; give at least a start token")
            if len(p) > self.stepper.capacity:
                raise ValueError(f"request {i} has {len(p)} prompt tokens, the cache takes {self.stepper.capacity}")
        results = [Generated() for _ in prompts]
        sampler = self.make_sampler(len(prompts))
        first = 0
        while first < len(prompts):
            n = self._admit(prompts, first, max_new_tokens)
            self._run_batch(prompts, list(range(first, first + n)), results, sampler, max_new_tokens, on_token)
            first += n
            self.stats.batches += 1
        return results

    def _run_batch(self, prompts, ids, results, sampler, max_new_tokens, on_token) -> None:
        st = self.stepper
        slots = st.begin(len(ids))
        slot_of = dict(zip(ids, slots))
        length = {i: len(prompts[i]) for i in ids}
        try:
            if max_new_tokens <= 0:
                for i in ids:
                    results[i].finish = "length"
                return
            t0 = self.clock()
            logits = st.step(slots, [list(prompts[i]) for i in ids])
            self.sync()
            self.stats.prefill_seconds += self.clock() - t0
            self.stats.prompt_tokens += sum(length.values())
            self.stats.steps += 1
            live = list(ids)
            t0 = self.clock()
            if hasattr(st, "step_ahead") and hasattr(sampler, "launch"):
                self._decode_one_ahead(sampler, logits, live, slot_of, length, results, max_new_tokens, on_token)
                live = []
            while live:
                tokens = sampler.sample(logits, live)
                nxt = []
                for i, tok in zip(live, tokens):
                    tok = int(tok)
                    results[i].tokens.append(tok)
                    self.stats.generated_tokens += 1
                    if on_token:
                        on_token(i, tok)
                    if tok in self.stop_ids:
                        results[i].finish = "stop"
                    elif len(results[i].tokens) >= max_new_tokens:
                        results[i].finish = "length"
                    elif length[i] + 1 > st.capacity:
                        results[i].finish = "capacity"
                    else:
                        nxt.append(i)
                # sequences that ended give their slots back at once; the rest go on
                ended = [i for i in live if i not in set(nxt)]
                if ended:
                    st.release([slot_of.pop(i) for i in ended])
                live = nxt
                if not live:
                    break
                logits = st.step([slot_of[i] for i in live], [[results[i].tokens[-1]] for i in live])
                self.stats.steps += 1
                for i in live:
                    length[i] += 1
            self.sync()
            self.stats.decode_seconds += self.clock() - t0
        finally:
            if slot_of:
                st.release(list(slot_of.values()))

    def _decode_one_ahead(self, sampler, logits, ids, slot_of, length, results, max_new_tokens, on_token) -> None:
        """The decode loop of `_run_batch` with the next step launched before this step's tokens
        are read.  Whether a sequence ends by its count of tokens or at the cache's capacity is
        known without its token; only a stop token is found out one step late."""
        st = self.stepper
        rows = list(ids)                   # the sequences that the pending tokens belong to, row by row
        pending = sampler.launch(logits, rows)
        ended = set()
        while rows:
            ahead = [i for i in rows if i not in ended and len(results[i].tokens) + 1 < max_new_tokens
                     and length[i] + 1 <= st.capacity]
            next_pending = None
            if ahead:
                pick = None if ahead == rows else [rows.index(i) for i in ahead]
                logits = st.step_ahead([slot_of[i] for i in ahead], pending.on_device(pick))
                self.stats.steps += 1
                for i in ahead:
                    length[i] += 1
                next_pending = sampler.launch(logits, ahead)
            goes_on = set(ahead)
            now_ended = []
            for i, tok in zip(rows, pending.wait()):
                if i in ended:             # stepped once more before its stop token was seen
                    continue
                tok = int(tok)
                results[i].tokens.append(tok)
                self.stats.generated_tokens += 1
                if on_token:
                    on_token(i, tok)
                if tok in self.stop_ids:
                    results[i].finish = "stop"
                elif i in goes_on:
                    continue
                else:
                    results[i].finish = "length" if len(results[i].tokens) >= max_new_tokens else "capacity"
                now_ended.append(i)
            if now_ended:
                # a step that is still running for one of these reads and writes that sequence's
                # own pages only, and whatever uses them next comes after it in the stream
                st.release([slot_of.pop(i) for i in now_ended])
                ended.update(now_ended)
            rows, pending = ahead, next_pending


# ---------------------------------------------------------------------------------------------
PREFILL_STEP_TOKENS = 16384        # most tokens of one prefill step: what sizes the step's workspace


def prefill_steps(lengths, budget: int = PREFILL_STEP_TOKENS, most: int = 0):
    """How a batch of prompts of these lengths goes through the model: a list of steps, each a list
    of (sequence, first token, count).  Prompts that fit the budget together are one step (picolm
    prefills a prompt in one call too, picolm/picolm.c:1502-1530).  Otherwise every step gives each
    unfinished sequence an equal share of the budget, in whole cache pages, and a sequence joins
    the later steps with what it has left, appended to what its slot already holds.  `most`: the
    most tokens a sequence may bring in one step (0: any number)."""
    lengths = [int(n) for n in lengths]
    if sum(lengths) <= budget and not (most and max(lengths, default=0) > most):
        return [[(i, 0, n) for i, n in enumerate(lengths)]]
    done = [0] * len(lengths)
    steps = []
    while any(d < n for d, n in zip(done, lengths)):
        left = [i for i, n in enumerate(lengths) if done[i] < n]
        share = max(64, budget // len(left) // 64 * 64)
        if most:
            share = min(share, most)
        step, room = [], max(budget, 64 * len(left))
        for i in left:
            take = min(lengths[i] - done[i], share, room)
            if take <= 0:
                continue
            step.append((i, done[i], take))
            done[i] += take
            room -= take
        steps.append(step)
    return steps


def generate(model_or_session, prompts, max_new_tokens: int = 256, params: SamplingParams | None = None,
             stop_ids=None, batch_size: int = 64, max_tokens: int | None = None, on_token=None,
             return_stats: bool = False, prefill_step_tokens: int = PREFILL_STEP_TOKENS, dtype: str = "bfloat16"):
    """The Python entry point: token ids in, generated token ids out.

    `model_or_session`: a model folder (loaded in `dtype`, as picolm's entry takes a file name,
    picolm/model.h:504), a loaded model (a session sized for the work is made) or a Session.
    `prompts`: a list of token-id lists.  `stop_ids`: default, the configuration's
    eos_token_id.  Returns one `Generated` per prompt (and the timing record on request).
    """
    import torch

    from .cache import PAGE_TOKENS, pages_for
    from .engine.session import Session
    from .sampling.sampler import Sampler
    params = params or SamplingParams()
    prompts = [list(p) for p in prompts]
    if isinstance(model_or_session, (str, os.PathLike)):
        from .engine import load_model
        model_or_session = load_model(os.fspath(model_or_session), dtype=dtype)
    if isinstance(model_or_session, Session):
        session = model_or_session
    else:
        if max_tokens is None:
            per = sorted((pages_for(len(p) + max_new_tokens) for p in prompts), reverse=True)
            max_tokens = max(1, sum(per[:batch_size])) * PAGE_TOKENS
        session = Session(model_or_session, max_tokens=max_tokens)
    if stop_ids is None:
        stop_ids = getattr(session.model.config, "eos_token_ids", ())
    device = session.model.runtime.device
    loop = GenerationLoop(SessionStepper(session, prefill_step_tokens), lambda n: Sampler(params, n, device), stop_ids, batch_size,
                          sync=lambda: torch.cuda.synchronize(device))
    out = loop.run(prompts, max_new_tokens, on_token)
    return (out, loop.stats) if return_stats else out


class SessionStepper:
    """The face of a Session that the loop needs."""

    def __init__(self, session, prefill_step_tokens: int = PREFILL_STEP_TOKENS):
        self.session = session
        self.capacity = session.cache.max_seq_len
        self.prefill_step_tokens = prefill_step_tokens

    def begin(self, n):
        return self.session.begin(n)

    def step(self, slots, tokens):
        """The last row's logits of every sequence.  Prompts beyond the budget of one step go in as
        several steps (`prefill_steps`); each sequence's row is kept from the step that ends it."""
        plan = prefill_steps([len(t) for t in tokens], self.prefill_step_tokens, self.session.most_new_tokens)
        if len(plan) == 1:
            return self.session.step(slots, tokens)
        import torch
        out = torch.empty((len(slots), self.session.vocab_size), dtype=torch.float32, device=self.session.model.runtime.device)
        for step in plan:
            ends = [i for i, first, count in step if first + count == len(tokens[i])]
            logits = self.session.step([slots[i] for i, _, _ in step], [tokens[i][first:first + count] for i, first, count in step],
                                       [[count - 1] if first + count == len(tokens[i]) else [] for i, first, count in step])
            if ends:
                out[torch.tensor(ends, device=out.device)] = logits
        return out

    def step_ahead(self, slots, tokens_on_device):
        return self.session.step_tokens_on_device(slots, tokens_on_device)

    def release(self, slots):
        self.session.release(slots)

    def fits(self, lengths) -> bool:
        from .cache import PAGE_TOKENS
        from .cache import pages_for
        c = self.session.cache
        if len(lengths) > c.slots.n_free:
            return False
        need = sum(pages_for(n) for n in lengths)
        return need * PAGE_TOKENS <= c.free_tokens()
