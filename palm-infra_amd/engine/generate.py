"""The generation loop above the step function.

The reference generates for one sequence: reset, ``prefill`` (which yields the first token), then
``decode`` until the stop token or ``max_new_tokens``; the stop token is part of the output; time is
split into prefill and decode (examples/cli_common.cpp:438-530) and the metrics are
``decode_tokens = generated - 1``, ``ttft = prefill_ms``, ``tpot = decode_ms / decode_tokens``,
``prefill_tps``, ``decode_tps`` (examples/cli_common.cpp:418-436).  Here the same loop runs over
batches of requests with unequal prompts: all prompts of a batch in one step, then one token for each
sequence that is still running; a sequence that ends leaves the batch at once and its slot goes back;
batches follow one another until every request is served.

Where the engine takes tokens that are still on the device (``takes_fed``) and the sampler's draw does not depend
on earlier draws (no penalties), the loop runs one step ahead of itself: it launches step t+1 with the tokens
that step t's sampling left on the device, and only then looks at step t's tokens, while the device is busy.  What
can end a sequence without knowing its newest token (the lengths) is decided before the launch; a stop token shows
one step late, and the one draw made for that sequence meanwhile is dropped.  The results are the same as
without; the host's work between two steps no longer leaves the device idle.

The loop only decides; the engine steps and the sampler chooses.  Both are handed in, so the decisions
can be tested with stand-ins.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field

from ..cache.pool import PAGE_TOKENS, pages_for
from ..sampling import SequenceSampling
from .engine import FedTokens, StepEntry


class TokenFetch:
    """A step's drawn tokens on their way to the host: asked for at once (so that the copy stands before the next
    step in the device's queue), looked at later."""

    def __init__(self, ids):
        self.ids, self.host, self.event = ids, None, None
        if getattr(ids, "is_cuda", False):
            import torch
            self.host = torch.empty(ids.shape, dtype=ids.dtype, pin_memory=True)
            self.host.copy_(ids, non_blocking=True)
            self.event = torch.cuda.Event()
            self.event.record()

    def tokens(self) -> list:
        if self.event is None:
            return self.ids.tolist()
        self.event.synchronize()
        return self.host.tolist()


@dataclass
class GenerationResult:
    """Of one request.  ``finish_reason``: "stop" (a stop token came, and is the last token), "length"
    (max_new_tokens), "context" (the sequence filled the longest context the cache takes)."""
    prompt_tokens: int
    token_ids: list = field(default_factory=list)
    finish_reason: str = ""
    prefill_ms: float = 0.0
    decode_ms: float = 0.0

    @property
    def hit_eos(self) -> bool:
        return self.finish_reason == "stop"


@dataclass
class GenerationMetrics:
    prompt_tokens: int = 0
    generated_tokens: int = 0
    decode_tokens: int = 0
    ttft_ms: float = 0.0
    tpot_ms: float = 0.0
    prefill_tps: float = 0.0
    decode_tps: float = 0.0
    total_ms: float = 0.0


def compute_metrics(results, prefill_ms: float, decode_ms: float) -> GenerationMetrics:
    """The reference's definitions (examples/cli_common.cpp:418-436), summed over the requests of a run:
    every request's first token comes from the prefill, the others from decode steps."""
    m = GenerationMetrics()
    m.prompt_tokens = sum(r.prompt_tokens for r in results)
    m.generated_tokens = sum(len(r.token_ids) for r in results)
    m.decode_tokens = sum(max(len(r.token_ids) - 1, 0) for r in results)
    m.ttft_ms = prefill_ms
    m.tpot_ms = decode_ms / m.decode_tokens if m.decode_tokens > 0 and decode_ms > 0 else 0.0
    m.prefill_tps = 1000.0 * m.prompt_tokens / prefill_ms if prefill_ms > 0 else 0.0
    m.decode_tps = 1000.0 * m.decode_tokens / decode_ms if decode_ms > 0 else 0.0
    m.total_ms = prefill_ms + decode_ms
    return m


class RequestTooLong(ValueError):
    pass


def plan_batches(prompt_lengths, max_new_tokens: int, max_batch: int, cache_tokens: int, max_seq_tokens: int):
    """Which requests run together: in the order given, as many as ``max_batch`` allows and as the cache
    can hold when every sequence of the batch grows to its full length (pages of PAGE_TOKENS each).
    Returns lists of request indices."""
    if max_batch < 1:
        raise ValueError("max_batch must be at least 1")
    batches, current, held = [], [], 0
    for i, n in enumerate(prompt_lengths):
        if n < 1:
            raise RequestTooLong(f"request {i}: the prompt is empty")
        if n > max_seq_tokens:
            raise RequestTooLong(f"request {i}: a prompt of {n} tokens exceeds the longest sequence the cache takes "
                                 f"({max_seq_tokens})")
        full = min(n + max_new_tokens, max_seq_tokens)
        need = pages_for(full) * PAGE_TOKENS
        if need > cache_tokens:
            raise RequestTooLong(f"request {i}: {full} tokens do not fit a cache of {cache_tokens}")
        if current and (len(current) >= max_batch or held + need > cache_tokens):
            batches.append(current)
            current, held = [], 0
        current.append(i)
        held += need
    if current:
        batches.append(current)
    return batches


def generate(engine, sampler, prompts, max_new_tokens: int = 2048, stop_token_ids=(), max_batch: int = 64,
             on_token=None, timer=time.perf_counter, sync=None):
    """Generate for every prompt (a list of token ids); results come in the order of the prompts.

    ``engine``: ``open() -> slot``, ``close(slot)``, ``step(entries) -> logits [rows, vocab]``,
    ``cache.max_tokens``, ``cache.max_seq_tokens``.  ``sampler``: ``sample(logits, states) -> ids`` (anything
    with ``.tolist()``).  ``on_token(request index, token id)`` is called for every token as it comes.
    ``sync()`` waits for the device before a time is taken.  Returns (results, metrics).
    """
    if max_new_tokens < 1:
        raise ValueError("max_new_tokens must be >= 1")
    prompts = [list(map(int, p)) for p in prompts]
    stop = set(int(t) for t in stop_token_ids)
    max_seq = engine.cache.max_seq_tokens
    results = [GenerationResult(prompt_tokens=len(p)) for p in prompts]
    # a batch holds no more sequences than the cache has slots for
    max_batch = min(max_batch, getattr(engine.cache, "max_seqs", max_batch))
    batches = plan_batches([len(p) for p in prompts], max_new_tokens, max_batch, engine.cache.max_tokens, max_seq)
    sync = sync or (lambda: None)
    total_prefill = total_decode = 0.0

    for batch in batches:
        slots = {}
        states = {i: SequenceSampling(stream=i) for i in batch}
        try:
            for i in batch:                  # one by one inside the try: if a slot cannot be had, those taken go back
                slots[i] = engine.open()
            # ---- all prompts in one step; it yields each request's first token ----
            sync()
            t0 = timer()
            logits = engine.step([StepEntry(slots[i], prompts[i], [len(prompts[i]) - 1]) for i in batch])
            for i in batch:
                states[i].accept(prompts[i])
            tokens = sampler.sample(logits, [states[i] for i in batch]).tolist()
            sync()
            prefill_ms = (timer() - t0) * 1000.0
            total_prefill += prefill_ms

            def take(i, tok):
                """Record a token; True if the sequence goes on."""
                r = results[i]
                r.token_ids.append(tok)
                if on_token:
                    on_token(i, tok)
                if tok in stop:
                    r.finish_reason = "stop"
                elif len(r.token_ids) >= max_new_tokens:
                    r.finish_reason = "length"
                elif len(prompts[i]) + len(r.token_ids) > max_seq:
                    # the next step would have to hold one token more than the cache takes
                    r.finish_reason = "context"
                if r.finish_reason:
                    engine.close(slots.pop(i))
                    return False
                return True

            live = []
            for i, tok in zip(batch, tokens):
                results[i].prefill_ms = prefill_ms
                if take(i, int(tok)):
                    live.append(i)

            # ---- one token for each sequence that still runs ----
            t1 = timer()
            if live and getattr(engine, "takes_fed", False) and not getattr(sampler, "needs_history", True):
                def goes_on(i, n):
                    """Whether request i runs on after its n-th token if that is no stop token (as take decides)."""
                    return n < max_new_tokens and len(prompts[i]) + n <= max_seq

                logits = engine.step([StepEntry(slots[i], [results[i].token_ids[-1]], [0]) for i in live])
                for i in live:
                    states[i].accept([results[i].token_ids[-1]])
                pending = TokenFetch(sampler.sample(logits, [states[i] for i in live]))
                order = [(i, row) for row, i in enumerate(live)]        # whose newest token is which row of `pending`
                while order:
                    ahead = [(i, row) for i, row in order if goes_on(i, len(results[i].token_ids) + 1)]
                    following = None
                    if ahead:
                        logits = engine.step([StepEntry(slots[i], [0], [0]) for i, _ in ahead],
                                             fed=FedTokens(pending.ids, [row for _, row in ahead]))
                        following = TokenFetch(sampler.sample(logits, [states[i] for i, _ in ahead]))
                    toks = pending.tokens()                              # the device runs the next step meanwhile
                    alive = set()
                    for i, row in order:
                        states[i].accept([int(toks[row])])
                        if take(i, int(toks[row])):
                            alive.add(i)
                    # a sequence that ended on a stop token was stepped once more: its draw is dropped with it
                    order = [(i, row) for row, (i, _) in enumerate(ahead) if i in alive]
                    pending = following
                live = []
            while live:
                last = {i: results[i].token_ids[-1] for i in live}
                logits = engine.step([StepEntry(slots[i], [last[i]], [0]) for i in live])
                for i in live:
                    states[i].accept([last[i]])
                tokens = sampler.sample(logits, [states[i] for i in live]).tolist()
                live = [i for i, tok in zip(live, tokens) if take(i, int(tok))]
            sync()
            decode_ms = (timer() - t1) * 1000.0
            total_decode += decode_ms
            for i in batch:
                results[i].decode_ms = decode_ms
        finally:
            for slot in slots.values():      # only after a fault: every sequence that ended has left already
                engine.close(slot)
    return results, compute_metrics(results, total_prefill, total_decode)


class Conversation:
    """One sequence kept alive from turn to turn: a turn feeds only its new tokens on top of what the cache holds
    and generates until a stop token, ``max_new_tokens`` or the cache's end, as the reference's chat loop does with
    its ``cached_token_ids`` (examples/main.cpp:394-466).  ``reset()`` gives the slot back (the loop's ``/reset``).

    ``engine`` and ``sampler`` as for ``generate``.  The tokens a turn generates are part of the sequence; the
    last one of a turn (a stop token, or the token at which the turn's length ran out) was chosen but not yet fed
    to the model, and goes in front of the next turn's tokens."""

    def __init__(self, engine, sampler, stop_token_ids=()):
        self.engine, self.sampler = engine, sampler
        self.stop = set(int(t) for t in stop_token_ids)
        self.slot = None
        self.state = SequenceSampling(stream=0)
        self.pending: list[int] = []          # chosen but not yet fed: they go in front of the next turn's tokens

    @property
    def length(self) -> int:
        """Tokens the cache holds for this conversation."""
        return 0 if self.slot is None else self.engine.length(self.slot)

    def reset(self) -> None:
        if self.slot is not None:
            self.engine.close(self.slot)
        self.slot = None
        self.pending = []
        self.state.reset()

    def say(self, tokens, max_new_tokens: int = 2048, on_token=None) -> GenerationResult:
        """Feed ``tokens`` (at least one, unless a token of the last turn is still pending) and generate."""
        if max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")
        feed = self.pending + [int(t) for t in tokens]
        if not feed:
            raise ValueError("a turn needs at least one token")
        max_seq = self.engine.cache.max_seq_tokens
        if self.length + len(feed) > max_seq:
            raise RequestTooLong(f"the conversation holds {self.length} tokens; {len(feed)} more exceed the longest "
                                 f"sequence the cache takes ({max_seq})")
        if self.slot is None:
            self.slot = self.engine.open()
        result = GenerationResult(prompt_tokens=len(feed))
        logits = self.engine.step([StepEntry(self.slot, feed, [len(feed) - 1])])
        self.pending = []
        self.state.accept(feed)
        while True:
            tok = int(self.sampler.sample(logits, [self.state]).tolist()[0])
            result.token_ids.append(tok)
            if on_token:
                on_token(0, tok)
            if tok in self.stop:
                result.finish_reason = "stop"
            elif len(result.token_ids) >= max_new_tokens:
                result.finish_reason = "length"
            elif self.length + 1 > max_seq:
                result.finish_reason = "context"
            if result.finish_reason:
                self.pending = [tok]          # the model has not seen it yet
                return result
            logits = self.engine.step([StepEntry(self.slot, [tok], [0])])
            self.state.accept([tok])
