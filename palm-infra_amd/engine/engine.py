"""The engine: a model, its cache, and the one step function that everything above it uses.

The reference has two entry points for one sequence, ``prefill_chunk(ids, past)`` and ``decode(id)``
(engine/engine.cpp:1248-1381, 1383-1460): embed, rotation table, mask, graph, final norm, head on the
last row.  Here one ``step`` takes a batch of sequences, each with its next tokens (a whole prompt, a
piece of one, or a single token), runs only those tokens from what the cache holds, and returns the
logits at the places asked for.  Sequences are packed without padding, so a sequence's result cannot
depend on its companions' lengths.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from pathlib import Path

import numpy as np
import torch

from ..cache import ModelCache
from ..config import config_from_dict, config_from_dir
from ..kernels import profile
from ..parts import context_ints, make_context
from ..weights import ModelFiles, load_weights, random_weights
from .model import DecoderModel

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


class StepError(ValueError):
    """A step was asked for something that cannot run: a token outside the vocabulary, a slot that is
    not open, a place outside the tokens given."""


@dataclass
class StepEntry:
    """The next tokens of one sequence and the places among them whose logits are wanted."""
    slot: int
    tokens: list
    want: list = field(default_factory=list)


@dataclass
class FedTokens:
    """Tokens that an earlier step's sampling left on the device, for a step of single tokens that is launched
    before the host has seen them: the step's k-th sequence takes ``ids[rows[k]]``."""
    ids: torch.Tensor            # int32 [m] on the engine's device
    rows: list


def resolve_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype {dtype} is neither bfloat16 nor float32")
        return dtype
    if dtype not in DTYPES:
        raise ValueError(f"dtype {dtype!r} is not one of {sorted(DTYPES)}")
    return DTYPES[dtype]


class Engine:
    takes_fed = True             # step(entries, fed=..) takes tokens that are still on the device

    def __init__(self, config, spec, weights, dtype: torch.dtype, max_tokens: int, max_seqs: int | None = None,
                 device="cuda:0", graphs: bool = True, max_step_tokens: int = 32768):
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError(f"the engine runs on a GPU; device {device!r} was asked for and there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible to torch; the engine cannot run")
        torch.cuda.set_device(self.device)
        self.config, self.spec, self.dtype = config, spec, dtype
        self.model = DecoderModel(spec, weights, dtype, self.device)
        needs, shares = self.model.cache_plan()
        self.cache = ModelCache(needs, shares, max_tokens, max_seqs, spec.max_positions, dtype, self.device)
        self.vocab_size = spec.vocab_size
        self.graphs_enabled = bool(graphs)
        self._decode_graphs: dict = {}            # (batch bucket, length bucket) -> recorded step, least recently used first
        self._graph_pool_handle = None
        # a windowed group gives pages back only between steps, so long prompts go through it in pieces
        windows = [g.table.window for g in self.cache.paged_groups if g.table.window]
        self.step_tokens_per_seq = max(1024, 2 * max(windows)) if windows else None
        # the most tokens that run through the layers at once: longer steps go through in pieces, so that a step's
        # activations (the widest: tokens x twice the feed-forward width) stay within a few gigabytes
        if max_step_tokens < 1:
            raise ValueError(f"max_step_tokens = {max_step_tokens} must be positive")
        self.max_step_tokens = int(max_step_tokens)

    # ---- construction ------------------------------------------------------------------------
    @classmethod
    def from_dir(cls, model_dir, dtype="bfloat16", max_tokens: int | None = None, device="cuda:0",
                 strict_weights: bool = True, **options):
        """A folder with config.json and safetensors; the model class is chosen by config.json.  ``strict_weights``
        false: tensors of the checkpoint that the model does not name are listed on standard error and left alone
        instead of refused."""
        dt = resolve_dtype(dtype)
        model_dir = Path(model_dir)
        config = config_from_dir(model_dir)
        files = ModelFiles(model_dir)
        spec = config.spec(files.names())
        weights = load_weights(spec, files, dt, device, strict=strict_weights)
        return cls(config, spec, weights, dt, max_tokens or 16384, device=device, **options)

    @classmethod
    def from_config(cls, config, seed: int = 0, dtype="bfloat16", max_tokens: int | None = None, device="cuda:0",
                    **options):
        """Random weights made on the device (no folder is written)."""
        dt = resolve_dtype(dtype)
        if isinstance(config, dict):
            config = config_from_dict(config)
        spec = config.spec()
        weights = random_weights(spec, seed, dt, device)
        return cls(config, spec, weights, dt, max_tokens or 16384, device=device, **options)

    # ---- sequences ---------------------------------------------------------------------------
    def open(self) -> int:
        """A slot for a new sequence."""
        return self.cache.open()

    def close(self, slot: int) -> None:
        """The sequence is over: what it holds goes back."""
        self.cache.close(slot)

    def length(self, slot: int) -> int:
        return self.cache.lengths[slot]

    # ---- the step ----------------------------------------------------------------------------
    @staticmethod
    def _entry(e) -> StepEntry:
        """The entry with its tokens as an array of integers (a long prompt is checked and laid out by numpy, not
        token by token)."""
        if not isinstance(e, StepEntry):
            e = StepEntry(*e)
        try:
            tokens = np.asarray(e.tokens)
        except Exception as exc:
            raise StepError(f"slot {e.slot}: the tokens are no list of integers ({exc})") from None
        if tokens.ndim != 1 or (tokens.size and tokens.dtype.kind not in "iu"):
            raise StepError(f"slot {e.slot}: the tokens are no list of integers (they come as {tokens.dtype}, {tokens.ndim} axes)")
        return StepEntry(e.slot, tokens.astype(np.int64, copy=False), list(e.want))

    def _validate(self, entries) -> None:
        if not entries:
            raise StepError("a step needs at least one sequence")
        seen = set()
        for e in entries:
            if e.slot in seen:
                raise StepError(f"slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            if not self.cache.slots.is_held(e.slot):
                raise StepError(f"slot {e.slot} is not open")
            if len(e.tokens) == 0:
                raise StepError(f"slot {e.slot} brings no tokens")
            lo, hi = int(e.tokens.min()), int(e.tokens.max())
            if lo < 0 or hi >= self.vocab_size:
                raise StepError(f"token id {lo if lo < 0 else hi} lies outside the vocabulary of {self.vocab_size}")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise StepError(f"slot {e.slot}: logits wanted at place {w} of {len(e.tokens)} tokens")

    def step(self, entries, fed: FedTokens | None = None) -> torch.Tensor:
        """Run the entries' tokens as one batch from the cache; float32 logits [wanted, vocab] in the
        order of the entries and of each entry's ``want``.  Nothing changes if the step is refused.

        ``fed``: every entry brings one token, and which one is not known on the host yet: entry k's is
        ``fed.ids[fed.rows[k]]`` on the device (what its ``tokens`` holds is a stand-in).  The step is then launched
        without waiting for the device, so that a caller can look at one step's tokens while the next one runs.
        Fed tokens are meant to be a sampler's draws, which lie in the vocabulary; the host cannot look at them
        without waiting, so a recorded step takes them unchecked, and an id outside the table is not read from
        memory but makes that sequence's logits NaN (the embedding kernel's rule)."""
        entries = [self._entry(e) for e in entries]
        self._validate(entries)
        if fed is not None:
            return self._run_fed(entries, fed)
        per_seq, per_step = self.step_tokens_per_seq, self.max_step_tokens
        total = sum(len(e.tokens) for e in entries)
        if (per_seq is None or all(len(e.tokens) <= per_seq for e in entries)) and total <= per_step:
            return self._run(entries)
        # Pieces: a sequence's tokens go through in order, at most `per_seq` of them a step (a windowed group gives
        # pages back between steps) and at most `per_step` tokens of all sequences together (what bounds the memory
        # of a step's activations).  A sequence's result does not depend on how its tokens are cut.
        self.cache.check_room([(e.slot, len(e.tokens)) for e in entries], in_pieces=True)
        per_seq = per_seq or per_step
        fed = [0] * len(entries)
        results = {}
        while any(fed[i] < len(e.tokens) for i, e in enumerate(entries)):
            piece, back, room = [], [], per_step
            for i, e in enumerate(entries):
                if room == 0:
                    break
                n = min(len(e.tokens) - fed[i], per_seq, room)
                if n <= 0:
                    continue
                lo, hi = fed[i], fed[i] + n
                want = [w - lo for w in e.want if lo <= w < hi]
                piece.append(StepEntry(e.slot, e.tokens[lo:hi], want))
                back.extend((i, w + lo) for w in want)
                fed[i], room = hi, room - n
            logits = self._run(piece)
            for r, key in enumerate(back):
                results[key] = logits[r]
        rows = [results[(i, w)] for i, e in enumerate(entries) for w in e.want]
        if not rows:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        return torch.stack(rows)

    # ---- decode steps as HIP graphs -----------------------------------------------------------
    # A decode step is some hundred small kernels; launched one by one the host is the bottleneck.  For a
    # batch of single tokens the whole forward pass is recorded once into a HIP graph and replayed with
    # new contents in the same buffers.  A graph is keyed by the batch size, rounded up (rows that pad it
    # belong to a slot of their own and write into a page that is never read), and by the longest sequence,
    # rounded up to a power of two (it only sizes how attention cuts the key range).
    GRAPH_MAX_BATCH = 128        # as many rows as the products' own kernels take: a recorded step runs no library code

    @staticmethod
    def _batch_bucket(n: int) -> int:
        return n if n <= 8 else (n + 7) // 8 * 8

    @staticmethod
    def _length_bucket(n: int) -> int:
        b = 256
        while b < n:
            b *= 2
        return b

    def _graph_serves(self, entries) -> bool:
        return (self.graphs_enabled and self.model.capturable and len(entries) <= self.GRAPH_MAX_BATCH
                and all(len(e.tokens) == 1 for e in entries) and profile.active() is None)

    # Recorded steps kept at once, decode steps and short prompts counted apart (a burst of prompts of many lengths
    # must not push out the decode steps that run between them); the least recently used of its kind goes when
    # another is recorded.
    GRAPH_LIMIT = 24
    PROMPT_GRAPH_LIMIT = 8

    def _recorded(self, key, n_tokens: int, n_seqs: int, n_rows: int | None) -> dict:
        """The state of the recorded step ``key`` (made if new; the most recently used is kept last)."""
        state = self._decode_graphs.pop(key, None)
        if state is None:
            is_prompt = key[0] == "prompt"
            kin = [k for k in self._decode_graphs if (k[0] == "prompt") == is_prompt]
            limit = self.PROMPT_GRAPH_LIMIT if is_prompt else self.GRAPH_LIMIT
            if len(kin) >= limit:                 # a graph holds its activations and logits: bound them
                # a step launched ahead may still be queued or running: its graph and buffers go only when it is done
                torch.cuda.current_stream().synchronize()
                for k in kin[:len(kin) - limit + 1]:
                    self._decode_graphs.pop(k)
            size = context_ints(n_tokens, n_seqs)
            state = {"buf": torch.zeros((size,), dtype=torch.int32, device=self.device),
                     "staging": [torch.zeros((size,), dtype=torch.int32, pin_memory=True) for _ in range(2)],
                     "staged": [None, None], "turn": 0,
                     "rows": None if n_rows is None else torch.zeros((n_rows,), dtype=torch.int32, device=self.device),
                     "graph": None, "logits": None, "calls": 0}
        self._decode_graphs[key] = state
        return state

    def _replay(self, state, ctx) -> torch.Tensor:
        """Run the step whose arrays ``ctx`` has just laid into the state's buffer: as it is the first time (which
        loads or builds whatever it needs), recorded the second time, replayed from then on."""
        if state["graph"] is None and state["calls"] == 0:
            logits = self.model.forward(ctx, self.cache, state["rows"])
        else:
            if state["graph"] is None:
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, pool=self._graph_pool()):
                    state["logits"] = self.model.forward(ctx, self.cache, state["rows"])
                state["graph"] = graph
            state["graph"].replay()
            logits = state["logits"].clone()        # the graph's own buffer is overwritten by the next replay
        state["calls"] += 1
        return logits

    def _run_fed(self, entries, fed: FedTokens) -> torch.Tensor:
        if any(len(e.tokens) != 1 for e in entries) or len(fed.rows) != len(entries):
            raise StepError("a step fed from the device brings one token for each sequence and one row for each token")
        if fed.ids.dtype != torch.int32 or fed.ids.device != self.device or fed.ids.dim() != 1:
            raise StepError(f"fed tokens are int32 [m] on {self.device}, not {fed.ids.dtype} {tuple(fed.ids.shape)} on {fed.ids.device}")
        if any(not 0 <= int(r) < fed.ids.shape[0] for r in fed.rows):
            raise StepError(f"a fed row lies outside the {fed.ids.shape[0]} tokens given")
        if self._graph_serves(entries):
            return self._run_decode_graph(entries, fed)
        # no recorded step serves these entries: the tokens come to the host first (which waits for them) and are
        # checked like any others
        ids = fed.ids.tolist()
        entries = [self._entry(StepEntry(e.slot, [ids[int(r)]], e.want)) for e, r in zip(entries, fed.rows)]
        self._validate(entries)
        return self._run(entries)

    def _run_decode_graph(self, entries, fed: FedTokens | None = None) -> torch.Tensor:
        cache = self.cache
        growth = [(e.slot, 1) for e in entries]
        cache.reserve(growth)
        starts = [cache.lengths[e.slot] for e in entries]
        B = len(entries)
        Bb = self._batch_bucket(B)
        key = (Bb, self._length_bucket(max(starts) + 1))
        pad = Bb - B
        state = self._recorded(key, Bb, Bb, None)
        # the step's arrays, laid out as for any step, at the addresses the recording reads; rows that pad the batch
        # belong to a slot of their own whose page is never read
        # through pinned memory, so that the host need not wait for the device: two buffers in turn, each written
        # again only after the copy that last read it has run
        turn = state["turn"] = state["turn"] ^ 1
        if state["staged"][turn] is not None:
            state["staged"][turn].synchronize()
        ctx = make_context([e.slot for e in entries] + [cache.pad_slot] * pad, starts + [0] * pad,
                           [[int(e.tokens[0])] for e in entries] + [[0]] * pad, self.dtype, self.device,
                           max_total=key[1], into=state["buf"], staging=state["staging"][turn])
        state["staged"][turn] = torch.cuda.Event()
        state["staged"][turn].record()
        if fed is not None:
            rows = [int(r) for r in fed.rows]
            if rows == list(range(B)):
                ctx.token_ids[:B].copy_(fed.ids[:B])
            else:
                index = torch.tensor(rows, dtype=torch.int64).pin_memory().to(self.device, non_blocking=True)
                torch.index_select(fed.ids, 0, index, out=ctx.token_ids[:B])
        logits = self._replay(state, ctx)
        cache.commit(growth)
        wanted = [b for b, e in enumerate(entries) if e.want]
        if len(wanted) == B:
            return logits[:B]
        return logits[torch.tensor(wanted, dtype=torch.long, device=self.device)] if wanted else logits[:0]

    # A short prompt (or a short further piece) of one sequence is some hundred launches of kernels that take a few
    # microseconds each: launched one by one the host takes longer than the device.  Such steps are recorded too, by
    # the number of tokens rounded up to the next multiple of 8; the tokens that pad the step are a sequence of their
    # own in the slot whose page is never read.  (Longer prompts gain nothing from it: recorded up to 1,023 tokens,
    # by the count rounded up to a multiple of 32 or 64, a prompt of 64 took 6.8 ms instead of 5.4 and one of 512
    # 13.0 instead of 11.1: there the device is the slower side, and the tokens that pad the step cost more than
    # the launches.  A prompt of 2,048 tokens recorded whole: 35.3 ms against 27.9 launched, the library choosing
    # other kernels for its products while a stream is being recorded.  With the products of up to 128 rows all this
    # engine's own, recorded steps of 64 to 127 tokens were timed again: 64 tokens 4.9 ms against 5.3, 96 tokens 5.3
    # against 5.3, 127 tokens 5.6 against 5.7: too little for eight more recorded steps.)
    PROMPT_GRAPH_MAX_TOKENS = 63

    def _prompt_graph_serves(self, entries) -> bool:
        return (self.graphs_enabled and self.model.capturable and len(entries) == 1
                and 2 <= len(entries[0].tokens) <= self.PROMPT_GRAPH_MAX_TOKENS and len(entries[0].want) == 1
                and profile.active() is None)

    def _run_prompt_graph(self, entries) -> torch.Tensor:
        cache, e = self.cache, entries[0]
        n = len(e.tokens)
        bucket = (n // 8 + 1) * 8                   # at least one token pads the step
        growth = [(e.slot, n)]
        cache.reserve(growth)
        start = cache.lengths[e.slot]
        state = self._recorded(("prompt", bucket), bucket, 2, 1)
        ctx = make_context([e.slot, cache.pad_slot], [start, 0], [e.tokens, [0] * (bucket - n)], self.dtype,
                           self.device, into=state["buf"], max_new=bucket)
        state["rows"].copy_(torch.tensor([int(e.want[0])], dtype=torch.int32))
        logits = self._replay(state, ctx)
        cache.commit(growth)
        return logits

    def _graph_pool(self):
        """One memory pool for all recorded steps: replays never overlap (one stream, one at a time), so their
        activations may share memory, and a dropped recording's memory serves the next."""
        if self._graph_pool_handle is None:
            self._graph_pool_handle = torch.cuda.graph_pool_handle()
        return self._graph_pool_handle

    def _run(self, entries) -> torch.Tensor:
        recorder = profile.active()
        if recorder is not None:
            # a step with a recorder installed launches kernel by kernel (no graph) and is filed as a whole
            single = all(len(e.tokens) == 1 and self.cache.lengths[e.slot] > 0 for e in entries)
            label = f"{'decode' if single else 'prefill'} {len(entries)} x {max(len(e.tokens) for e in entries)}"
            with recorder.step("decode" if single else "prefill", label):
                return self._run_plain(entries)
        if self._graph_serves(entries):
            return self._run_decode_graph(entries)
        if self._prompt_graph_serves(entries):
            return self._run_prompt_graph(entries)
        return self._run_plain(entries)

    def _run_plain(self, entries) -> torch.Tensor:
        cache = self.cache
        growth = [(e.slot, len(e.tokens)) for e in entries]
        cache.reserve(growth)
        starts = [cache.lengths[e.slot] for e in entries]
        ctx = make_context([e.slot for e in entries], starts, [e.tokens for e in entries],
                           self.dtype, self.device)
        want_rows = [ctx.host["cu"][b] + int(w) for b, e in enumerate(entries) for w in e.want]
        if want_rows:
            rows = torch.tensor(want_rows, dtype=torch.int32).to(self.device)
        else:
            # nothing is wanted: the layers still run (they fill the cache); the head does not
            rows = torch.empty((0,), dtype=torch.int32, device=self.device)
        logits = self.model.forward(ctx, cache, rows)
        cache.commit(growth)
        return logits

    # ---- facts -------------------------------------------------------------------------------
    def memory_report(self) -> dict:
        return {"weights_bytes": self.model.weights.nbytes(), "cache_bytes": self.cache.nbytes(),
                "cache_tokens": self.cache.max_tokens, "slots": self.cache.max_seqs}

    # ---- generation --------------------------------------------------------------------------
    def generate(self, prompts, sampling=None, max_new_tokens: int = 2048, stop_token_ids=None, ignore_eos: bool = False,
                 max_batch: int = 64, on_token=None, **sampling_options):
        """Token ids in, token ids out: ``prompts`` is a list of lists of ids; returns (results, metrics),
        the results in the order of the prompts.  ``sampling`` is a ``SamplingParams``; its fields may also be
        given by name (``temperature=0.7, seed=1``) and then replace those of ``sampling`` or of the defaults.
        ``stop_token_ids`` defaults to the model's ``eos_token_id``; ``ignore_eos`` switches stopping off, as
        the reference's benchmark does (examples/bench.cpp:583)."""
        import dataclasses
        from ..sampling import DeviceSampler, SamplingParams
        from .generate import generate
        sampling = sampling or SamplingParams()
        if sampling_options:
            unknown = sorted(set(sampling_options) - {f.name for f in dataclasses.fields(SamplingParams)})
            if unknown:
                raise TypeError(f"generate() got unknown options {unknown}; sampling options are "
                                f"{[f.name for f in dataclasses.fields(SamplingParams)]}")
            sampling = dataclasses.replace(sampling, **sampling_options)
        sampler = DeviceSampler(sampling)
        if ignore_eos:
            stop = ()
        else:
            stop = self.spec.stop_token_ids if stop_token_ids is None else stop_token_ids
        return generate(self, sampler, prompts, max_new_tokens=max_new_tokens, stop_token_ids=stop, max_batch=max_batch,
                        on_token=on_token, sync=torch.cuda.synchronize)

    def conversation(self, sampling=None, stop_token_ids=None, ignore_eos: bool = False):
        """A sequence that stays in the cache from turn to turn: ``say(new tokens)`` feeds only what is new and
        generates; ``reset()`` starts over.  See ``engine.generate.Conversation``."""
        from ..sampling import DeviceSampler, SamplingParams
        from .generate import Conversation
        stop = () if ignore_eos else (self.spec.stop_token_ids if stop_token_ids is None else stop_token_ids)
        return Conversation(self, DeviceSampler(sampling or SamplingParams()), stop)
