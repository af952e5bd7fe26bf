"""Choosing next tokens for a batch of sequences.

The rules are the reference's (engine/sampler.cpp): penalties over a window of the tokens the model has
consumed (:304-343), then greedy, or the temperature/top-k/min-p/top-p candidates and a draw (:90-188).
What differs is where it runs and where the randomness comes from: the logits stay on the device and
the kernels of ``csrc/sampling.hip`` choose; each sequence has a stream of uniform numbers of its own,
u = hash(seed, stream, draw number), instead of one ``rand_r`` state for the engine, so a sequence's
tokens do not depend on what else is in its batch.  ``reset()`` of a stream restores its first number,
as the reference's ``reset()`` restores the seed (:276-282).
"""
from __future__ import annotations

import numpy as np
import torch

from .params import SamplingParams

_MASK = (1 << 64) - 1


def _mix(z: int) -> int:
    """splitmix64's finaliser."""
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, stream: int, draw: int) -> float:
    """A float32 in [0, 1) that depends on (seed, stream, draw) only."""
    h = _mix(_mix(_mix(int(seed)) ^ int(stream)) ^ int(draw))
    return float(np.float32((h >> 40) / float(1 << 24)))


def penalty_counts(history, repeat_last_n: int, vocab_size: int) -> dict[int, int]:
    """token -> count within the last ``repeat_last_n`` tokens of the history (-1: all of it)
    (engine/sampler.cpp:317-329)."""
    window = len(history) if repeat_last_n < 0 else min(len(history), repeat_last_n)
    counts: dict[int, int] = {}
    for t in history[len(history) - window:]:
        if 0 <= t < vocab_size:
            counts[t] = counts.get(t, 0) + 1
    return counts


class SequenceSampling:
    """What sampling remembers of one sequence: the tokens the model has consumed and its place in
    its stream of random numbers."""

    def __init__(self, stream: int):
        self.stream = int(stream)
        self.history: list[int] = []
        self.draws = 0

    def accept(self, tokens) -> None:
        self.history.extend(int(t) for t in tokens if int(t) >= 0)

    def reset(self) -> None:
        self.history.clear()
        self.draws = 0


class DeviceSampler:
    """``sample(logits, states)``: logits float32 [B, vocab] on the device, one state for each row;
    returns int32 [B] on the device."""

    def __init__(self, params: SamplingParams | None = None):
        self.params = params or SamplingParams()
        self.params.validate()

    @property
    def needs_history(self) -> bool:
        """Whether a draw depends on the tokens drawn before (the penalties do): a loop may then not ask for a
        sequence's next draw before the host has seen its last one."""
        return bool(self.params.penalties_enabled)

    def sample(self, logits: torch.Tensor, states) -> torch.Tensor:
        from ..kernels import ops
        p = self.params
        if len(states) != logits.shape[0]:
            raise ValueError(f"{logits.shape[0]} rows of logits for {len(states)} sequences")
        V = logits.shape[1]
        if p.penalties_enabled:
            rows, toks, cnts = [], [], []
            for r, st in enumerate(states):
                for t, c in penalty_counts(st.history, p.repeat_last_n, V).items():
                    rows.append(r); toks.append(t); cnts.append(c)
            if rows:
                logits = logits.clone()     # the caller's logits stay as they are (engine/sampler.cpp:347-349)
                packed = torch.tensor([rows, toks, cnts], dtype=torch.int32).to(logits.device)
                ops.apply_penalties(logits, packed[0], packed[1], packed[2], p.repeat_penalty, p.presence_penalty,
                                    p.frequency_penalty)
        if p.greedy:
            return ops.argmax(logits)
        # through pinned memory: the host does not wait for the device here
        u = torch.tensor([uniform(p.seed, st.stream, st.draws) for st in states], dtype=torch.float32).pin_memory().to(
            logits.device, non_blocking=True)
        for st in states:
            st.draws += 1
        top_k = p.top_k if 0 < p.top_k < V else 0
        return ops.sample(logits, u, p.temperature, top_k, p.top_p, p.min_p)

    def probabilities(self, logits: torch.Tensor, states) -> torch.Tensor:
        """The distribution a draw would come from, [B, vocab]; changes no state
        (engine/sampler.cpp:352-395)."""
        from ..kernels import ops
        p = self.params
        V = logits.shape[1]
        if p.penalties_enabled:
            logits = logits.clone()
            rows, toks, cnts = [], [], []
            for r, st in enumerate(states):
                for t, c in penalty_counts(st.history, p.repeat_last_n, V).items():
                    rows.append(r); toks.append(t); cnts.append(c)
            if rows:
                packed = torch.tensor([rows, toks, cnts], dtype=torch.int32).to(logits.device)
                ops.apply_penalties(logits, packed[0], packed[1], packed[2], p.repeat_penalty, p.presence_penalty,
                                    p.frequency_penalty)
        u = torch.zeros((logits.shape[0],), dtype=torch.float32, device=logits.device)
        top_k = p.top_k if 0 < p.top_k < V else 0
        _, probs = ops.sample(logits, u, p.temperature, top_k, p.top_p, p.min_p, want_probs=True)
        return probs
