"""The inputs of one step, as the kernels see them.

A step is a list of entries, one per request: its next tokens (a portion of a
prompt, or one decoded token) and the places among them whose logits are wanted.
The reference's forward call takes either n consecutive tokens of one sequence or
one token for each of n sequences (src/model.c:542-545); here any mix is one batch.
All integer arrays of a step travel to the device in one copy.
"""
from dataclasses import dataclass

import numpy as np
import torch

from .. import memory


@dataclass
class Entry:
    req_id: object
    tokens: list
    want: list          # indices into `tokens` whose logits are returned, in this order


@dataclass
class GroupInputs:
    block_table: torch.Tensor     # int32 [n_slots, max_blocks]: page of block b of the request in slot s
    slot_map: torch.Tensor        # int32 [T]: cache row each token's key and value are stored in


class StepInputs:
    """Device views (int32) and host facts of one step.

    tokens[T], positions[T], token_slot[T] (the state slot = block-table row of the
    token's request), q_start[S + 1] (token range of each request), seq_slot[S],
    seq_len[S] (the request's length after this step), logit_rows[R].

    Requests that bring few tokens (fewer than the model's ``short_request_rows``, which a part sets: decoded tokens, ends of prompts)
    come first in a step: the first ``n_short_seqs`` requests with ``n_short_tokens`` tokens, none
    of them more than ``max_short_q_len``. ``q_start_long`` is ``q_start`` of the remaining requests
    counted from their first token, so that a kernel can be given either part as a step of its own.
    """

    def __init__(self, n_tokens, n_seqs, n_logit_rows):
        self.n_tokens, self.n_seqs, self.n_logit_rows = n_tokens, n_seqs, n_logit_rows
        self.tokens = self.positions = self.token_slot = None
        self.q_start = self.seq_slot = self.seq_len = self.logit_rows = None
        self.groups = []
        self.max_q_len = 0
        self.max_seq_len = 0
        self.n_short_seqs = self.n_short_tokens = self.max_short_q_len = 0
        self.q_start_long = None
        self.host = None          # dict of the numpy arrays the device views were copied from
        self.rows_in_order = False    # logits are wanted for every token, in the tokens' order (a decode step)

    def group(self, index):
        return self.groups[index]


class IntStaging:
    """Pinned host buffers and one device buffer through which a step's integers go
    up in a single copy. Two host buffers alternate so that one can be filled while
    the other's copy may still be in flight."""

    def __init__(self, device, capacity=1 << 16):
        self.device = device
        self.capacity = 0
        self.host = []
        self.events = []
        self.dev = None
        self.turn = 0
        self.generation = 0
        self._grow(capacity)

    def _grow(self, capacity):
        torch.cuda.synchronize(self.device)
        # all three first, then the switch: a failed allocation leaves the old buffers in use
        host = [memory.empty(capacity, torch.int32, None, "pinned staging buffer", pin=True) for _ in range(2)]
        dev = memory.empty(capacity, torch.int32, self.device, "device staging buffer")
        self.generation += 1                      # captured graphs hold the old address
        self.capacity = capacity
        self.host, self.dev = host, dev
        self.events = [None, None]

    def upload(self, arrays):
        """Copies the int32 numpy arrays one after the other; returns device views of them.
        Each array starts at a multiple of 4 elements."""
        offsets, total = [], 0
        for a in arrays:
            offsets.append(total)
            total += (a.size + 3) & ~3
        if total > self.capacity:
            self._grow(max(total, 2 * self.capacity))
        self.turn ^= 1
        if self.events[self.turn] is not None:
            self.events[self.turn].synchronize()
        host = self.host[self.turn]
        flat = host.numpy()
        for a, off in zip(arrays, offsets):
            flat[off:off + a.size] = a
        if total:
            self.dev[:total].copy_(host[:total], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.events[self.turn] = ev
        return [self.dev[off:off + a.size] for a, off in zip(arrays, offsets)]


def as_i32(values):
    return np.asarray(values, dtype=np.int32).reshape(-1)
