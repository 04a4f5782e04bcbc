"""Choosing next tokens for a batch of logits rows on the GPU.

One kernel call serves all rows; each row carries its own options.  The "seen"
sets of the presence penalty live in the per-request slots (one bit per
vocabulary entry), are cleared when a slot is taken and updated as tokens
arrive.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..ops import kernels
from .params import SamplingParams, uniform_for


class Sampler:
    def __init__(self, vocab_size: int, num_slots: int, device: torch.device,
                 banned_tokens: Optional[Sequence[int]] = None):
        self.vocab = int(vocab_size)
        self.device = torch.device(device)
        self.words = (self.vocab + 31) // 32
        self.num_slots = int(num_slots)
        self.seen: Optional[torch.Tensor] = None  # [slots, words], made when a request first needs it
        self.banned: Optional[torch.Tensor] = None
        self._part_val: Optional[torch.Tensor] = None
        self._part_idx: Optional[torch.Tensor] = None
        self._chunked: Optional[dict] = None             # scratch of the sampling in chunks
        # pinned [6, rows] int32 and device twins, two of each used in turn: a step's per-row options go up without
        # the host waiting, and a caller may queue a step's sampling while it still waits for the tokens of the step
        # before (not for older ones: a pair is used again two calls later)
        self._options_host: List[Optional[torch.Tensor]] = [None, None]
        self._options_dev: List[Optional[torch.Tensor]] = [None, None]
        self._turn = 0
        if banned_tokens:
            host = torch.zeros(self.words, dtype=torch.int64)
            for tok in banned_tokens:
                if 0 <= tok < self.vocab:
                    host[tok >> 5] |= 1 << (tok & 31)
            # keep the bit patterns when narrowing to int32
            host = torch.where(host >= 2 ** 31, host - 2 ** 32, host)
            self.banned = host.to(torch.int32).to(self.device)

    # -------------------------------------------------------------- seen sets
    def start_request(self, slot: int, params: SamplingParams, tokens: Sequence[int]) -> None:
        """A request took ``slot``: clear its seen set and mark the tokens it starts with."""
        if params.presence_penalty > 0.0:
            if self.seen is None:
                self.seen = torch.zeros((self.num_slots, self.words), dtype=torch.int32, device=self.device)
            self.seen[slot].zero_()
            self.note_tokens([slot] * len(tokens), list(tokens))

    def note_tokens(self, slots: Sequence[int], tokens: Sequence[int]) -> None:
        if self.seen is None or not slots:
            return
        both = torch.tensor([list(slots), list(tokens)], dtype=torch.int32).to(self.device)   # one upload
        kernels.mark_seen(self.seen, both[0], both[1], self.vocab)

    def note_on_device(self, slots: torch.Tensor, tokens: torch.Tensor) -> None:
        """``note_tokens`` for tokens that are still on the device (``launch``'s result): ``slots`` int32 on the
        device, -1 where a row's request keeps no seen set; rows without a token (-1) mark nothing."""
        if self.seen is not None and slots.numel():
            kernels.mark_seen(self.seen, slots, tokens, self.vocab)

    # ---------------------------------------------------------------- sampling
    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], slots: Sequence[int],
               counters: Sequence[int], default_seeds: Sequence[int]) -> List[int]:
        """One token per row.  ``counters[r]`` is how many tokens row r's request has drawn before."""
        if logits.shape[0] == 0:
            return []
        return self.launch(logits, params, slots, counters, default_seeds).tolist()

    def launch(self, logits: torch.Tensor, params: Sequence[SamplingParams], slots: Sequence[int],
               counters: Sequence[int], default_seeds: Sequence[int]) -> torch.Tensor:
        """``sample`` without waiting: the tokens as an int32 vector on the device, the kernels only queued."""
        rows = logits.shape[0]
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        if rows == 0:
            return out
        if all(p.greedy and p.presence_penalty == 0.0 for p in params) and self.banned is None:
            need = rows * kernels.argmax_chunks(logits.shape[1])
            if self._part_val is None or self._part_val.numel() < need:
                self._part_val = torch.empty(need, dtype=torch.float32, device=self.device)
                self._part_idx = torch.empty(need, dtype=torch.int32, device=self.device)
            kernels.argmax(logits, out, self._part_val, self._part_idx)
            return out
        # every per-row option in one upload: rows of a [6, R] int32 array, the float ones as their bit patterns
        use_penalty = self.seen is not None and any(p.presence_penalty > 0.0 for p in params)
        turn = self._turn
        self._turn = 1 - turn
        if self._options_host[turn] is None or self._options_host[turn].shape[1] < rows:
            self._options_host[turn] = torch.empty((6, max(rows, 64)), dtype=torch.int32, pin_memory=True)
            self._options_dev[turn] = torch.empty((6, max(rows, 64)), dtype=torch.int32, device=self.device)
        # (the copy out of these pinned rows two calls ago has run: its tokens have been waited for)
        host = self._options_host[turn].numpy()[:, :rows]
        as_float = host.view(np.float32)
        as_float[0] = [p.temperature for p in params]
        host[1] = [p.top_k for p in params]
        as_float[2] = [p.top_p for p in params]
        as_float[3] = [uniform_for(p.seed if p.seed is not None else d, c)
                       for p, c, d in zip(params, counters, default_seeds)]
        as_float[4] = [p.presence_penalty for p in params]
        host[5] = [s if p.presence_penalty > 0.0 else -1 for p, s in zip(params, slots)]
        self._options_dev[turn].copy_(self._options_host[turn], non_blocking=True)
        dev = self._options_dev[turn]
        temperature, top_p, uniform = (dev[i, :rows].view(torch.float32) for i in (0, 2, 3))
        top_k = dev[1, :rows]
        penalty = dev[4, :rows].view(torch.float32) if use_penalty else None
        seen_row = dev[5, :rows] if use_penalty else None
        seen = self.seen if penalty is not None else None
        # in chunks of the vocabulary; which way a row goes there depends on its own options alone, so a seeded
        # request draws the same tokens whatever else is in the batch.  An option that no row uses is left out
        # (a kernel less), which changes no row's choice.
        if self._chunked is None or self._chunked["done"].numel() < rows:
            self._chunked = kernels.sample_chunked_scratch(rows, logits.shape[1], self.device)
        kernels.sample_chunked(logits, out, self._chunked, temperature=temperature,
                               top_k=top_k if any(p.top_k > 0 for p in params) else None,
                               top_p=top_p if any(0.0 < p.top_p < 1.0 for p in params) else None,
                               uniform=uniform, penalty=penalty, seen_row=seen_row, seen_masks=seen,
                               banned=self.banned)
        return out
