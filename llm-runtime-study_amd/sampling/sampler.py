"""Token choice for a batch of logits rows, on the device.

Greedy rows take the lowest index among the largest logits.  Other rows are filtered by
top-k and top-p (rule of the reference, mini_llm/sampling.py:40-69) and drawn from
softmax(logits / temperature) (89-91).  The reference draws on the CPU with a torch
generator per request; here the draw is a device kernel keyed by (request seed, number of
tokens the request has drawn), so a request's tokens depend on its own seed only, not on
its batch mates; the stream of numbers is not torch's.  A request without a seed gets one
from the operating system when it is admitted.
"""

from __future__ import annotations

import random
from dataclasses import dataclass

import numpy as np
import torch

from ..errors import SamplingError
from ..kernels import ops
from .config import SamplingConfig

_system_random = random.SystemRandom()


def request_seed(config: SamplingConfig) -> int:
    return config.seed if config.seed is not None else _system_random.getrandbits(62)


@dataclass
class SamplingRow:
    config: SamplingConfig
    seed: int
    counter: int  # tokens this request has drawn so far


def refuse_not_finite(tokens) -> None:
    """The kernels give -1 for a row of logits that holds a value that is not finite; the reference refuses
    such logits with this message (mini_llm/sampling.py:104-113)."""
    if any(token < 0 for token in tokens):
        raise SamplingError("logits must contain only finite values")


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)
        self._chosen = None      # pinned host memory the kernel writes the tokens into ...
        self._chosen_address = 0  # ... and where the device sees it
        self._settings_host = self._settings_dev = None   # the rows' sampling settings: pinned staging and its device copy
        self._settings_cap = 0

    def _settings_room(self, rows: int) -> int:
        """Staging for `rows` rows' settings (six int32 words a row, in five arrays of `cap` rows); returns cap.  The
        staging is written again only after the copy that last read it has finished."""
        if self._settings_cap < rows:
            self._settings_cap = cap = max(64, -(-rows // 4) * 4)
            self._settings_host = torch.zeros(6 * cap, dtype=torch.int32, pin_memory=True)
            self._settings_dev = torch.zeros(6 * cap, dtype=torch.int32, device=self.device)
        return self._settings_cap

    def _result(self, rows: int) -> torch.Tensor:
        if self._chosen is None or self._chosen.numel() < rows:
            self._chosen = torch.zeros(max(rows, 64), dtype=torch.int32, pin_memory=True)
            self._chosen_address = ops.pinned_device_address(self._chosen)
        return self._chosen[:rows]

    def _read(self, out: torch.Tensor) -> list[int]:
        torch.cuda.current_stream(self.device).synchronize()
        tokens = out.tolist()
        refuse_not_finite(tokens)
        return tokens

    def choose(self, logits: torch.Tensor, rows: list[SamplingRow]) -> list[int]:
        """One token per row of `logits` [R, V] float32 (filters the sampled rows in place)."""
        if logits.dim() != 2 or logits.shape[0] != len(rows) or logits.dtype != torch.float32:
            raise SamplingError(f"logits must be float32 [rows, vocabulary] with {len(rows)} rows, got {tuple(logits.shape)} {logits.dtype}")
        vocab = logits.shape[1]
        for row in rows:
            if row.config.top_k is not None and row.config.top_k > vocab:
                raise SamplingError(f"top_k {row.config.top_k} exceeds vocabulary size {vocab}")
        out = self._result(len(rows))
        if all(row.config.greedy for row in rows):
            ops.choose_tokens(out, logits, out_address=self._chosen_address)
            return self._read(out)
        # temperature, top-p, top-k, draws so far and seed of every row: written into pinned memory and sent in one copy
        # (five tensors made from Python lists would be five pageable copies, each waiting for the device)
        n = len(rows)
        cap = self._settings_room(n)
        host = self._settings_host.numpy()
        host[:cap].view(np.float32)[:n] = [row.config.temperature for row in rows]
        host[cap:2 * cap].view(np.float32)[:n] = [row.config.top_p for row in rows]
        host[2 * cap:3 * cap][:n] = [row.config.top_k or 0 for row in rows]
        host[3 * cap:4 * cap][:n] = [row.counter for row in rows]
        host[4 * cap:6 * cap].view(np.int64)[:n] = [row.seed for row in rows]
        ops.copy_h2d(self._settings_dev, self._settings_host, 6 * cap)
        dev = self._settings_dev
        temperature, top_p = dev[:cap].view(torch.float32)[:n], dev[cap:2 * cap].view(torch.float32)[:n]
        top_k, counters, seeds = dev[2 * cap:3 * cap][:n], dev[3 * cap:4 * cap][:n], dev[4 * cap:6 * cap].view(torch.int64)[:n]
        filtered = any((row.config.top_k is not None and row.config.top_k < vocab) or row.config.top_p < 1.0 for row in rows if not row.config.greedy)
        if filtered:
            ops.filter_logits(logits, temperature, top_k, top_p)
        ops.choose_tokens(out, logits, temperature, seeds, counters, out_address=self._chosen_address, filtered=filtered)
        return self._read(out)
