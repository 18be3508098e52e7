"""Token selection on the device: greedy, temperature and nucleus (top-p) sampling.

Same rules as the reference's sampler (miniserve/engine/sampler.py:1-112): greedy rows take the
first maximal index whatever else is in the batch; sampled rows take ``argmax(logits / T + g)`` with
Gumbel noise hashed from (request seed, index of the token being sampled, vocabulary index), so a
request draws the same noise wherever it sits in a batch and whether or not it was preempted and
recomputed; ``top_p < 1`` masks the tokens outside the nucleus first. One kernel does all of it
without ``[rows, vocab]`` temporaries; the tokens stay on the device until the engine copies them
back once per step.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass
class SamplingArgs:
    temperature: torch.Tensor  # float32 [rows], 0 for greedy rows
    top_p: torch.Tensor | None  # float32 [rows]; None if every row has top_p == 1
    seed: torch.Tensor  # int32 [rows]: the 32 bits of the request's seed
    counter: torch.Tensor  # int32 [rows]: index of the sampled token in its sequence


def _bits32(v: int) -> int:
    return v - (1 << 32) if v >= (1 << 31) else v


class Sampler:
    def __init__(self, device, vocab_size: int, ops=None):
        self.device = torch.device(device)
        self.vocab_size = vocab_size
        if ops is None:
            from ..kernels import ops
        self.ops = ops

    def prepare(self, requests) -> SamplingArgs | None:
        """Per-row parameters for the next token of each request; None if all rows are greedy.
        The counter is ``seq_len``: the sampled token's index, both in a decode step and at the end
        of the prefill of a preempted request (miniserve/engine/sampler.py:74-76)."""
        params = [r.params for r in requests]
        if all(p.is_greedy for p in params):
            return None
        rows = len(requests)
        host = torch.empty((4, rows), dtype=torch.float32, pin_memory=self.device.type == "cuda")
        host[0] = torch.tensor([p.temperature for p in params], dtype=torch.float32)
        host[1] = torch.tensor([p.top_p for p in params], dtype=torch.float32)
        ints = host[2:].view(torch.int32)
        ints[0] = torch.tensor([_bits32(r.seed) for r in requests], dtype=torch.int32)
        ints[1] = torch.tensor([r.seq_len for r in requests], dtype=torch.int32)
        dev = host.to(self.device, non_blocking=True)
        dints = dev[2:].view(torch.int32)
        any_top_p = any(p.top_p < 1 for p in params)
        return SamplingArgs(dev[0], dev[1] if any_top_p else None, dints[0], dints[1])

    def sample(self, logits: torch.Tensor, args: SamplingArgs | None) -> torch.Tensor:
        """``logits`` float32 ``[rows, vocab]`` -> int32 ``[rows]`` on the device."""
        if args is None:
            return self.ops.sample_rows(logits)
        return self.ops.sample_rows(logits, args.temperature, args.top_p, args.seed, args.counter)
