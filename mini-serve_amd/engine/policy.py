"""Admission order and preemption victim. First come first served is the default, as in the
reference (miniserve/engine/policy.py:44-51); shortest job first is its second policy (:60-68).
Its third, ordering by cached prefix, needs a prefix cache and is not offered."""

from __future__ import annotations


class FCFS:
    name = "fcfs"

    def order(self, waiting):
        return list(waiting)

    def pick_victim(self, candidates):
        return candidates[-1]  # the most recently admitted


class ShortestJobFirst:
    """Least remaining work first; the victim is the request with the most left to do."""

    name = "sjf"

    @staticmethod
    def _remaining(r) -> int:
        return r.params.max_new_tokens - r.num_output

    def order(self, waiting):
        return sorted(waiting, key=lambda r: (r.seq_len + self._remaining(r), r.rid))

    def pick_victim(self, candidates):
        return max(candidates, key=lambda r: (self._remaining(r), r.rid))


POLICIES = {"fcfs": FCFS, "sjf": ShortestJobFirst}


def make_policy(name: str):
    try:
        return POLICIES[name]()
    except KeyError:
        raise ValueError(f"unknown schedule policy {name!r}, expected one of {sorted(POLICIES)}") from None
