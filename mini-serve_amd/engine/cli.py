"""Command-line options shared by everything that builds an ``Engine``, under the reference's
names and meanings where it has them (miniserve/engine/cli.py:12-106). Options of the reference
that have nothing to switch here (``--attention``, ``--disable-radix``, ``--attn-workspace-mb``,
``--fused-ops``: the cache is always paged, prefixes are never shared, the kernels size their own
scratch and are always the fused ones) are not offered; argparse names them in its error."""

from __future__ import annotations

import argparse

from ..cache.backend import BACKENDS
from .policy import POLICIES


def add_engine_args(parser: argparse.ArgumentParser) -> None:
    g = parser.add_argument_group("engine")
    g.add_argument("--max-running", type=int, default=64, help="max requests in the running batch")
    g.add_argument("--max-prefill-tokens", type=int, default=8192, help="token budget of one prefill batch")
    g.add_argument("--kv-pool-tokens", type=int, default=None,
                   help="exact cache pool size in tokens (rounded down to whole pages); default: as large as GPU memory allows")
    g.add_argument("--seed", type=int, default=0, help="seeds sampling for requests that bring no seed of their own")
    g.add_argument("--chunked-prefill-size", type=int, default=None,
                   help="tokens per step, decodes included, with prefills cut into portions batched with decodes; "
                        "0: whole prefills in prefill-only steps (default 2048)")
    g.add_argument("--schedule-policy", choices=sorted(POLICIES), default="fcfs",
                   help="admission order and preemption choice: fcfs, sjf (least remaining work first)")
    g.add_argument("--disable-cuda-graph", "--disable-hip-graph", dest="disable_graph", action="store_true",
                   help="run decode steps eagerly (no captured HIP graphs)")
    g.add_argument("--cuda-graph-max-bs", "--hip-graph-max-bs", dest="graph_max_bs", type=int, default=None,
                   help="largest decode batch captured in a graph (default: --max-running); graphs are captured "
                        "for powers of two below it and for it")
    g.add_argument("--block-backend", choices=BACKENDS, default=None,
                   help="page bookkeeping: python (default) or cpp; also settable with MINISERVE_BLOCK_BACKEND")
    g.add_argument("--page-size", type=int, default=16, help="tokens per cache page")
    g.add_argument("--kv-mem-fraction", type=float, default=0.9, help="share of free GPU memory the cache pool may take")
    g.add_argument("--disable-overlap", action="store_true",
                   help="read back each step's tokens before scheduling the next (default: one step later)")


def engine_kwargs(args: argparse.Namespace) -> dict:
    return dict(
        max_running=args.max_running,
        max_prefill_tokens=args.max_prefill_tokens,
        kv_pool_tokens=args.kv_pool_tokens,
        seed=args.seed,
        chunked_prefill_size=args.chunked_prefill_size,
        schedule_policy=args.schedule_policy,
        decode_graph=not args.disable_graph,
        decode_graph_max_bs=args.graph_max_bs,
        block_backend=args.block_backend,
        page_size=args.page_size,
        kv_mem_fraction=args.kv_mem_fraction,
        overlap=not args.disable_overlap,
    )
