"""Replay of a recorded run: feed given token ids through the engine step by step and write the logits.

    python -m vllm_distributed_amd.entrypoints.trace_replay --model DIR --dtype bfloat16|float32 --out DIR
                                                             --max-tokens N        (or: bin/trace_run ...)

Standard input carries one JSON object per step,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["b"]}
``entries``: for every request its next tokens (a request is admitted at its first entry and may sit out steps),
``want``: indices among these tokens whose logits are written, ``end``: requests that are finished after the step
(their pages and state slot go back to the pools).  A step with wanted logits writes ``<out>/<step>.f32``
(little-endian fp32, [wanted, vocab], in the order of the entries); every step answers ``done <step>``.

Nothing here computes anything: the steps go through the engine core's scheduler (which admits requests, allocates
pages and batches exactly the given tokens: ``Scheduler.schedule(plan=...)``), its executor, worker and model runner
-- the generation path -- with the requests marked as fed from outside, so what the sampler picks is dropped.
``--max-tokens`` sizes the page pool (tokens live at any time); four requests can be live at once.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np


class TraceReplayer:
    def __init__(self, model: str, dtype: str, max_tokens: int, max_live: int = 4, block_size: int = 16,
                 device: str = "auto", enforce_eager: bool = False):
        import torch
        if device == "auto":
            device = "cuda" if torch.cuda.is_available() else "cpu"
        if dtype == "float32":
            # true fp32 matrix products: no reduced-precision modes of the vendor libraries
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False
            torch.set_float32_matmul_precision("highest")
        from ..engine.arg_utils import EngineArgs
        from ..engine.core import EngineCore
        from ..executor.base import Executor
        pool = -(-int(max_tokens) // block_size)
        args = EngineArgs(
            model=model, skip_tokenizer_init=True, dtype=dtype, device=device, block_size=block_size,
            max_model_len=pool * block_size + 1, max_num_seqs=max_live, max_num_batched_tokens=pool * block_size,
            num_gpu_blocks_override=pool + 1,             # + the pool's reserved null page
            enable_prefix_caching=False, enable_chunked_prefill=True, enforce_eager=enforce_eager,
            gpu_memory_utilization=0.5, distributed_executor_backend="uni", async_scheduling=False,
            disable_log_stats=True)
        cfg = args.create_engine_config()
        self.core = EngineCore(cfg, Executor.get_class(cfg), log_stats=False)
        self.vocab = cfg.model_config.get_vocab_size()
        self.live: set[str] = set()

    def step(self, entries: list[dict], end: list[str]):
        """Run one step; returns fp32 logits [wanted, vocab] (None when nothing was wanted)."""
        from ..request import Request, RequestStatus
        from ..sampling_params import SamplingParams
        sched = self.core.scheduler
        plan, taps = {}, {}
        for e in entries:
            rid, toks = str(e["id"]), [int(t) for t in e["tokens"]]
            if not toks:
                continue
            if rid in self.live:
                sched.extend_request(rid, toks)
            else:
                sp = SamplingParams(temperature=0.0, max_tokens=1 << 30, ignore_eos=True)
                sched.add_request(Request(rid, toks, sp), forced=True)
                self.live.add(rid)
            plan[rid] = len(toks)
            if e.get("want"):
                taps[rid] = [int(w) for w in e["want"]]
        rows = None
        if plan:
            so = sched.schedule(plan=plan)
            if set(so.num_scheduled_tokens) != set(plan) or any(so.num_scheduled_tokens[r] != n
                                                                 for r, n in plan.items()):
                raise RuntimeError(f"the scheduler ran {so.num_scheduled_tokens}, the step asks for {plan}")
            so.logit_taps = taps
            mro = self.core.execute_model(so)
            sched.update_from_output(so, mro)
            if taps:
                rows = np.concatenate([mro.tapped_logits[str(e["id"])] for e in entries if e.get("want")], axis=0)
        gone = [str(r) for r in end if str(r) in self.live]
        if gone:
            sched.finish_requests(gone, RequestStatus.FINISHED_ABORTED)
            self.live.difference_update(gone)
        return rows

    def shutdown(self) -> None:
        self.core.shutdown()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "float16"])
    ap.add_argument("--out", required=True, help="folder the logits are written to")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens that live requests hold at most")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--max-live", type=int, default=4, help="requests that can be live at once")
    ap.add_argument("--device", default="auto")
    ap.add_argument("--enforce-eager", action="store_true", help="no captured decode graphs")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    # the engine logs to standard output's neighbour only: the protocol owns stdout
    r = TraceReplayer(a.model, a.dtype, a.max_tokens, a.max_live, a.block_size, a.device, a.enforce_eager)
    out = sys.stdout
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        rows = r.step(msg.get("entries", []), msg.get("end", []))
        if rows is not None:
            tmp = os.path.join(a.out, f".{msg['step']}.f32.part")
            np.ascontiguousarray(rows, dtype="<f4").tofile(tmp)
            os.replace(tmp, os.path.join(a.out, f"{msg['step']}.f32"))
        out.write(f"done {msg['step']}\n")
        out.flush()
    r.shutdown()
    return 0


if __name__ == "__main__":
    sys.exit(main())
