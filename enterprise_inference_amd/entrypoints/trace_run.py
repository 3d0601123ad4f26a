"""Replay a recorded schedule of token ids through the engine and write logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry carries a request's next tokens (a request is admitted at its first entry and may
skip steps); all entries of a step run as ONE batch through the engine's scheduler bookkeeping
(``Scheduler.plan_given``: cache blocks, state slots), the model runner's step staging and the
model's kernels -- the path generation uses, minus sampling.  ``want`` lists the places among
the entry's tokens whose logits are written, in entry order, to ``<out>/<step>.f32`` as
little-endian fp32 [wanted, vocab].  Requests in ``end`` give their blocks and slot back after
the step.  After each step ``done <step>`` is printed.  The cache pool holds ``--max-tokens``
tokens in 64-token blocks and there are state slots for four live requests.

Exit code 3: ``--dtype float32`` asked of a model that has no fp32 kernels.
"""

from __future__ import annotations

import argparse
import json
import logging
import os
import sys

BLOCK = 64
MAX_LIVE = 4


class TraceSession:
    """The engine pieces a replay drives: executor (model runner, caches), scheduler (block
    manager, state slots) and the live requests."""

    def __init__(self, cfg):
        from ..engine.executor import make_executor
        from ..engine.sampling_params import SamplingParams
        from ..engine.scheduler import Scheduler

        self.cfg = cfg
        self.executor = make_executor(cfg)
        self.runner = self.executor.runner
        self.scheduler = Scheduler(cfg.scheduler, cfg.cache, self.executor.num_blocks)
        self.live = {}
        self._params = SamplingParams(max_tokens=1 << 30, temperature=0.0, ignore_eos=True)

    def step(self, entries, end=()):
        """entries: [{"id", "tokens", "want"}]; returns fp32 logits [wanted, vocab] (rows in
        entry order) or None when nothing is wanted; then frees the requests in ``end``."""
        from ..engine.sequence import SeqStatus, Sequence

        chunks, wants = [], {}
        for e in entries:
            seq = self.live.get(e["id"])
            if seq is None:
                seq = self.live[e["id"]] = Sequence(str(e["id"]), [], self._params)
            seq.prompt_token_ids.extend(int(t) for t in e["tokens"])
            chunks.append((seq, len(e["tokens"])))
            wants[seq.seq_id] = [int(w) for w in e.get("want", [])]
        logits = None
        if chunks:
            sched = self.scheduler
            plan = sched.plan_given(chunks)
            # batch rows: decode rows first, then the prefill chunks, in the planner's order
            first, row = {}, 0
            for it in plan.decodes + plan.prefills:
                first[it.seq.seq_id] = row
                row += it.num_tokens
            rows = [first[seq.seq_id] + w for seq, _ in chunks for w in wants[seq.seq_id]]
            logits = self.runner.step_logits(sched.bm, plan, rows)
            sched.update_after_step(plan)
            if not rows:
                logits = None
        for rid in end:
            seq = self.live.pop(rid, None)
            if seq is not None:
                self.scheduler.finish(seq, SeqStatus.FINISHED_STOPPED)
        return logits

    def close(self) -> None:
        self.executor.shutdown()


def replay_config(model_cfg, model_path, dtype, device: str, max_tokens: int,
                  block_size: int = BLOCK, max_live: int = MAX_LIVE, load_format: str = "auto"):
    """Engine configuration of a replay: a pool of ``max_tokens`` tokens in ``block_size``
    blocks, ``max_live`` sequences (and state slots), no prefix reuse, eager steps."""
    from ..config import CacheConfig, EngineConfig, SchedulerConfig

    pool = -(-max_tokens // block_size)
    return EngineConfig(
        model=model_cfg, dtype=dtype, device=device, model_path=model_path,
        load_format=load_format,
        cache=CacheConfig(block_size=block_size, num_gpu_blocks=pool, enable_prefix_caching=False,
                          swap_space_gb=0.0),
        scheduler=SchedulerConfig(max_num_seqs=max_live, max_num_batched_tokens=pool * block_size,
                                  max_model_len=pool * block_size, enable_chunked_prefill=True,
                                  delayed_sampling=False),
        enforce_eager=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--device", default="auto", choices=["auto", "cuda", "cpu"])
    a = ap.parse_args(argv)
    logging.basicConfig(stream=sys.stderr, level=logging.WARNING)

    import numpy as np
    import torch

    from ..config import parse_dtype
    from ..models import get_model_class
    from ..models.loader import resolve_model_config

    dtype = parse_dtype(a.dtype)
    device = a.device
    if device == "auto":
        device = "cuda" if torch.cuda.is_available() else "cpu"
    mcfg = resolve_model_config(a.model)
    if dtype == torch.float32 and device == "cuda" and not getattr(
            get_model_class(mcfg.architecture), "supports_float32", False):
        print(f"{mcfg.architecture} has no float32 kernels", file=sys.stderr)
        return 3
    sess = TraceSession(replay_config(mcfg, a.model, dtype, device, a.max_tokens))
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = sess.step(st["entries"], st.get("end", []))
        if logits is not None:
            out = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
            tmp = os.path.join(a.out, f".{st['step']}.tmp")
            with open(tmp, "wb") as f:
                f.write(np.ascontiguousarray(out).tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        elif device == "cuda":
            torch.cuda.synchronize()
        print(f"done {st['step']}", flush=True)
    sess.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
