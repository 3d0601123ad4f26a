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

    from ..config import CacheConfig, EngineConfig, SchedulerConfig, parse_dtype
    from ..engine.executor import make_executor
    from ..engine.sampling_params import SamplingParams
    from ..engine.scheduler import Scheduler
    from ..engine.sequence import SeqStatus, Sequence
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
    pool = -(-a.max_tokens // BLOCK)
    cfg = EngineConfig(
        model=mcfg, dtype=dtype, device=device, model_path=a.model,
        cache=CacheConfig(block_size=BLOCK, num_gpu_blocks=pool, enable_prefix_caching=False,
                          swap_space_gb=0.0),
        scheduler=SchedulerConfig(max_num_seqs=MAX_LIVE, max_num_batched_tokens=pool * BLOCK,
                                  max_model_len=pool * BLOCK, enable_chunked_prefill=True,
                                  delayed_sampling=False),
        enforce_eager=True)
    ex = make_executor(cfg)
    runner = ex.runner
    sched = Scheduler(cfg.scheduler, cfg.cache, ex.num_blocks)
    os.makedirs(a.out, exist_ok=True)
    live = {}
    params = SamplingParams(max_tokens=1 << 30, temperature=0.0, ignore_eos=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        chunks, by_seq = [], {}
        for e in st["entries"]:
            seq = live.get(e["id"])
            if seq is None:
                seq = live[e["id"]] = Sequence(str(e["id"]), [], params)
            seq.prompt_token_ids.extend(int(t) for t in e["tokens"])
            chunks.append((seq, len(e["tokens"])))
            by_seq[seq.seq_id] = e
        if chunks:
            plan = sched.plan_given(chunks)
            # batch rows: decode rows first, then the prefill chunks, in the planner's order
            first, row = {}, 0
            for it in plan.decodes + plan.prefills:
                first[it.seq.seq_id] = row
                row += it.num_tokens
            rows = [first[seq.seq_id] + int(w) for seq, _ in chunks
                    for w in by_seq[seq.seq_id].get("want", [])]
            logits = runner.step_logits(sched.bm, plan, rows)
            sched.update_after_step(plan)
            if rows:
                out = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                tmp = os.path.join(a.out, f".{st['step']}.tmp")
                with open(tmp, "wb") as f:
                    f.write(np.ascontiguousarray(out).tobytes())
                os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
            elif device == "cuda":
                torch.cuda.synchronize()
        for rid in st.get("end", []):
            seq = live.pop(rid, None)
            if seq is not None:
                sched.finish(seq, SeqStatus.FINISHED_STOPPED)
        print(f"done {st['step']}", flush=True)
    ex.shutdown()
    return 0


if __name__ == "__main__":
    sys.exit(main())
