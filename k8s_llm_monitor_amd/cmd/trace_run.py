"""Trace replay: feed given token ids through the engine step by step and write the logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

``DIR`` holds ``config.json`` and ``model.safetensors``.  Steps arrive on standard input, one JSON
object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}

Each entry gives a request's NEXT tokens (a request is admitted at its first entry) and ``want``,
the places among these tokens whose logits are asked for; ``end`` lists requests that are finished
after the step (their pages and state slot return to the pools).  All entries of a step run as ONE
engine step: an entry of a single token of a request that already holds tokens is a decode row, the
others are prompt chunks (a mixed step when both occur; a step of decode rows only goes through
the decode path).  For a step with wanted places ``<out>/<step>.f32`` receives the logits
[wanted, vocab] as little-endian fp32, in entry then ``want`` order; after every step the line
``done <step>`` is printed.

Nothing is sampled and the scheduler's policy is bypassed (the trace IS the schedule); the model,
the model runner's step functions, the block manager with its page pool and state slots and the
kernels are the serving engine's.  The page pool holds ``--max-tokens`` tokens and there are four
sequence slots.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

MAX_SEQS = 4


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="replay a step trace through the engine and write logits")
    ap.add_argument("--model", required=True, help="directory with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="directory for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the page pool holds")
    ap.add_argument("--device", default=None, help="default: cuda if present")
    ap.add_argument("--graphs", action="store_true", help="replay decode-only steps from captured hipGraphs")
    a = ap.parse_args(argv)

    import numpy as np
    import torch

    from ..engine import EngineConfig, LLMEngine
    from ..engine.runner import BLOCK_SIZE
    from ..engine.sequence import SamplingParams, Sequence

    torch.backends.cuda.matmul.allow_tf32 = False  # float32 means float32
    torch.backends.cudnn.allow_tf32 = False
    dev = a.device or ("cuda" if torch.cuda.is_available() else "cpu")
    nb = (a.max_tokens + BLOCK_SIZE - 1) // BLOCK_SIZE
    eng = LLMEngine(EngineConfig(model=a.model, weights=a.model, dtype=a.dtype, max_num_seqs=MAX_SEQS,
                                 max_model_len=1 << 30, num_blocks=nb, use_graphs=a.graphs, keep_logits=True, sample=False,
                                 prefix_caching=False, pipeline=False), device=dev)
    if getattr(eng.model, "uses_tile_gemm", False) and dev != "cpu":
        from ..ops import build

        build.ensure(("ops",))  # large steps of this model's experts run on the prefill tile GEMM
    if a.graphs:
        eng.warmup()
    runner, blocks = eng.runner, eng.blocks
    os.makedirs(a.out, exist_ok=True)
    live: dict = {}
    greedy = SamplingParams(temperature=0.0)
    with torch.no_grad():
        for line in sys.stdin:
            line = line.strip()
            if not line:
                continue
            st = json.loads(line)
            chunks, decode, wants = [], [], {}
            for e in st["entries"]:
                q = live.get(e["id"])
                if q is None:
                    q = live[e["id"]] = Sequence(prompt_ids=[], params=greedy, request_id=str(e["id"]))
                    if len(live) > MAX_SEQS or not blocks.admit(q):
                        raise RuntimeError(f"step {st['step']}: no free sequence slot for {e['id']!r}")
                toks = [int(t) for t in e["tokens"]]
                if not toks:
                    continue
                have = q.num_tokens
                if not blocks.ensure_tokens(q, have + len(toks)):
                    raise RuntimeError(f"step {st['step']}: page pool exhausted at {e['id']!r}")
                q.prompt_ids.extend(toks)
                q.num_computed = have
                wants[id(q)] = list(e.get("want", []))
                if len(toks) == 1 and have > 0:
                    decode.append(q)
                else:
                    q.chunk = len(toks)
                    chunks.append(q)
            rows = decode + chunks
            logits = None
            if chunks:
                h = runner.prefill_launch(chunks, decode, logit_rows=[wants[id(q)] for q in rows])
                logits = h.logits
            elif decode:
                runner.decode_collect(runner.decode_launch(decode))
                keep = [i for i, q in enumerate(decode) if wants[id(q)]]
                logits = runner.last_logits[keep] if keep else None
            for q in chunks:
                q.num_computed += q.chunk
                q.chunk = 0
            order = {id(q): i for i, q in enumerate(rows)}
            if logits is not None and logits.shape[0]:
                # rows come back decode rows first; the file wants the entries' order
                parts, o = {}, 0
                for q in rows:
                    n = len(wants[id(q)])
                    parts[id(q)] = (o, n)
                    o += n
                sel = []
                for e in st["entries"]:
                    q = live[e["id"]]
                    if id(q) in order and e["tokens"]:
                        o, n = parts[id(q)]
                        sel += list(range(o, o + n))
                arr = logits.float()[sel].cpu().numpy().astype("<f4")
                tmp = os.path.join(a.out, ".%s.part" % st["step"])
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(a.out, "%s.f32" % st["step"]))
            elif dev != "cpu":
                torch.cuda.synchronize()
            for i in st.get("end", []):
                q = live.pop(i, None)
                if q is not None:
                    blocks.free(q)
            sys.stdout.write("done %s\n" % st["step"])
            sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
