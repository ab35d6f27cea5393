"""Trace replay: feed GIVEN token ids through the engine, step by step,
and write the logits at requested places.  Nothing is sampled.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR \\
                  --max-tokens N

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3],
                             "want": [0, 2]}], "end": ["a"]}

`entries` lists, per request, its next tokens and which of them need
logits; all entries of a step run as ONE engine batch (prompt portions
beside single decoded tokens) from the cache and state earlier steps
left.  `end` names requests whose slot and pages are given back after
the step.  For a step that wants logits, OUT/<step>.f32 holds them as
little-endian fp32 [wanted, vocab] in entry/want order; every step is
answered with a flushed line `done <step>`.

The replay drives LLMEngine.replay_step: the engine's own model, batch
assembly, block manager, state slots and kernels — the ones its
generation loop uses.  The page pool is sized from --max-tokens (the
most tokens live at once, per request rounded up to 64) and there are
four sequence slots, so pages and slots are recycled during a trace.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

REPLAY_SLOTS = 4


def build_engine(model_dir: str, dtype: str, max_tokens: int):
    from .config import EngineConfig
    from .engine import LLMEngine
    from .models.registry import model_config_from_dir

    model_cfg = model_config_from_dir(model_dir)
    block = 16
    cfg = EngineConfig(
        model=model_cfg,
        block_size=block,
        # +1: page 0 is the engine's reserved scratch page
        num_gpu_blocks=(max_tokens + block - 1) // block + 1,
        max_num_seqs=REPLAY_SLOTS,
        max_batched_tokens=1 << 30,
        max_model_len=1 << 30,
        use_hip_graphs=False,
        enforce_eager=True,
        weights_path=model_dir,
        dtype=dtype,
    )
    return LLMEngine(cfg)


def run(engine, out_dir: str, lines, reply) -> None:
    import numpy as np

    ids = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        feeds, want = [], {}
        for e in step["entries"]:
            if e["id"] not in ids:
                ids[e["id"]] = engine.open_stream()
            sid = ids[e["id"]]
            if not e["tokens"]:
                continue             # admitted, nothing to run yet
            feeds.append((sid, e["tokens"]))
            want[sid] = e.get("want") or []
        n_want = sum(len(w) for w in want.values())
        if feeds:
            logits = engine.replay_step(feeds, want)
            if n_want:
                arr = logits.detach().to("cpu").numpy().astype("<f4")
                tmp = os.path.join(out_dir, f".{step['step']}.part")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir,
                                             f"{step['step']}.f32"))
        elif n_want:
            np.zeros((0,), dtype="<f4").tofile(
                os.path.join(out_dir, f"{step['step']}.f32"))
        for name in step.get("end") or []:
            if name in ids:
                engine.close_stream(ids.pop(name))
        reply(f"done {step['step']}")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.
                                 RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"),
                    default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    engine = build_engine(a.model, a.dtype, a.max_tokens)

    def reply(text: str) -> None:
        sys.stdout.write(text + "\n")
        sys.stdout.flush()

    run(engine, a.out, sys.stdin, reply)
    return 0


if __name__ == "__main__":
    sys.exit(main())
