"""Trace replay: feeds given token ids through a model step by step and writes the logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object a line,
``{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}``:
every entry continues its request with the next tokens (a request is admitted into a free slot
at its first entry), ``want`` names the places among these tokens whose logits are written, as
float32 [wanted, vocab] in entry order, to ``<out>/<step>.f32``; requests listed in ``end``
give their slot and cache pages back after the step.  After every step the line
``done <step>`` is printed.  All entries of a step run as ONE engine step (Batch.step): portions
of prompts beside single tokens.  Nothing is sampled.

The cache pool holds --max-tokens tokens (each request rounded up to whole pages of 64) and the
batch has four slots.  The library is built at the first call when it is missing.
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys

PAGE_TOKENS = 64
SLOTS = 4


def ensure_library() -> None:
    from . import _lib
    if os.path.exists(_lib.LIB_PATH):
        return
    csrc = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
    jobs = str(max(1, min(16, os.cpu_count() or 4)))
    subprocess.check_call(["make", "-s", "-j", jobs, "-C", csrc, "lib"], stdout=sys.stderr, stderr=sys.stderr)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--device", type=int, default=0)
    a = ap.parse_args(argv)

    from .spec import LayeredSpec, spec_from_dir
    spec = spec_from_dir(a.model)
    if not isinstance(spec, LayeredSpec):
        if a.dtype == "float32":
            print("trace_run: this model class has no float32 path", file=sys.stderr)
            return 3
        print("trace_run: this model class has no ragged step; use the generation entry points", file=sys.stderr)
        return 2
    ensure_library()
    from .engine import Engine
    pages = -(-a.max_tokens // PAGE_TOKENS)
    max_ctx = max(pages * PAGE_TOKENS, 2 * PAGE_TOKENS)
    eng = Engine(spec, device=a.device, max_ctx=max_ctx, dtype=a.dtype).load_dir(a.model)
    batch = eng.batch(SLOTS, max_ctx, page_tokens=PAGE_TOKENS, n_pages=pages + 1)   # + the scratch page
    os.makedirs(a.out, exist_ok=True)
    slot_of = {}
    free = list(range(SLOTS - 1, -1, -1))
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries, want, row0 = [], [], 0
        for en in st["entries"]:
            rid = en["id"]
            if rid not in slot_of:
                if not free:
                    raise RuntimeError(f"step {st['step']}: more than {SLOTS} live requests")
                slot_of[rid] = free.pop()
            if not en["tokens"]:                # admitted, nothing to run yet
                continue
            entries.append((slot_of[rid], en["tokens"]))
            want += [row0 + int(w) for w in en.get("want", ())]
            row0 += len(en["tokens"])
        if entries:
            logits = batch.step(entries, want)
            if want:
                tmp = os.path.join(a.out, f".{st['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(logits.astype("<f4", copy=False).tobytes())
                os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        for rid in st.get("end", ()):
            if rid in slot_of:
                s = slot_of.pop(rid)
                batch.release(s)
                free.append(s)
        sys.stdout.write(f"done {st['step']}\n")
        sys.stdout.flush()
    batch.close()
    eng.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
