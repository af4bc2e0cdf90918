"""Command line: generate token ids with any model the engine serves.

    python -m qwen_inference_engine_amd.cli --model DIR_OR_PRESET --prompt 1,2,3 --gen 32

--model is a folder with config.json (+ model.safetensors for a layered design; the model class
is chosen by the config, spec.spec_from_config) or the name of a Qwen preset (synthetic weights,
--synthetic SEED).  Requests run through the ContinuousBatcher: several --prompt options are
served together.  Prints one line ``tokens[<i>]: ...`` per request.
"""
from __future__ import annotations

import argparse
import os
import sys


def _ids(text: str):
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="qie", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--prompt", action="append", default=[], help="token ids, comma or space separated (repeatable)")
    ap.add_argument("--prompt-file", action="append", default=[], help="a file of token ids (repeatable)")
    ap.add_argument("--gen", type=int, default=16, help="tokens to generate per request")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--top-k", type=int, default=1)
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--synthetic", type=int, default=5, help="seed of the synthetic weights of a preset")
    ap.add_argument("--slots", type=int, default=4)
    ap.add_argument("--max-ctx", type=int, default=0)
    ap.add_argument("--page-tokens", type=int, default=0)
    ap.add_argument("--chunk-tokens", type=int, default=512)
    ap.add_argument("--stop", type=int, action="append", default=[])
    ap.add_argument("--device", type=int, default=0)
    a = ap.parse_args(argv)
    prompts = [_ids(p) for p in a.prompt] + [_ids(open(f).read()) for f in a.prompt_file]
    if not prompts:
        ap.error("give --prompt or --prompt-file")
    from . import spec as S
    from .engine import Engine, Sampling
    from .scheduler import ContinuousBatcher
    from .weights import SynthParams
    need = max(len(p) for p in prompts) + a.gen + 2
    if os.path.isdir(a.model):
        spec = S.spec_from_dir(a.model)
    elif a.model in S.PRESETS:
        spec = S.PRESETS[a.model]
    else:
        ap.error(f"--model: neither a folder nor one of {sorted(S.PRESETS)}")
    layered = isinstance(spec, S.LayeredSpec)
    page = a.page_tokens or (64 if layered else 128)
    max_ctx = a.max_ctx or -(-need // page) * page
    if layered:
        eng = Engine(spec, device=a.device, max_ctx=max_ctx, dtype=a.dtype).load_dir(a.model)
    else:
        eng = Engine(spec, device=a.device, max_ctx=max_ctx).init_synthetic(SynthParams(seed=a.synthetic))
    smp = Sampling(top_k=a.top_k, temperature=a.temperature, top_p=a.top_p, seed=a.seed)
    cb = ContinuousBatcher(eng, slots=min(a.slots, 8) if not layered else a.slots, max_ctx=max_ctx, page_tokens=page,
                           sampling=smp, chunk_tokens=a.chunk_tokens)
    rids = [cb.submit(p, a.gen, a.stop) for p in prompts]
    out = cb.run()
    for i, rid in enumerate(rids):
        print(f"tokens[{i}]:", " ".join(str(t) for t in out[rid]))
    sys.stdout.flush()
    cb.close()
    eng.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
