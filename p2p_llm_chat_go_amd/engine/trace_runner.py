"""Replay a trace of steps through an engine and write the logits it produces.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object per line,

    {"step": 7, "entries": [{"id": "r1", "tokens": [40, 2, 91, 8], "want": [3]}, {"id": "r2", "tokens": [12], "want": [0]}], "end": ["r2"]}

``entries``: per request its next tokens and the places among them whose logits are wanted;
``end``: requests that are finished after the step (their pages and state slot go back to
the pool).  All entries of a step run as one batch through the engine's step function.  For
a step with wanted places the fp32 logits [wanted, vocab] are written to ``<out>/<step>.f32``
(little endian, entry order); after every step ``done <step>`` is printed.  Nothing is
sampled.  The cache pool holds ``--max-tokens`` tokens in pages and ``--slots`` sequences.
Exit code 3: the model's engine does not run in the requested number format.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="tokens the cache pool holds (each live request rounded up to a page)")
    ap.add_argument("--slots", type=int, default=4, help="live requests at most")
    ap.add_argument("--device", default=None, help="cuda:N (default) or cpu")
    a = ap.parse_args(argv)

    import torch

    from ..models import registry
    from ..ops import PAGE

    dtype = torch.float32 if a.dtype == "float32" else torch.bfloat16
    if not registry.supports_dtype(a.model, dtype):
        print("this model's engine does not run in %s" % a.dtype, file=sys.stderr)
        return 3
    if not registry.is_hybrid_dir(a.model):
        print("trace replay drives engines with a step function over a sequence cache "
              "(hybrid models)", file=sys.stderr)
        return 2
    dev = a.device or ("cuda:0" if torch.cuda.is_available() else "cpu")
    if str(dev).startswith("cuda"):
        from ..ops import seqmix

        seqmix.lib()  # compiles the kernels of these models on first use
    cfg, weights = registry.load_checkpoint(a.model, dev, dtype)
    pages = (a.max_tokens + PAGE - 1) // PAGE + 1   # + the null page
    eng = registry.make_engine(cfg, weights, dev, kv_pages=pages, num_slots=a.slots,
                               max_batch=a.slots, dtype=dtype)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", [])) for e in st["entries"] if e["tokens"]]
        logits = eng.step(entries) if entries else None
        if logits is not None:
            data = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4")
            tmp = os.path.join(a.out, ".%d.part" % st["step"])
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(a.out, "%d.f32" % st["step"]))
        for key in st.get("end", []):
            if key in eng.cache:
                eng.release(key)
        sys.stdout.write("done %d\n" % st["step"])
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
