"""Replay a recorded schedule through the engine and write logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

DIR holds config.json and model.safetensors; the model class is chosen from
config.json as `--model DIR` does everywhere else. Steps arrive on standard
input, one JSON object a line:

    {"step": 7, "entries": [{"id": "req-1", "tokens": [11, 4], "want": [1]},
                            {"id": "req-2", "tokens": [9], "want": []}],
     "end": ["req-2"]}

Each step runs exactly the tokens it brings, all entries as one batch, on
the cache pages and state slots earlier steps left (LLMEngine.replay_step:
the engine's allocators, model runner and kernels; nothing is sampled).
For a step that wants logits the fp32 rows go to OUT/<step>.f32 in entry
and `want` order; after every step a line `done <step>` is printed.

The cache pool holds --max-tokens tokens in 64-token pages and there are
four sequence slots, so pages and slots are reused as requests end.

On a fresh checkout the native extensions this model needs are built first
(in-tree, a minute or so).
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def _missing(names):
    import importlib.util
    out = []
    for n in names:
        try:
            if importlib.util.find_spec("dynamo_amd." + n) is None:
                out.append(n)
        except (ImportError, ValueError):
            out.append(n)
    return out


def ensure_built(names):
    """Build the named extensions in-tree if their libraries are absent."""
    need = _missing(names)
    if not need:
        return
    print(f"building {need} (first use)", file=sys.stderr, flush=True)
    env = dict(os.environ, DYNAMO_AMD_EXTS=",".join(need))
    env.setdefault("PYTORCH_ROCM_ARCH", "gfx950")
    subprocess.run([sys.executable, "setup.py", "build_ext", "--inplace"],
                   cwd=ROOT, env=env, check=True, stdout=sys.stderr)
    import importlib
    importlib.invalidate_caches()
    left = _missing(names)
    if left:
        raise RuntimeError(f"extensions {left} did not build")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"],
                    default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--device", default="auto",
                    help="cuda:0 when a GPU is present, else cpu")
    ap.add_argument("--slots", type=int, default=4,
                    help="sequences that may be live at once")
    a = ap.parse_args(argv)

    import torch
    device = a.device
    if device == "auto":
        device = "cuda:0" if torch.cuda.is_available() else "cpu"
    ensure_built(["_core"])      # the engine package itself imports it
    from dynamo_amd.models.registry import (native_extensions,
                                            resolve_model_config)
    model = resolve_model_config(a.model)
    ensure_built(native_extensions(model, device))

    if a.dtype == "float32":
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")

    from dynamo_amd.engine import EngineConfig, LLMEngine
    page = 64
    cfg = EngineConfig(
        model=model, device=device, dtype=a.dtype, page_size=page,
        max_num_seqs=a.slots, max_model_len=model.max_position,
        max_batched_tokens=max(a.max_tokens, page),
        kv_pool_pages=max(1, -(-a.max_tokens // page)),
        enable_prefix_caching=False, enable_hip_graphs=False, kv_events=False)
    eng = LLMEngine(cfg)
    os.makedirs(a.out, exist_ok=True)

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", []))
                   for e in step["entries"]]
        logits = eng.replay_step(entries, step.get("end", []))
        if logits is not None and logits.shape[0]:
            data = logits.float().cpu().contiguous().numpy().astype("<f4")
            path = os.path.join(a.out, f"{step['step']}.f32")
            with open(path + ".part", "wb") as f:
                f.write(data.tobytes())
            os.replace(path + ".part", path)
        print(f"done {step['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
