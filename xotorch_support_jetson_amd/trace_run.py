"""Replay recorded traffic through the serving runner and write the logits it is asked for.

  bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

DIR holds config.json + safetensors; the model class comes from config.json as everywhere in the framework
(models.config.load_config).  Steps arrive on standard input, one JSON object a line:

  {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["b"]}

Each step is ONE batched forward of the ShardRunner the engine serves with (paged KV pool, state slots, HIP-graph
decode for steps of single tokens): every entry's tokens continue that request from what earlier steps left in
the cache; "want" lists the token places of the entry whose logits go to OUT/<step>.f32 (little-endian fp32
[wanted, vocab], in entry order); "end" lists requests whose pages and state slot are returned after the step.
After every step a line "done <step>" is printed.  Nothing is sampled.

The KV pool is sized for --max-tokens live tokens (each request rounded up to whole pages) and four state slots:
requests beyond that have to wait for pages and slots given back.

Exit code 3: --dtype float32 asked of an architecture that serves in bfloat16 only.
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
MAX_LIVE = 4  # state slots / batch rows


def ensure_built() -> None:
  """Build the in-tree kernel library and host runtime when they are missing (a fresh checkout)."""
  pkg = Path(__file__).resolve().parent
  if list(pkg.glob("_C*.so")) and list(pkg.glob("_runtime*.so")):
    return
  env = dict(os.environ)
  env.setdefault("PYTORCH_ROCM_ARCH", "gfx950")
  print("building the kernel library (first call in this checkout) ...", file=sys.stderr, flush=True)
  subprocess.run([sys.executable, "setup.py", "build_ext", "--inplace"], cwd=str(ROOT), env=env, check=True,
                 stdout=sys.stderr)


def main(argv=None) -> int:
  ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
  ap.add_argument("--model", required=True)
  ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
  ap.add_argument("--out", required=True)
  ap.add_argument("--max-tokens", type=int, required=True)
  ap.add_argument("--device", default=None, help="default: the GPU when there is one")
  a = ap.parse_args(argv)

  import torch
  dev = torch.device(a.device) if a.device else torch.device("cuda:0" if torch.cuda.is_available() else "cpu")
  if dev.type == "cuda":
    ensure_built()
  from .inference.shard import Shard
  from .models.config import load_config
  from .models.weights import load_hf_weights
  from .runtime.runner import PAGE, ShardRunner

  cfg = load_config(a.model)
  dtype = getattr(torch, a.dtype)
  if dtype != torch.bfloat16 and not cfg.is_mixed:
    print(f"{cfg.model_type} serves in bfloat16 only", file=sys.stderr)
    return 3
  if dtype == torch.float32:
    torch.backends.cuda.matmul.allow_tf32 = False
  shard = Shard(Path(a.model).name or "model", 0, cfg.num_layers - 1, cfg.num_layers)
  weights = load_hf_weights(a.model, cfg, shard, dev, dtype)
  pages = -(-a.max_tokens // PAGE)
  runner = ShardRunner(cfg, shard, dev, weights=weights, num_pages=pages, max_batch=MAX_LIVE,
                       max_ctx=max(pages * PAGE, PAGE), **({"dtype": dtype} if cfg.is_mixed else {}))
  os.makedirs(a.out, exist_ok=True)
  for line in sys.stdin:
    line = line.strip()
    if not line:
      continue
    step = json.loads(line)
    rids, qlens, toks, rows, base = [], [], [], [], 0
    for e in step.get("entries", []):
      if not e["tokens"]:
        continue
      rids.append(str(e["id"]))
      qlens.append(len(e["tokens"]))
      toks += e["tokens"]
      rows += [base + int(p) for p in e.get("want", [])]
      base += len(e["tokens"])
    if rids:
      x = torch.tensor(toks, dtype=torch.int32)
      if rows:
        logits = runner.forward(rids, qlens, x, logit_rows=rows)
        with open(os.path.join(a.out, f"{step['step']}.f32"), "wb") as f:
          f.write(logits.float().cpu().contiguous().numpy().astype("<f4").tobytes())
      else:
        runner.forward(rids, qlens, x)
        if dev.type == "cuda":
          torch.cuda.synchronize()
    for rid in step.get("end", []):
      runner.free(str(rid))
    print(f"done {step['step']}", flush=True)
  return 0


if __name__ == "__main__":
  sys.exit(main())
