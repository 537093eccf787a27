"""Tarepel in the framework against the plain implementation in tests/tarepel_oracle.py.

Every test makes its own small configuration and random checkpoint tensors, runs them through the serving runner
(paged KV pool, state slots, batched steps; HIP kernels and HIP-graph decode on a GPU, the torch twins on the CPU)
and compares logits at every position with the oracle's token-by-token float64 run.  Each body runs on the CPU and,
marked gpu, on cuda:0 in float32 and bfloat16.
"""
import asyncio
import copy
import math

import numpy as np
import pytest
import torch

from tarepel_oracle import Oracle
from xotorch_support_jetson_amd.inference.shard import Shard
from xotorch_support_jetson_amd.models.config import TINY_TAREPEL, from_hf_config
from xotorch_support_jetson_amd.models.weights import mixed_weights, random_mixed_tensors
from xotorch_support_jetson_amd.runtime.runner import ShardRunner

RUNS = [pytest.param("cpu", torch.float32, id="cpu-f32"),
        pytest.param("cuda:0", torch.float32, id="gpu-f32", marks=pytest.mark.gpu),
        pytest.param("cuda:0", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]
TOL = {torch.float32: 2e-4, torch.bfloat16: 6e-2}


def attn(heads=4, kv=2, dim=32, chunk=48, rot=16, base=10000.0, scale=0.2):
  return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "mask": {"size": chunk},
          "rot": {"base": base, "dims": rot}, "scale": scale}


def delta(heads=4, kv=2, dim=16, vdim=32, conv=3):
  return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def par(left, right, ff=96, ls=0.7, rs=0.9):
  return {"type": "parallel", "mlp": {"kind": "dense", "ff": ff} if ff else None,
          "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}}


def gla(heads=2, dim=32, vdim=64, tau=8.0, ff=64):
  return {"type": "gla", "mlp": {"kind": "dense", "ff": ff} if ff else None,
          "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}}


def config(layers, width=64, vocab=96, logit_scale=0.5, eps=1e-5):
  return {"architecture": "Tarepel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
          "layers": layers}


SMALL = config([par(attn(), delta()), gla(), gla(heads=4, dim=16, vdim=16, tau=3.0, ff=0),
                par(attn(heads=2, kv=2, dim=64, chunk=64, rot=64, base=5e4, scale=0.125), delta(2, 1, 32, 16, 4), ff=0)])


class Rig:
  """A configuration + random tensors in the runner and in the oracle."""

  def __init__(self, cfg, dev, dtype, seed=1, pages=24, slots=4, tweak=None, graphs=None):
    self.cfg, self.dev, self.dtype = cfg, torch.device(dev), dtype
    self.c = from_hf_config(cfg)
    self.tensors = random_mixed_tensors(self.c, seed)
    if tweak:
      tweak(self.tensors)
    self.oracle = Oracle(cfg, self.tensors)
    shard = Shard("t", 0, self.c.num_layers - 1, self.c.num_layers)
    w = mixed_weights(self.c, shard, self.tensors.__getitem__, self.dev, dtype)
    self.runner = ShardRunner(self.c, shard, self.dev, weights=w, num_pages=pages, max_batch=slots, max_ctx=pages * 64,
                              dtype=dtype, use_graphs=graphs)
    self.V = self.c.vocab_size

  def tokens(self, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, self.V, (n,), generator=g).tolist()

  def step(self, entries):
    """entries [(rid, tokens)] -> logits of every token of the step, split per entry."""
    rids = [r for r, _ in entries]
    qlens = [len(t) for _, t in entries]
    flat = [t for _, ts in entries for t in ts]
    out = self.runner.forward(rids, qlens, torch.tensor(flat, dtype=torch.int32), logit_rows=list(range(len(flat))))
    return list(out.double().cpu().split(qlens))

  def run_alone(self, rid, toks, cuts):
    """One request in portions of the given sizes (the last size repeats); logits at every position."""
    outs, lo, i = [], 0, 0
    while lo < len(toks):
      n = min(cuts[min(i, len(cuts) - 1)], len(toks) - lo)
      outs.append(self.step([(rid, toks[lo:lo + n])])[0])
      lo, i = lo + n, i + 1
    self.runner.free(rid)
    return torch.cat(outs)

  def check(self, got, toks, what=""):
    want = self.oracle.logits(toks)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
    worst = int(err.argmax())
    assert err.max() < TOL[self.dtype], f"{what}: position {worst} of {len(toks)} is off by {float(err.max()):.3g}"


# ------------------------------------------------------------------ whole prompts, portions, decoding
@pytest.mark.parametrize("dev,dtype", RUNS)
def test_whole_prompt(dev, dtype):
  rig = Rig(SMALL, dev, dtype)
  toks = rig.tokens(150, 3)
  rig.check(rig.run_alone("a", toks, [len(toks)]), toks, "whole prompt")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_first_tokens(dev, dtype):
  """Sequences of one, two and three tokens: empty history for the convolutions, the state and the cache."""
  rig = Rig(SMALL, dev, dtype)
  for n in (1, 2, 3):
    toks = rig.tokens(n, 10 + n)
    rig.check(rig.run_alone("a", toks, [n]), toks, f"{n}-token prompt")
    rig.check(rig.run_alone("a", toks, [1]), toks, f"{n} tokens one by one")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_prefill_against_decoding(dev, dtype):
  rig = Rig(SMALL, dev, dtype)
  toks = rig.tokens(140, 4)
  whole = rig.run_alone("a", toks, [len(toks)])
  single = rig.run_alone("b", toks, [1])
  rig.check(single, toks, "token by token")
  assert (whole - single).abs().max() < TOL[dtype] * whole.abs().max()


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("cuts", [[2], [3, 2, 5, 1, 1, 7], [47, 1, 1, 17, 2], [64, 64, 1], [63, 2, 63, 1], [100, 1]])
def test_portions(dev, dtype, cuts):
  """A prompt cut anywhere (inside pages, chunks and convolution windows, down to two tokens)."""
  rig = Rig(SMALL, dev, dtype)
  toks = rig.tokens(135, 5)
  rig.check(rig.run_alone("a", toks, cuts), toks, f"portions {cuts}")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_long_decoding(dev, dtype):
  """A short prompt, then 200 single tokens: several pages and chunks are crossed while decoding."""
  rig = Rig(SMALL, dev, dtype)
  toks = rig.tokens(215, 6)
  rig.check(rig.run_alone("a", toks, [15, 1]), toks, "long decoding")


# ------------------------------------------------------------------ batches, pages and slots
@pytest.mark.parametrize("dev,dtype", RUNS)
def test_mixed_batches_match_alone(dev, dtype):
  """Unequal requests in one step (portions beside single tokens, a request that sits a step out) give each the
  logits it gets alone."""
  rig = Rig(SMALL, dev, dtype, pages=12)
  seqs = {"a": rig.tokens(130, 21), "b": rig.tokens(70, 22), "c": rig.tokens(9, 23), "d": rig.tokens(40, 24)}
  plan = [[("a", 50), ("b", 2)], [("a", 1), ("b", 30), ("c", 9)], [("a", 1), ("d", 17)], [("a", 40), ("b", 1), ("d", 1)],
          [("b", 37), ("d", 22)], [("a", 38)]]
  at = {k: 0 for k in seqs}
  got = {k: [] for k in seqs}
  for stepplan in plan:
    entries = [(r, seqs[r][at[r]:at[r] + n]) for r, n in stepplan]
    for (r, n), o in zip(stepplan, rig.step(entries)):
      got[r].append(o)
      at[r] += n
      if at[r] == len(seqs[r]):
        rig.runner.free(r)
  for r, toks in seqs.items():
    assert at[r] == len(toks)
    rig.check(torch.cat(got[r]), toks, f"request {r} in mixed batches")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_pages_and_slots_are_reused(dev, dtype):
  """A pool of four pages and two state slots serves six requests in turn, two at a time: every page and slot is
  handed out again with another request's keys and state in it."""
  rig = Rig(SMALL, dev, dtype, pages=4, slots=2)
  for rnd in range(3):
    seqs = {f"r{rnd}x": rig.tokens(100 + rnd, 30 + rnd), f"r{rnd}y": rig.tokens(90 - rnd, 40 + rnd)}
    got = {k: [] for k in seqs}
    for lo in range(0, 128, 16):
      entries = [(r, t[lo:lo + 16]) for r, t in seqs.items() if t[lo:lo + 16]]
      if not entries:
        break
      for (r, _), o in zip(entries, rig.step(entries)):
        got[r].append(o)
    for r, toks in seqs.items():
      rig.runner.free(r)
      rig.check(torch.cat(got[r]), toks, f"round {rnd} request {r}")
  assert rig.runner.bm.num_free == 4 and rig.runner.sm.num_free == 2


def test_slots_run_out_and_come_back():
  rig = Rig(SMALL, "cpu", torch.float32, pages=8, slots=2)
  rig.step([("a", [1, 2]), ("b", [3])])
  assert not rig.runner.can_admit("c", 1)
  with pytest.raises(RuntimeError, match="state slots"):
    rig.step([("c", [4])])
  rig.runner.free("a")
  assert rig.runner.can_admit("c", 1)


# ------------------------------------------------------------------ other sizes
SIZES = [
  # one head everywhere, kv_heads == heads, full rotation, chunk of one page, two taps
  config([par(attn(1, 1, 32, 64, 32), delta(1, 1, 32, 32, 2)), gla(1, 16, 16, 1.0)], width=48, vocab=50, logit_scale=1.0),
  # rotation on a quarter of the head, chunk shorter than a page and not dividing it, wide heads, five taps
  config([par(attn(6, 3, 128, 40, 32, 1e6, 0.09), delta(6, 2, 64, 48, 5), ff=160, ls=1.3, rs=0.4), gla(3, 64, 128, 16.0)],
         width=160, vocab=130),
  # chunk longer than a page, no rotation at all, key dim above value dim, a layer without feed-forward first
  config([gla(2, 48, 16, 2.0, ff=0), par(attn(2, 1, 16, 100, 0), delta(3, 3, 48, 16, 4), ff=32)], width=32, vocab=40),
  # a chunk of two tokens and a chunk of one
  config([par(attn(2, 2, 16, 2, 8), delta(2, 1, 16, 16, 3)), par(attn(2, 1, 16, 1, 16), delta(2, 2, 8, 24, 4))], width=40),
]


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("n", range(len(SIZES)))
def test_other_sizes(dev, dtype, n):
  rig = Rig(SIZES[n], dev, dtype, seed=50 + n)
  toks = rig.tokens(210 if n == 2 else 90, 60 + n)
  rig.check(rig.run_alone("a", toks, [33, 2, 1, 1, 29, 1]), toks, f"sizes {n}")


# ------------------------------------------------------------------ faults that random weights would hide
def _edge_rig(dev, dtype, chunk, mark):
  """One attention layer whose query at the last position and key at position `mark` are scaled so that this one
  score stands out (its weight is ~1 where all others are ~0.02): seeing or not seeing that key moves the logits."""
  cfg = config([par(attn(2, 1, 32, chunk, 16, scale=0.25), delta(2, 1, 16, 16, 3), ff=0, ls=1.0, rs=0.05)], width=64, vocab=64)
  c = from_hf_config(cfg)
  t = random_mixed_tensors(c, 7)
  t["l0.mix.left.pb"] = torch.full((2,), -4.0)
  t["l0.ls1"] = torch.full((64,), 1.0)
  return cfg, t


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("chunk,n", [(48, 48), (48, 49), (48, 96), (48, 97), (64, 64), (64, 65), (100, 100), (100, 101),
                                     (100, 129), (100, 201)])
def test_chunk_edges(dev, dtype, chunk, n):
  """The last token is the last of its chunk (n a multiple of the chunk: it sees chunk keys) or the first of the
  next (n one more: it sees itself only).  The sequence repeats one token, so every key matches the query and a
  key let in from the wrong side of the edge counts in full; the oracle agrees position by position, in a prompt,
  in portions that straddle the edge, and token by token."""
  cfg, t = _edge_rig(dev, dtype, chunk, 0)
  rig = Rig(cfg, dev, dtype, tweak=lambda d: d.update(t))
  toks = [5] * n
  rig.check(rig.run_alone("a", toks, [n]), toks, "prompt")
  rig.check(rig.run_alone("a", toks, [n - 3, 2, 1]), toks, "portions over the edge")
  rig.check(rig.run_alone("a", toks, [max(n - 40, 1), 1]), toks, "decoding over the edge")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_far_token_lives_in_the_state(dev, dtype):
  """Decays pushed to ~1 - 1e-4 and a first token unlike all later ones: 400 tokens on, the read-out still holds the
  first token's write; a state that was dropped, cleared or attached to the wrong slot changes the last logits."""
  cfg = config([gla(2, 32, 32, 4.0, ff=0), par(attn(2, 1, 16, 32, 16), delta(2, 1, 32, 32, 4), ff=0, ls=0.1, rs=1.0)])

  def tweak(t):
    t["l0.mix.a2.b"] = torch.full_like(t["l0.mix.a2.b"], 9.0)
    t["l0.mix.a2"] = t["l0.mix.a2"] * 0.01
    t["l1.mix.right.A_log"] = torch.full_like(t["l1.mix.right.A_log"], -9.0)
    t["embed"][0] = t["embed"][0] * 6.0
  rig = Rig(cfg, dev, dtype, tweak=tweak, pages=16)
  toks = [0] + [1 + (i * 7) % 90 for i in range(420)]
  got = rig.run_alone("a", toks, [200, 1, 1, 150, 2, 1])
  rig.check(got, toks, "far token")
  other = rig.oracle.logits([3] + toks[1:], want=[len(toks) - 1])[0]  # the same run without that first token
  gap = (other - rig.oracle.logits(toks, want=[len(toks) - 1])[0]).abs().max()
  if dtype == torch.float32:  # (bf16 rounding is of the first token's size here: the fp32 runs carry this check)
    assert gap > 30 * TOL[dtype] * got[-1].abs().max(), "the first token must matter at the end for this test to bite"


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_convolution_history_across_portions(dev, dtype):
  """Five taps and portions shorter than the taps: the convolution reads inputs of two and three steps back."""
  cfg = config([par(attn(2, 1, 16, 32, 16), delta(2, 2, 16, 16, 5), ff=0, ls=0.1, rs=1.5)], width=32)
  rig = Rig(cfg, dev, dtype)
  toks = rig.tokens(40, 70)
  rig.check(rig.run_alone("a", toks, [1, 2, 1, 1, 3, 2, 4, 1]), toks, "short portions")


# ------------------------------------------------------------------ the engine's own entry point
@pytest.mark.parametrize("dev", ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_engine(dev):
  """Three prompts of unequal length at once through ShardedInferenceEngine (queue, batched steps, sampler at
  temperature 0): every token drawn is the oracle's greedy token for the text so far (ties within rounding
  aside), and slots and pages are all free at the end."""
  from xotorch_support_jetson_amd.download.shard_download import NoopShardDownloader
  from xotorch_support_jetson_amd.inference.sharded_engine import ShardedInferenceEngine
  from xotorch_support_jetson_amd.models.config import preset
  c = preset("tiny-tarepel")
  oracle = Oracle(TINY_TAREPEL, random_mixed_tensors(c, 0))
  shard = Shard("tiny-tarepel", 0, c.num_layers - 1, c.num_layers)
  prompts = {"p0": [7, 3, 99, 42, 5, 17], "p1": [11] * 53, "p2": [200, 1]}
  steps = 24

  async def one(e, rid, ids):
    out, st = await e.infer_tensor(rid, shard, np.array([ids]), {"temperature": 0.0})
    seq = list(ids)
    for _ in range(steps):
      tok = int(np.asarray(await e.sample(out, temp=0.0)).reshape(-1)[0])
      seq.append(tok)
      out, st = await e.infer_tensor(rid, shard, np.array([[tok]]), dict(st, temperature=0.0))
    await e.finish_request(rid)
    return seq

  async def main():
    e = ShardedInferenceEngine(NoopShardDownloader(), device=torch.device(dev))
    seqs = await asyncio.gather(*[one(e, r, p) for r, p in prompts.items()])
    return e, seqs
  e, seqs = asyncio.run(main())
  assert e.runner.sm.num_free == e.runner.sm.slots and e.runner.bm.num_free == e.runner.bm.num_blocks
  assert e.prefix_cache is None
  for (rid, p), seq in zip(prompts.items(), seqs):
    lg = oracle.logits(seq[:-1])
    for t in range(len(p) - 1, len(seq) - 1):
      best = float(lg[t].max())
      assert float(lg[t][seq[t + 1]]) >= best - 0.05 * float(lg[t].std()), f"{rid}: token {t + 1} is not the greedy one"


def test_checkpoint_directory_through_registry_and_engine(tmp_path):
  """config.json + model.safetensors (bf16) in a folder: registered as a local model, loaded by the engine's own
  build path, and the prompt's last-token logits match the oracle run on the same tensors."""
  import json
  from safetensors.torch import save_file
  from xotorch_support_jetson_amd.download.shard_download import NoopShardDownloader
  from xotorch_support_jetson_amd.inference.sharded_engine import ShardedInferenceEngine
  from xotorch_support_jetson_amd.models import registry
  cfg = SIZES[1]
  c = from_hf_config(cfg)
  tensors = random_mixed_tensors(c, 5)
  (tmp_path / "config.json").write_text(json.dumps(cfg))
  save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()}, str(tmp_path / "model.safetensors"))
  mid = registry.register_local_model(str(tmp_path))
  assert mid is not None and registry.model_cards[mid]["layers"] == len(cfg["layers"])
  shard = registry.build_full_shard(mid, "ShardedInferenceEngine")
  toks = [3, 99, 7, 7, 120, 64, 1, 0, 55]

  async def main():
    e = ShardedInferenceEngine(NoopShardDownloader(), device=torch.device("cpu"))
    out, _ = await e.infer_tensor("r", shard, np.array([toks]), {})
    return e, out
  e, out = asyncio.run(main())
  assert e.config.model_type == "tarepel" and e.config.layer_specs[1].rec.rank == 0 and e.runner.weights.layers[1].a2_w.shape[1] == 8
  want = Oracle(cfg, tensors).logits(toks, want=[len(toks) - 1])[0]
  got = out.double().reshape(-1)
  assert (got - want).abs().max() < 0.03 * want.abs().max()  # bf16 activations on the serving path


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_two_pipeline_shards_match_one(dev, dtype):
  """Layers 0-1 on one runner, 2-3 on another (the fp32 residual stream travels between them): the same logits as
  the unsplit model, in portions and token by token."""
  c = from_hf_config(SMALL)
  tensors = random_mixed_tensors(c, 11)
  n = c.num_layers
  runners = []
  for lo, hi in ((0, 1), (2, n - 1)):
    shard = Shard("t", lo, hi, n)
    w = mixed_weights(c, shard, tensors.__getitem__, torch.device(dev), dtype)
    runners.append(ShardRunner(c, shard, torch.device(dev), weights=w, num_pages=8, max_batch=2, max_ctx=512, dtype=dtype))
  assert runners[0].hidden_dtype == torch.float32
  toks = torch.randint(0, c.vocab_size, (90,), generator=torch.Generator().manual_seed(3)).tolist()
  outs, lo = [], 0
  for m in (40, 1, 1, 30, 2, 16):
    ids = torch.tensor(toks[lo:lo + m], dtype=torch.int32)
    hidden = runners[0].forward(["a"], [m], ids)
    assert hidden.dtype == torch.float32 and tuple(hidden.shape) == (m, c.hidden_size)
    outs.append(runners[1].forward(["a"], [m], hidden.clone(), logit_rows=list(range(m))).double().cpu())
    lo += m
  want = Oracle(SMALL, tensors).logits(toks)
  d = torch.cat(outs) - want
  d = d - d.mean(-1, keepdim=True)
  assert (d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()).max() < TOL[dtype]


def test_native_slot_manager_matches_python_twin():
  _runtime = pytest.importorskip("xotorch_support_jetson_amd._runtime")
  from xotorch_support_jetson_amd.runtime.runner import SlotManager
  a, b = _runtime.SlotManager(3), SlotManager(3)
  g = torch.Generator().manual_seed(0)
  live = []
  for step in range(200):
    if live and (len(live) == 3 or int(torch.randint(0, 2, (1,), generator=g))):
      rid = live.pop(int(torch.randint(0, len(live), (1,), generator=g)))
      a.release(rid)
      b.release(rid)
    else:
      rid = f"r{step}"
      assert a.acquire(rid) == b.acquire(rid)
      live.append(rid)
    assert a.num_free == b.num_free and all(a.slot(r) == b.slot(r) and a.has(r) for r in live)
  for m in (a, b):
    for r in list(live):
      m.release(r)
    for i in range(3):
      assert m.acquire(f"x{i}") == i
    with pytest.raises(RuntimeError, match="state slots"):
      m.acquire("y")
