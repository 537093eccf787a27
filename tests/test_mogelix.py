"""Mogelix in the framework against the plain implementation in tests/mogelix_oracle.py.

Every test makes its own small configuration and random checkpoint tensors, runs them through the serving runner
(paged KV pool with pooled-block entries, state slots, batched steps; HIP kernels and HIP-graph decode on a GPU, the
torch twins on the CPU) and compares logits at every position with the oracle's float64 run over the whole sequence.
Each body runs on the CPU and, marked gpu, on cuda:0 in float32 and bfloat16.
"""
import asyncio
import json

import numpy as np
import pytest
import torch

import mogelix_oracle as oracle
from xotorch_support_jetson_amd.inference.shard import Shard
from xotorch_support_jetson_amd.models.config import TINY_MOGELIX, from_hf_config
from xotorch_support_jetson_amd.models.weights import mixed_weights, random_mixed_tensors
from xotorch_support_jetson_amd.runtime.runner import ShardRunner

RUNS = [pytest.param("cpu", torch.float32, id="cpu-f32"),
        pytest.param("cuda:0", torch.float32, id="gpu-f32", marks=pytest.mark.gpu),
        pytest.param("cuda:0", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]
TOL = {torch.float32: 2e-4, torch.bfloat16: 6e-2}
ROT = {"base": 10000.0, "dims": 16, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 48}}


def attn(heads=4, kv=2, dim=32, vdim=32, window=24, pool=6, rot=ROT, scale=0.3, kv_from=None):
  m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
  if window:
    m["mask"] = {"size": window, **({"pool": pool} if pool else {})}
  if rot:
    m["rot"] = rot
  if kv_from is not None:
    m["kv_from"] = kv_from
  return m


def ssd(heads=4, vdim=16, state=16, groups=2, conv=4, norm_groups=2):
  return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def dense(ff=80):
  return {"kind": "dense", "ff": ff}


def moe(ff=32, experts=5, top=2, shared=48):
  m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
  if shared:
    m["shared"] = {"ff": shared}
  return m


def layer(kind, mixer, mlp):
  return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=64, vocab=96, alpha=1.5, eps=1e-5):
  return {"architecture": "Mogelix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
          "layers": layers}


SMALL = config([layer("attention", attn(), dense()), layer("mamba2", ssd(), moe()),
                layer("attention", attn(window=10, pool=3, scale=0.2, kv_from=0), moe(top=1, shared=0)),
                layer("mamba2", ssd(2, 32, 24, 1, 3, 1), None)])
_ORACLE = {}


class Rig:
  """A configuration + random tensors in the runner and in the oracle."""

  def __init__(self, cfg, dev, dtype, seed=1, pages=24, slots=4, tweak=None, graphs=None):
    self.cfg, self.dev, self.dtype = cfg, torch.device(dev), dtype
    self.c = from_hf_config(cfg)
    self.tensors = random_mixed_tensors(self.c, seed)
    if tweak:
      tweak(self.tensors)
    self.key = (json.dumps(cfg, sort_keys=True), seed, getattr(tweak, "__name__", None))
    shard = Shard("t", 0, self.c.num_layers - 1, self.c.num_layers)
    w = mixed_weights(self.c, shard, self.tensors.__getitem__, self.dev, dtype)
    self.runner = ShardRunner(self.c, shard, self.dev, weights=w, num_pages=pages, max_batch=slots, max_ctx=pages * 64,
                              dtype=dtype, use_graphs=graphs)
    self.V = self.c.vocab_size

  def tokens(self, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, self.V, (n,), generator=g).tolist()

  def want(self, toks):
    k = self.key + (tuple(toks),)
    if k[2] is None or k not in _ORACLE:  # (an anonymous tweak is not a cache key)
      _ORACLE[k] = oracle.forward(self.cfg, self.tensors, toks)
    return _ORACLE[k]

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
    want = self.want(toks)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
    worst = int(err.argmax())
    if self.dtype == torch.bfloat16 and any(L.get("mlp") and L["mlp"]["kind"] == "moe" for L in self.cfg["layers"]):
      # two router logits closer than bf16 rounding send a token to another expert: a rare position differs by a whole
      # expert's output, and a recurrent layer above carries a fading trace of it over the next few tokens; all others
      # stay inside the tolerance (the float32 runs are exact about every position, and the layouts without experts
      # are exact in bf16 too)
      over = int((err >= TOL[self.dtype]).sum())
      assert over <= max(2, len(toks) // 12) and err.median() < TOL[self.dtype] / 4, \
        f"{what}: {over} of {len(toks)} positions off, the worst ({worst}) by {float(err.max()):.3g}"
      return
    assert err.max() < TOL[self.dtype], f"{what}: position {worst} of {len(toks)} is off by {float(err.max()):.3g}"


def small_rig(dev, dtype, **kw):
  def small(t):
    pass
  return Rig(SMALL, dev, dtype, tweak=small, **kw)


# ------------------------------------------------------------------ whole prompts, portions, decoding
@pytest.mark.parametrize("dev,dtype", RUNS)
def test_whole_prompt(dev, dtype):
  rig = small_rig(dev, dtype)
  toks = rig.tokens(110, 3)
  rig.check(rig.run_alone("a", toks, [len(toks)]), toks, "whole prompt")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_first_tokens(dev, dtype):
  """Sequences of one, two and three tokens: empty history for the convolution, the state, the cache and the pools."""
  rig = small_rig(dev, dtype)
  for n in (1, 2, 3):
    toks = rig.tokens(n, 10 + n)
    rig.check(rig.run_alone("a", toks, [n]), toks, f"{n}-token prompt")
    rig.check(rig.run_alone("a", toks, [1]), toks, f"{n} tokens one by one")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_prefill_against_decoding(dev, dtype):
  rig = small_rig(dev, dtype)
  toks = rig.tokens(110, 3)
  whole = rig.run_alone("a", toks, [len(toks)])
  single = rig.run_alone("b", toks, [1])
  rig.check(single, toks, "token by token")
  diff = (whole - single).abs().max(-1).values / whole.abs().max()
  assert diff.median() < TOL[dtype] / 4 and (diff >= TOL[dtype]).sum() <= (0 if dtype == torch.float32 else 9)


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("cuts", [[2], [3, 2, 5, 1, 1, 7], [47, 1, 1, 17, 2], [64, 1], [63, 2, 1], [100, 1]])
def test_portions(dev, dtype, cuts):
  """A prompt cut anywhere (inside pages, windows, pooled blocks and convolution taps, down to two tokens)."""
  rig = small_rig(dev, dtype)
  toks = rig.tokens(110, 3)
  rig.check(rig.run_alone("a", toks, cuts), toks, f"portions {cuts}")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_long_decoding(dev, dtype):
  """A short prompt, then 150 single tokens: pages, windows and pooled blocks are crossed while decoding (HIP-graph
  steps on a GPU)."""
  rig = small_rig(dev, dtype)
  toks = rig.tokens(165, 6)
  rig.check(rig.run_alone("a", toks, [15, 1]), toks, "long decoding")


# ------------------------------------------------------------------ batches, pages and slots
@pytest.mark.parametrize("dev,dtype", RUNS)
def test_mixed_batches_match_alone(dev, dtype):
  """Unequal requests in one step (portions beside single tokens, a request that sits a step out) give each the
  logits it gets alone."""
  rig = small_rig(dev, dtype, pages=12)
  seqs = {"a": rig.tokens(110, 3), "b": rig.tokens(70, 22), "c": rig.tokens(9, 23), "d": rig.tokens(40, 24)}
  plan = [[("a", 50), ("b", 2)], [("a", 1), ("b", 30), ("c", 9)], [("a", 1), ("d", 17)], [("a", 40), ("b", 1), ("d", 1)],
          [("b", 37), ("d", 22)], [("a", 18)]]
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
  """A pool of four pages and two state slots serves six requests in turn, two at a time: every page (with its pooled
  entries) and slot is handed out again with another request's keys and state in it."""
  rig = small_rig(dev, dtype, pages=4, slots=2)
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


# ------------------------------------------------------------------ other sizes
SIZES = [
  # one head everywhere, kv_heads == heads, groups == heads, full rotation without scaling, a pool of one token (every
  # token before the window is its own block), one expert of one, two taps
  config([layer("attention", attn(1, 1, 32, 32, 7, 1, {"base": 100.0, "dims": 32}, 0.4), moe(16, 1, 1, 0)),
          layer("mamba2", ssd(1, 16, 16, 1, 2, 1), dense(48))], width=48, vocab=50, alpha=1.0),
  # key dim above value dim and no multiple of 8, rotation on a quarter of the head, window longer than a page, blocks that
  # straddle pages, every expert chosen, wide state, one tap (no convolution history)
  config([layer("mamba2", ssd(6, 8, 40, 3, 1, 3), moe(24, 3, 3, 16)),
          layer("attention", attn(6, 3, 36, 20, 70, 9, {"base": 1e6, "dims": 8}, 0.15), dense(40))], width=72, vocab=130,
         alpha=3.0),
  # no mask at all (every earlier token), no rotation, a window without pooled blocks, a window of one token with blocks
  # of two, layers without feed-forward
  config([layer("attention", attn(2, 1, 16, 48, 0, 0, None, 0.5), None),
          layer("attention", attn(2, 2, 16, 16, 5, 0, ROT, 0.5), dense(32)),
          layer("attention", attn(4, 2, 16, 16, 1, 2, ROT, 0.7, kv_from=1), None)], width=32, vocab=40),
  # three layers that read one layer's keys with three different masks, one of them the source's own
  config([layer("attention", attn(4, 2, 16, 8, 12, 4), dense(32)), layer("attention", attn(4, 2, 16, 8, 12, 4, kv_from=0), None),
          layer("mamba2", ssd(2, 8, 8, 2, 5, 1), None), layer("attention", attn(2, 2, 16, 8, 30, 8, kv_from=0), moe(8, 7, 3, 8)),
          layer("attention", attn(2, 2, 16, 8, 0, 0, kv_from=0), None)], width=40),
  # more experts and more chosen than the small routing kernel takes
  config([layer("mamba2", ssd(2, 8, 8, 1, 2, 1), moe(8, 70, 9, 0)), layer("attention", attn(2, 1, 16, 16, 6, 2), moe(8, 3, 2, 8))],
         width=32, vocab=40),
]


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("n", range(len(SIZES)))
def test_other_sizes(dev, dtype, n):
  rig = Rig(SIZES[n], dev, dtype, seed=50 + n)
  toks = rig.tokens(150 if n == 1 else 90, 60 + n)
  rig.check(rig.run_alone("a", toks, [33, 2, 1, 1, 29, 1]), toks, f"sizes {n}")


# ------------------------------------------------------------------ faults that random weights would hide
def _marked(window, pool):
  """One attention layer without rotation whose key projection is minus its query projection, and a token C whose
  embedding is minus token B's: C's query scores scale * dim with a B's key, minus that with its own key and about zero
  with the A tokens around, so whether an earlier B is inside C's window, inside a pooled block (at 1 / pool of its
  weight) or nowhere moves C's logits."""
  cfg = config([layer("attention", attn(2, 2, 16, 16, window, pool, None, 1.0), None)], width=32, vocab=24)

  def marked(t):
    t["l0.mix.k"] = -t["l0.mix.q"]
    t["l0.mix.q.b"], t["l0.mix.k.b"] = torch.zeros(32), torch.zeros(32)
    t["l0.mix.sink"] = torch.full((2,), 4.0)
    t["embed"][1] = t["embed"][1] * 3.0
    t["embed"][2] = -t["embed"][1]
    t["l0.mix.o"] = t["l0.mix.o"] * 4.0
  return cfg, marked


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("window,pool", [(16, 4), (64, 10), (20, 64), (9, 1)])
def test_window_and_block_edges(dev, dtype, window, pool):
  """A token B, then a token C at distance window - 1, window, window + 1, window + pool - 1, window + pool, ...: for C
  the B is the last token inside the window, the first outside, in a block that is just complete or not yet.  In a
  prompt, in portions that end on and straddle the edges, and decoded one by one."""
  cfg, tweak = _marked(window, pool)
  rig = Rig(cfg, dev, dtype, tweak=tweak, pages=16)
  gaps = [window - 1, window, window + 1, window + pool - 1, window + pool, window + 2 * pool - 1, window + pool + 1]
  toks, marks = [0, 0, 0], []
  for g in gaps:
    marks.append(len(toks))
    toks += [1] + [0] * (g - 1) + [2, 0, 0]
  rig.check(rig.run_alone("a", toks, [len(toks)]), toks, "prompt")
  rig.check(rig.run_alone("a", toks, [marks[1] + 1, 2, 1, window, pool, 1]), toks, "portions over the edges")
  rig.check(rig.run_alone("a", toks, [marks[0] + 2, 1]), toks, "decoding over the edges")
  # the test bites: widening the window by one or dropping the pooled blocks changes some C's logits
  for w2, p2, least in ((window + 1, pool, 0.1), (window, 0, 0.02)):
    if pool == 1 and p2:  # (blocks of one token: what leaves the window is still seen, as its own block)
      continue
    c2 = config([layer("attention", attn(2, 2, 16, 16, w2, p2, None, 1.0), None)], width=32, vocab=24)
    a, b = oracle.forward(c2, rig.tensors, toks), rig.want(toks)
    assert (a - b).abs().max() > least * b.abs().max()


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_far_token_lives_in_the_state(dev, dtype):
  """Decays pushed to almost one and a first token unlike all later ones: 300 tokens on, beyond every window, the
  read-out still holds the first token's write; a state that was dropped, cleared or attached to the wrong slot changes
  the last logits."""
  cfg = config([layer("mamba2", ssd(2, 16, 16, 1, 3, 1), None), layer("attention", attn(2, 1, 16, 16, 8, 4), None)], width=32)

  def far(t):
    t["l0.mix.A_log"] = torch.full_like(t["l0.mix.A_log"], -9.0)
    t["l0.mix.dt_bias"] = torch.full_like(t["l0.mix.dt_bias"], -2.0)
    t["embed"][0] = t["embed"][0] * 6.0
  rig = Rig(cfg, dev, dtype, tweak=far, pages=8)
  toks = [0] + [1 + (i * 7) % 90 for i in range(300)]
  got = rig.run_alone("a", toks, [150, 1, 1, 100, 2, 1])
  rig.check(got, toks, "far token")
  other = oracle.forward(cfg, rig.tensors, [3] + toks[1:])[-1]  # the same run without that first token
  gap = (other - rig.want(toks)[-1]).abs().max()
  if dtype == torch.float32:
    assert gap > 30 * TOL[dtype] * got[-1].abs().max(), "the first token must matter at the end for this test to bite"


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_convolution_history_across_portions(dev, dtype):
  """Five taps and portions shorter than the taps: the convolution reads inputs of two and three steps back."""
  cfg = config([layer("mamba2", ssd(2, 16, 8, 2, 5, 1), dense(32))], width=32)
  rig = Rig(cfg, dev, dtype)
  toks = rig.tokens(40, 70)
  rig.check(rig.run_alone("a", toks, [1, 2, 1, 1, 3, 2, 4, 1]), toks, "short portions")


def test_borrowed_keys_must_stay_on_one_shard():
  c = from_hf_config(SMALL)
  with pytest.raises(ValueError, match="not on this shard"):
    ShardRunner(c, Shard("t", 1, 3, 4), "cpu", num_pages=4, max_batch=2, max_ctx=256, dtype=torch.float32)


# ------------------------------------------------------------------ the engine's own entry point
@pytest.mark.parametrize("dev", ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_engine(dev):
  """Three prompts of unequal length at once through ShardedInferenceEngine (queue, batched steps, sampler at
  temperature 0): every token drawn is the oracle's greedy token for the text so far (ties within rounding
  aside), and slots and pages are all free at the end."""
  from xotorch_support_jetson_amd.download.shard_download import NoopShardDownloader
  from xotorch_support_jetson_amd.inference.sharded_engine import ShardedInferenceEngine
  from xotorch_support_jetson_amd.models.config import preset
  c = preset("tiny-mogelix")
  tensors = random_mixed_tensors(c, 0)
  shard = Shard("tiny-mogelix", 0, c.num_layers - 1, c.num_layers)
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
  for (rid, p), seq in zip(prompts.items(), seqs):
    lg = oracle.forward(TINY_MOGELIX, tensors, seq[:-1])
    for t in range(len(p) - 1, len(seq) - 1):
      best = float(lg[t].max())
      assert float(lg[t][seq[t + 1]]) >= best - 0.05 * float(lg[t].std()), f"{rid}: token {t + 1} is not the greedy one"


def test_checkpoint_directory_through_registry_and_engine(tmp_path):
  """config.json + model.safetensors (bf16) in a folder: registered as a local model, loaded by the engine's own
  build path, and the prompt's last-token logits match the oracle run on the same tensors."""
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
  assert e.config.model_type == "mogelix" and e.config.layer_specs[1].wattn.pool == 9
  want = oracle.forward(cfg, tensors, toks)[-1]
  got = out.double().reshape(-1)
  assert (got - want).abs().max() < 0.03 * want.abs().max()  # bf16 activations on the serving path
