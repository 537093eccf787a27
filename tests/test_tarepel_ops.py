"""Each Tarepel mechanism alone: the kernel library's op (HIP on a GPU, its torch twin on the CPU) against the
matching function of tests/tarepel_oracle.py, fed the same projections.  Pages are handed out in scrambled order,
sequences are cut into two steps, and a second sequence shares the batch."""
import math

import pytest
import torch

import tarepel_oracle as O
from xotorch_support_jetson_amd.ops import kernels as K

DEVS = [pytest.param("cpu", torch.float32, id="cpu"),
        pytest.param("cuda:0", torch.float32, id="gpu-f32", marks=pytest.mark.gpu),
        pytest.param("cuda:0", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]


def rnd(*shape, seed=0, scale=1.0):
  return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


def close(got, want, dtype, what):
  tol = 3e-5 if dtype == torch.float32 else 2e-2
  err = (got.double().cpu() - want).abs().max() / want.abs().max()
  assert err < tol, f"{what}: off by {float(err):.3g}"


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("D", [40, 256, 1000])
def test_residual_and_scalar_norm(dev, dtype, D):
  x, y1, y2, s1, s2 = rnd(5, D, seed=1), rnd(5, D + 24, seed=2), rnd(5, D, seed=3), rnd(D, seed=4), rnd(D, seed=5)
  g, eps = 1.7, 1e-3
  xs = x + s1 * y1[:, :D] + s2 * y2
  want = O.unit_rms(xs, eps) * g
  xd = x.float().to(dev)
  out = torch.zeros(5, D + 8, dtype=dtype, device=dev)
  K.resid_scale_norm(xd, y1.float().to(dev), s1.float().to(dev), y2.float().to(dev), s2.float().to(dev),
                     torch.tensor([g], device=dev), eps, out)
  close(xd, xs, torch.float32, "residual sum")
  close(out[:, :D], want, dtype, "norm")
  assert float(out[:, D:].abs().max()) == 0.0


@pytest.mark.parametrize("dev,dtype", DEVS)
def test_gelu_gate(dev, dtype):
  P = rnd(7, 100, seed=6, scale=2.0)
  out = torch.zeros(7, 48, dtype=dtype, device=dev)
  K.gelu_mul(P.float().to(dev), 10, 60, 40, out)
  close(out[:, :40], O.gelu_tanh(P[:, 10:50]) * P[:, 60:100], dtype, "gelu gate")


def _batch(lens_done, lens_new, pages, dev, scramble):
  """Step inputs for sequences holding lens_done tokens that get lens_new more; tables over scrambled pages."""
  order = torch.randperm(pages, generator=torch.Generator().manual_seed(scramble)).tolist()
  tables, slots, pos, cu = [], [], [], [0]
  width = max(-(-(a + b) // 64) for a, b in zip(lens_done, lens_new))
  per = pages // len(lens_done)  # each sequence keeps its own pages from step to step
  for i, (a, b) in enumerate(zip(lens_done, lens_new)):
    n = -(-(a + b) // 64)
    tb = order[i * per:i * per + n]
    tables.append(tb + [0] * (width - n))
    slots += [tb[p // 64] * 64 + p % 64 for p in range(a, a + b)]
    pos += list(range(a, a + b))
    cu.append(cu[-1] + b)
  i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
  return (i32(tables), torch.tensor(slots, dtype=torch.int64, device=dev), i32(pos), i32(cu),
          i32([a + b for a, b in zip(lens_done, lens_new)]))


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("H,G,d,R,chunk", [(4, 2, 32, 16, 48), (2, 2, 64, 64, 64), (3, 1, 16, 0, 100), (2, 1, 128, 32, 7),
                                           (16, 1, 16, 8, 20), (6, 2, 20, 4, 33), (2, 1, 96, 32, 50), (4, 2, 160, 160, 64),
                                           (2, 2, 256, 64, 70), (2, 1, 224, 2, 130)])
def test_chunked_sigmoid_attention(dev, dtype, H, G, d, R, chunk):
  D, scale, base = 24, 0.3, 1000.0
  lens = [150, 70]
  W = {"q": rnd(H * d, D, seed=1, scale=0.4), "k": rnd(G * d, D, seed=2, scale=0.4), "pb": rnd(H, seed=3) - 1.0,
       "o": torch.eye(H * d, dtype=torch.float64)}
  m = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "mask": {"size": chunk}, "rot": {"dims": R or 2, "base": base},
       "scale": scale}
  if R == 0:  # no rotation: the oracle rotates nothing when the angle table is all zeros
    m["rot"] = {"dims": 2, "base": 1.0}
  hs = [rnd(n, D, seed=10 + i) for i, n in enumerate(lens)]
  want = []
  for h in hs:
    mem = {}
    if R == 0:
      rot = O.rotate
      O.rotate = lambda x, p, dims, b: x
    try:
      want.append(torch.stack([O.chunk_gated_attention(W, "", m, h[p], p, mem) for p in range(h.shape[0])]))
    finally:
      if R == 0:
        O.rotate = rot
  from xotorch_support_jetson_amd.ops.rope import build_cos_sin
  tab = build_cos_sin(R, 256, base, None, dev) if R else torch.zeros(1, 0, device=dev)
  pages = 8
  kc = torch.zeros(pages, G, 64, d, dtype=dtype, device=dev)
  vc = torch.zeros(pages, G, d, 64, dtype=dtype, device=dev)
  got = [[], []]
  done = [0, 0]
  for new in ([97, 3], [53, 67]):  # two steps; the first request's cut falls inside a page and a chunk
    tables, slots, pos, cu, ctx = _batch(done, new, pages, dev, scramble=5)
    rows = torch.cat([hs[i][done[i]:done[i] + new[i]] for i in range(2)])
    P = torch.cat([rows @ W["q"].t(), rows @ W["k"].t()], 1).float().to(dev)
    q = torch.empty(P.shape[0], H, d, dtype=dtype, device=dev)
    K.rope_kv_store(P, 0, H * d, -1, H, G, d, R, pos, tab, slots, q, kc, vc)
    out = torch.zeros(P.shape[0], H * d + 8, dtype=dtype, device=dev)
    K.attn_gated_chunk(q, kc, vc, tables, cu, ctx, W["pb"].float().to(dev), scale, chunk, 1.5, out[:, 4:4 + H * d],
                       max_qlen=max(new))
    for i in range(2):
      got[i].append(out[int(cu[i]):int(cu[i + 1]), 4:4 + H * d])
      done[i] += new[i]
  for i in range(2):
    close(torch.cat(got[i]), 1.5 * want[i], dtype, f"attention, sequence {i}")


def _slots_batch(lens_new, slots, dev):
  cu = [0]
  for n in lens_new:
    cu.append(cu[-1] + n)
  return torch.tensor(cu, dtype=torch.int32, device=dev), torch.tensor(slots, dtype=torch.int32, device=dev)


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("H,G,d,dv,taps", [(4, 2, 16, 32, 3), (2, 2, 64, 64, 4), (3, 1, 24, 80, 2), (1, 1, 128, 16, 5),
                                           (2, 1, 256, 40, 1), (2, 2, 200, 256, 3)])
def test_gated_delta_rule(dev, dtype, H, G, d, dv, taps):
  D, eps = 20, 1e-5
  lens = [45, 9]
  C = 2 * G * d + H * dv
  W = {"q": rnd(G * d, D, seed=1), "k": rnd(G * d, D, seed=2), "v": rnd(H * dv, D, seed=3), "b": rnd(H, D, seed=4),
       "a": rnd(H, D, seed=5), "g": rnd(H * dv, D, seed=6), "A_log": rnd(H, seed=7) - 1.0, "dt_bias": rnd(H, seed=8),
       "norm": 1 + 0.1 * rnd(dv, seed=9), "o": torch.eye(H * dv, dtype=torch.float64), "q.conv": rnd(G * d, taps, seed=11),
       "k.conv": rnd(G * d, taps, seed=12), "v.conv": rnd(H * dv, taps, seed=13)}
  m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": taps}
  hs = [rnd(n, D, seed=20 + i, scale=0.5) for i, n in enumerate(lens)]
  want = []
  for h in hs:
    mem = {}
    want.append(torch.stack([O.gated_delta_rule(W, "", m, h[p], mem, eps) for p in range(h.shape[0])]))
  f = lambda t: t.float().to(dev)
  conv_w = f(torch.cat([W["q.conv"], W["k.conv"], W["v.conv"]]))
  state = torch.full((3, H, dv, d), 7.0, device=dev)
  conv_state = torch.full((3, taps - 1, C), 7.0, device=dev)
  for s in (2, 0):  # the slots these sequences get, cleared as on admission
    state[s].zero_()
    conv_state[s].zero_()
  got, done = [[], []], [0, 0]
  for new in ([1, 4], [2, 1], [42, 4]):  # steps shorter than the taps, then the rest
    cu, slots = _slots_batch(new, [2, 0], dev)
    rows = torch.cat([hs[i][done[i]:done[i] + new[i]] for i in range(2)])
    P = f(torch.cat([rows @ W[k].t() for k in ("q", "k", "v", "b", "a", "g")], 1))
    T = P.shape[0]
    qkv = torch.empty(T, C, device=dev)
    beta, decay = torch.empty(T, H, device=dev), torch.empty(T, H, device=dev)
    K.delta_prep(P, 0, C, C + H, conv_w, conv_state, slots, cu, f(W["A_log"]), f(W["dt_bias"]), H, G, d, dv, qkv, beta, decay)
    o = torch.empty(T, H * dv, device=dev)
    K.linear_recurrence(qkv[:, :G * d], qkv[:, G * d:2 * G * d], qkv[:, 2 * G * d:], decay, beta, 1.0, state, slots, cu, o)
    out = torch.zeros(T, H * dv, dtype=dtype, device=dev)
    K.gated_rmsnorm(o, f(W["norm"]), P, C + 2 * H, eps, 1.0, out)
    for i in range(2):
      got[i].append(out[int(cu[i]):int(cu[i + 1])])
      done[i] += new[i]
  for i in range(2):
    close(torch.cat(got[i]), want[i], dtype, f"delta rule, sequence {i}")
  assert float((state[1] - 7.0).abs().max()) == 0.0, "a slot no sequence holds was written"


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("H,d,dv,rank,tau", [(2, 32, 64, 8, 8.0), (4, 16, 16, 4, 1.0), (1, 100, 72, 16, 16.0), (3, 64, 130, 5, 3.0),
                                             (2, 256, 48, 3, 2.0), (1, 8, 8, 1, 4.0)])
def test_gated_linear_attention(dev, dtype, H, d, dv, rank, tau):
  D, eps = 20, 1e-5
  lens = [60, 33]
  W = {"q": rnd(H * d, D, seed=1), "k": rnd(H * d, D, seed=2, scale=0.3), "v": rnd(H * dv, D, seed=3), "g": rnd(H * dv, D, seed=4),
       "a1": rnd(rank, D, seed=5), "a2": rnd(H * d, rank, seed=6, scale=0.5), "a2.b": rnd(H * d, seed=7) + 2.0,
       "norm": 1 + 0.1 * rnd(dv, seed=8), "o": torch.eye(H * dv, dtype=torch.float64)}
  m = {"heads": H, "dim": d, "vdim": dv, "tau": tau}
  hs = [rnd(n, D, seed=30 + i, scale=0.5) for i, n in enumerate(lens)]
  want = []
  for h in hs:
    mem = {}
    want.append(torch.stack([O.gated_linear_attention(W, "", m, h[p], mem, eps) for p in range(h.shape[0])]))
  f = lambda t: t.float().to(dev)
  state = torch.zeros(2, H, dv, d, device=dev)
  got, done = [[], []], [0, 0]
  for new in ([17, 1], [1, 30], [42, 2]):
    cu, slots = _slots_batch(new, [1, 0], dev)
    rows = torch.cat([hs[i][done[i]:done[i] + new[i]] for i in range(2)])
    P = f(torch.cat([rows @ W[k].t() for k in ("q", "k", "v", "g", "a1")], 1))
    T = P.shape[0]
    decay = torch.empty(T, H * d, device=dev)
    K.gla_prep(P, 2 * H * d + 2 * H * dv, f(W["a2"]), f(W["a2.b"]), tau, decay)
    o = torch.empty(T, H * dv, device=dev)
    K.linear_recurrence(P[:, :H * d], P[:, H * d:2 * H * d], P[:, 2 * H * d:2 * H * d + H * dv], decay, None, d ** -0.5, state,
                        slots, cu, o)
    out = torch.zeros(T, H * dv, dtype=dtype, device=dev)
    K.gated_rmsnorm(o, f(W["norm"]), P, 2 * H * d + H * dv, eps, 1.0, out)
    for i in range(2):
      got[i].append(out[int(cu[i]):int(cu[i + 1])])
      done[i] += new[i]
  for i in range(2):
    close(torch.cat(got[i]), want[i], dtype, f"gated linear attention, sequence {i}")


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("chunk,d", [(48, 32), (64, 64), (100, 32), (32, 128), (7, 32)])
def test_chunk_mask_is_exact(dev, dtype, chunk, d):
  """Queries and a few marked keys point along one unrotated dim, with a bias of -12: a marked key weighs 0.98, every
  other key 6e-6.  The marked keys sit on both sides of every chunk edge (and at position 0), so a key let in from
  the previous chunk, a key of the own chunk left out, or a future key changes the output by its whole value.
  Prompt portions (the MFMA kernel in bf16) and single decoded tokens."""
  H, G, R, n = 2, 1, 16, 230
  hq, hk = H * d, G * d
  W = {"q": torch.cat([torch.eye(hq, dtype=torch.float64), torch.zeros(hq, hk, dtype=torch.float64)], 1),
       "k": torch.cat([torch.zeros(hk, hq, dtype=torch.float64), torch.eye(hk, dtype=torch.float64)], 1),
       "pb": torch.full((H,), -12.0, dtype=torch.float64), "o": torch.eye(hq, dtype=torch.float64)}
  m = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "mask": {"size": chunk}, "rot": {"dims": R, "base": 100.0}, "scale": 1.0}
  marked = {0} | {c + o for c in range(chunk, n, chunk) for o in (-1, 0)} | {n - 1}
  q = torch.zeros(n, H, d, dtype=torch.float64)
  q[:, :, d - 1] = 4.0
  k = 0.01 * rnd(n, G, d, seed=3)
  for p in marked:
    k[p, :, d - 1] = 4.0
    k[p, :, 0] = 1.0 + p  # tells the marked keys apart in the output (rotated dim: only the value keeps it as is)
  hs = torch.cat([q.reshape(n, -1), k.reshape(n, -1)], 1)
  mem = {}
  want = torch.stack([O.chunk_gated_attention(W, "", m, hs[p], p, mem) for p in range(n)])
  from xotorch_support_jetson_amd.ops.rope import build_cos_sin
  tab = build_cos_sin(R, 256, 100.0, None, dev)
  kc = torch.zeros(4, G, 64, d, dtype=dtype, device=dev)
  vc = torch.zeros(4, G, d, 64, dtype=dtype, device=dev)
  got, done = [], 0
  for new in [101, 2, 60] + [1] * (n - 163):
    tables, slots, pos, cu, ctx = _batch([done], [new], 4, dev, scramble=9)
    P = hs[done:done + new].float().to(dev)
    qo = torch.empty(new, H, d, dtype=dtype, device=dev)
    K.rope_kv_store(P, 0, hq, -1, H, G, d, R, pos, tab, slots, qo, kc, vc)
    out = torch.zeros(new, hq, dtype=dtype, device=dev)
    K.attn_gated_chunk(qo, kc, vc, tables, cu, ctx, W["pb"].float().to(dev), 1.0, chunk, 1.0, out, max_qlen=new)
    got.append(out)
    done += new
  got = torch.cat(got).double().cpu()
  err = (got - want).abs().max(-1).values / want.abs().max()
  tol = 1e-4 if dtype == torch.float32 else 2e-2
  assert err.max() < tol, f"position {int(err.argmax())} (chunk {chunk}) is off by {float(err.max()):.3g}"
