"""Each Mogelix mechanism alone: the kernel library's op (HIP on a GPU, its torch twin on the CPU) against the matching
function of tests/mogelix_oracle.py, fed the same projections.  Pages are handed out in scrambled order, sequences are
cut into two steps, and a second sequence shares the batch."""
import pytest
import torch

import mogelix_oracle as O
from xotorch_support_jetson_amd.ops import kernels as K
from xotorch_support_jetson_amd.ops.rope import build_cos_sin

DEVS = [pytest.param("cpu", torch.float32, id="cpu"),
        pytest.param("cuda:0", torch.float32, id="gpu-f32", marks=pytest.mark.gpu),
        pytest.param("cuda:0", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
  return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64) * scale


def close(got, want, dtype, what, tol32=3e-5, tol16=2e-2):
  tol = tol32 if dtype == torch.float32 else tol16
  err = (got.double().cpu() - want).abs().max() / want.abs().max()
  assert err < tol, f"{what}: off by {float(err):.3g}"


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("D,gate", [(40, True), (256, True), (1000, False)])
def test_gated_post_norm(dev, dtype, D, gate):
  x, y, P, gb, w = rnd(5, D, seed=1), rnd(5, D + 24, seed=2), rnd(5, D + 10, seed=3), rnd(D, seed=4), rnd(D, seed=5)
  alpha, eps = 1.7, 1e-3
  yy = y[:, :D] * torch.sigmoid(P[:, 10:] + gb) if gate else y[:, :D]
  want = O.rms_div(alpha * x + yy, eps) * w
  xd = x.float().to(dev)
  out = torch.zeros(5, D + 8, dtype=dtype, device=dev)
  K.gated_postnorm(xd, y.float().to(dev), P.float().to(dev) if gate else None, 10, gb.float().to(dev) if gate else None,
                   alpha, w.float().to(dev), eps, out)
  close(xd, want, torch.float32, "stream")
  close(out[:, :D], want, dtype, "operand copy")
  assert float(out[:, D:].abs().max()) == 0.0
  x2 = x.float().to(dev)
  K.gated_postnorm(x2, None, None, 0, None, 1.0, w.float().to(dev), eps, None)  # a plain weighted norm
  close(x2, O.rms_div(x, eps) * w, torch.float32, "norm alone")


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("F", [24, 256, 1500])
def test_polynorm_and_squared_relu(dev, dtype, F):
  P = rnd(6, F + 12, seed=6, scale=1.5)
  coef = torch.tensor([0.7, -0.4, 0.25, 0.1], dtype=F64)
  out = torch.zeros(6, F + 4, dtype=dtype, device=dev)
  K.polynorm_act(P.float().to(dev), 12, F, coef.float().to(dev), 1e-4, out)
  close(out[:, :F], O.polynorm(P[:, 12:], coef, 1e-4), dtype, "polynorm")
  assert float(out[:, F:].abs().max()) == 0.0
  K.relu2(P.float().to(dev), 5, F, out)
  close(out[:, :F], torch.relu(P[:, 5:5 + F]) ** 2, dtype, "relu squared")


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


ATTN = [  # H, G, d, dv, R, window, pool, sink
  (4, 2, 32, 32, 16, 24, 6, True), (2, 2, 64, 64, 64, 70, 11, True), (3, 1, 16, 48, 0, 0, 0, True),
  (2, 1, 128, 32, 32, 7, 1, False), (16, 1, 16, 16, 8, 20, 64, True), (6, 2, 20, 12, 4, 33, 5, True),
  (2, 1, 96, 160, 32, 50, 0, False), (2, 2, 256, 256, 64, 70, 7, True), (4, 4, 64, 64, 64, 1, 2, True),
  (2, 1, 128, 128, 64, 40, 9, True), (4, 2, 64, 64, 32, 0, 0, False), (2, 2, 32, 32, 0, 100, 3, False)]


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("H,G,d,dv,R,window,pool,sink", ATTN)
def test_window_attention_with_pooled_blocks(dev, dtype, H, G, d, dv, R, window, pool, sink):
  """Biases, rotation with banded frequency scaling, per-head RMS division, paged write, the pooled caches' update and
  the attention itself: two sequences, each in two steps (the second straddles windows, blocks and pages)."""
  D, scale, eps = 24, 0.3, 1e-5
  lens = [150, 70]
  rot = {"dims": R, "base": 1000.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40}} if R else None
  t = {"q": rnd(H * d, D, seed=1, scale=0.4), "k": rnd(G * d, D, seed=2, scale=0.4), "v": rnd(G * dv, D, seed=3, scale=0.4),
       "q.b": rnd(H * d, seed=4, scale=0.3), "k.b": rnd(G * d, seed=5, scale=0.3), "v.b": rnd(G * dv, seed=6, scale=0.3),
       "o": torch.eye(H * dv, dtype=F64)}
  if sink:
    t["sink"] = rnd(H, seed=7) + 1.0
  m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": scale}
  if window:
    m["mask"] = {"size": window, "pool": pool}
  if rot:
    m["rot"] = rot
  xs = [rnd(n, D, seed=10 + i) for i, n in enumerate(lens)]
  want = [O.attention_mixer(x, m, t, "", eps, O.attention_keys(x, m, t, "", eps, torch.arange(x.shape[0]))) for x in xs]

  pages = 8
  adt = dtype
  kc = torch.zeros(pages, G, 64, d, dtype=adt, device=dev)
  vc = torch.zeros(pages, G, dv, 64, dtype=adt, device=dev)
  kp = vp = None
  if window and pool:
    per = K.pool_dims(pool)
    kp = torch.full((pages, G, per, d), 1e4, dtype=adt, device=dev)  # an entry read before it is written shows
    vp = torch.full((pages, G, per, dv), 1e4, dtype=adt, device=dev)
  W = torch.cat([t["q"], t["k"], t["v"]], 0)
  bias = torch.cat([t["q.b"], t["k.b"], t["v.b"]]).float().to(dev)
  sc = rot and dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=4.0,
                    original_max_position_embeddings=40)
  tab = build_cos_sin(R, 256, 1000.0, sc, dev) if R else torch.zeros(1, 0, device=dev)
  done = [0, 0]
  got = [[], []]
  for new in ([97, 31], [53, 39]):
    tables, slots, pos, cu, ctx = _batch(done, new, pages, dev, scramble=3)
    x = torch.cat([xs[i][done[i]:done[i] + new[i]] for i in range(2)])
    P = (x @ W.T).float().to(dev)
    T = P.shape[0]
    q = torch.empty(T, H, d, dtype=adt, device=dev)
    K.qk_norm_rope_store(P, bias, 0, H * d, (H + G) * d, H, G, d, dv, R, pos, tab, slots, eps, True, q, kc, vc)
    if kp is not None:
      K.kv_pool_update(kc, vc, kp, vp, tables, cu, ctx, pool, max(new))
    out = torch.zeros(T, H * dv + 8, dtype=adt, device=dev)
    K.attn_window_pool(q, kc, vc, kp, vp, tables, cu, ctx, t["sink"].float().to(dev) if sink else None, scale, window,
                       pool if kp is not None else 0, out[:, :H * dv], max_qlen=max(new))
    assert float(out[:, H * dv:].abs().max()) == 0.0
    for i, part in enumerate(out[:, :H * dv].split(new)):
      got[i].append(part)
    done = [a + b for a, b in zip(done, new)]
  for i in range(2):
    close(torch.cat(got[i]), want[i], dtype, f"sequence {i}", tol32=5e-5, tol16=3e-2)


@pytest.mark.parametrize("dev,dtype", DEVS)
def test_single_tokens_read_the_same_caches(dev, dtype):
  """A prompt portion, then the rest one token a step, two sequences a step: the single-token path."""
  H, G, d, dv, window, pool, D, scale, eps = 4, 2, 32, 16, 10, 3, 16, 0.4, 1e-5
  t = {"q": rnd(H * d, D, seed=1, scale=0.4), "k": rnd(G * d, D, seed=2, scale=0.4), "v": rnd(G * dv, D, seed=3, scale=0.4),
       "q.b": rnd(H * d, seed=4, scale=0.3), "k.b": rnd(G * d, seed=5, scale=0.3), "v.b": rnd(G * dv, seed=6, scale=0.3),
       "o": torch.eye(H * dv, dtype=F64), "sink": rnd(H, seed=7)}
  m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": scale, "mask": {"size": window, "pool": pool}}
  lens = [75, 69]
  xs = [rnd(n, D, seed=20 + i) for i, n in enumerate(lens)]
  want = [O.attention_mixer(x, m, t, "", eps, O.attention_keys(x, m, t, "", eps, torch.arange(x.shape[0]))) for x in xs]
  pages = 4
  kc = torch.zeros(pages, G, 64, d, dtype=dtype, device=dev)
  vc = torch.zeros(pages, G, dv, 64, dtype=dtype, device=dev)
  per = K.pool_dims(pool)
  kp = torch.zeros(pages, G, per, d, dtype=dtype, device=dev)
  vp = torch.zeros(pages, G, per, dv, dtype=dtype, device=dev)
  W = torch.cat([t["q"], t["k"], t["v"]], 0)
  bias = torch.cat([t["q.b"], t["k.b"], t["v.b"]]).float().to(dev)
  tab = torch.zeros(1, 0, device=dev)
  done, got = [0, 0], [[], []]
  steps = [[60, 61]] + [[1, 1]] * 8 + [[7, 0]]
  for new in steps:
    live = [i for i in range(2) if new[i]]
    tables, slots, pos, cu, ctx = _batch([done[i] for i in live], [new[i] for i in live], pages, dev, scramble=5)
    if len(live) == 1:  # the second sequence keeps the pages it had: rebuild its view of the scrambled order
      tables, slots, pos, cu, ctx = _batch(done, [new[0], 1], pages, dev, scramble=5)
      tables, cu, ctx = tables[:1], cu[:2], ctx[:1]
      slots, pos = slots[:new[0]], pos[:new[0]]
    x = torch.cat([xs[i][done[i]:done[i] + new[i]] for i in live])
    P = (x @ W.T).float().to(dev)
    q = torch.empty(P.shape[0], H, d, dtype=dtype, device=dev)
    K.qk_norm_rope_store(P, bias, 0, H * d, (H + G) * d, H, G, d, dv, 0, pos, tab, slots, eps, True, q, kc, vc)
    K.kv_pool_update(kc, vc, kp, vp, tables, cu, ctx, pool, max(new))
    out = torch.zeros(P.shape[0], H * dv, dtype=dtype, device=dev)
    K.attn_window_pool(q, kc, vc, kp, vp, tables, cu, ctx, t["sink"].float().to(dev), scale, window, pool, out, max_qlen=max(new))
    for i, part in zip(live, out.split([new[i] for i in live])):
      got[i].append(part)
    done = [a + b for a, b in zip(done, new)]
  for i in range(2):
    close(torch.cat(got[i]), want[i][:done[i]], dtype, f"sequence {i}", tol32=5e-5, tol16=3e-2)


SSD = [(4, 16, 16, 2, 4, 2), (6, 40, 56, 1, 4, 1), (1, 8, 24, 1, 2, 1), (3, 40, 100, 3, 1, 3), (2, 64, 128, 1, 5, 4)]


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("H,dv,N,G,taps,ng", SSD)
def test_state_space_mixer(dev, dtype, H, dv, N, G, taps, ng):
  """Convolution with its carried inputs, step sizes and decays, the recurrence on two state slots of a larger pool,
  skip, gate and grouped norm: two sequences, three steps each (one of a single token)."""
  D, eps = 20, 1e-5
  inner, C = H * dv, H * dv + 2 * G * N
  m = {"heads": H, "vdim": dv, "state": N, "groups": G, "conv": taps, "norm_groups": ng}
  t = {"in": rnd(2 * inner + 2 * G * N + H, D, seed=1, scale=0.3), "conv": rnd(C, taps, seed=2, scale=0.5),
       "conv.b": rnd(C, seed=3, scale=0.3), "dt_bias": rnd(H, seed=4), "A_log": rnd(H, seed=5) - 1.0, "D": rnd(H, seed=6),
       "norm": 1 + 0.1 * rnd(inner, seed=7), "o": torch.eye(inner, dtype=F64)}
  lens = [61, 40]
  xs = [rnd(n, D, seed=30 + i) for i, n in enumerate(lens)]
  want = [O.mamba2_mixer(x, m, t, "", eps) for x in xs]
  slots_n = 5
  S = torch.full((slots_n, H, dv, N), 7.0, device=dev)  # other requests' leftovers
  conv = torch.full((slots_n, taps - 1, C), -3.0, device=dev)
  sl = torch.tensor([3, 1], dtype=torch.int32, device=dev)
  S[sl.long()] = 0
  conv[sl.long()] = 0
  f = lambda a: a.float().to(dev)
  done, got = [0, 0], [[], []]
  for new in ([30, 2], [1, 1], [30, 37]):
    cu = torch.tensor([0, new[0], new[0] + new[1]], dtype=torch.int32, device=dev)
    x = torch.cat([xs[i][done[i]:done[i] + new[i]] for i in range(2)])
    P = f(x @ t["in"].T)
    T = P.shape[0]
    xbc = torch.empty(T, C, device=dev)
    v = torch.empty(T, inner, device=dev)
    decay = torch.empty(T, H, device=dev)
    o = torch.empty(T, inner, device=dev)
    K.ssd_prep(P, inner, 2 * inner + 2 * G * N, f(t["conv"]), f(t["conv.b"]), conv, sl, cu, f(t["A_log"]), f(t["dt_bias"]),
               H, dv, xbc, v, decay)
    K.linear_recurrence(xbc[:, inner + G * N:], xbc[:, inner:inner + G * N], v, decay, None, 1.0, S, sl, cu, o)
    out = torch.zeros(T, inner + 8, dtype=dtype, device=dev)
    K.ssd_gate_norm(o, xbc, f(t["D"]), P, 0, f(t["norm"]), ng, eps, out)
    assert float(out[:, inner:].abs().max()) == 0.0
    for i, part in enumerate(out[:, :inner].split(new)):
      got[i].append(part)
    done = [a + b for a, b in zip(done, new)]
  for i in range(2):
    close(torch.cat(got[i]), want[i], dtype, f"sequence {i}", tol32=1e-4)
  assert float(S[0].min()) == 7.0 and float(conv[2].max()) == -3.0 if taps > 1 else True  # other slots untouched


@pytest.mark.parametrize("dev,dtype", DEVS)
@pytest.mark.parametrize("shared", [True, False])
def test_routed_experts_sum(dev, dtype, shared):
  T, k, D = 9, 3, 50
  y, sh, P = rnd(T * k, D + 14, seed=1), rnd(T, D + 6, seed=2), rnd(T, 11, seed=3)
  topw = torch.softmax(rnd(T, k, seed=4), -1)
  slot_of = torch.randperm(T * k, generator=torch.Generator().manual_seed(5)).reshape(T, k)
  want = (y[slot_of][:, :, :D] * topw[:, :, None]).sum(1)
  if shared:
    want = want + torch.sigmoid(P[:, 4:5]) * sh[:, :D]
  out = torch.empty(T, D, device=dev)
  K.moe_weighted_sum(y.float().to(dev), slot_of.int().reshape(-1).to(dev), topw.float().reshape(-1).to(dev), k,
                     sh.float().to(dev) if shared else None, P.float().to(dev) if shared else None, 4, out)
  close(out, want, torch.float32, "experts' sum")
