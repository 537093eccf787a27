"""Plain float64 implementation of the Mogelix design, one function per mechanism, whole sequences at a time.

It shares no code with the package: tests compare the framework's ops, runner and engine against these functions.
A model is (cfg, tensors): cfg is the config.json dictionary, tensors maps checkpoint names to torch tensors.

Notation: n tokens, D width, positions 0 .. n-1.  rms(x) = sqrt(mean(x^2) + eps) over the last axis.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_div(x: torch.Tensor, eps: float) -> torch.Tensor:
  return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
  return x * torch.sigmoid(x)


def softplus(x):
  return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


# ------------------------------------------------------------------ rotation
def rot_freqs(rot: dict) -> torch.Tensor:
  """dims/2 angular frequencies base^(-2i/dims); with "scaling": long wavelengths divided by factor, short ones
  kept, a linear blend between the two wavelength bounds original/low and original/high."""
  dims = int(rot["dims"])
  f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
  sc = rot.get("scaling")
  if sc:
    factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = []
    for fi in f.tolist():
      wl = 2 * math.pi / fi
      if wl < orig / high:
        out.append(fi)
      elif wl > orig / low:
        out.append(fi / factor)
      else:
        s = (orig / wl - low) / (high - low)
        out.append((1 - s) * fi / factor + s * fi)
    f = torch.tensor(out, dtype=F64)
  return f


def rotate(x: torch.Tensor, pos: torch.Tensor, rot: dict | None) -> torch.Tensor:
  """x [n, heads, d]: dimension i pairs with i + dims/2 inside the first dims dimensions; the rest pass."""
  if not rot or not int(rot.get("dims", 0)):
    return x
  dims = int(rot["dims"])
  half = dims // 2
  ang = pos.to(F64)[:, None] * rot_freqs(rot)[None, :]  # [n, half]
  c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
  u, v = x[..., :half], x[..., half:dims]
  return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


# ------------------------------------------------------------------ attention
def visible_keys(i: int, window: int, pool: int):
  """(token positions, pooled block indices) that query position i sees.  window 0: every earlier token."""
  if window <= 0:
    return list(range(i + 1)), []
  toks = [j for j in range(i + 1) if i - j < window]
  blocks = [b for b in range((i // pool) + 1 if pool else 0) if b * pool + pool - 1 <= i - window] if pool else []
  return toks, blocks


def window_pool_attention(q, k, v, sink, scale: float, window: int, pool: int) -> torch.Tensor:
  """q [n, H, d], k [n, G, d], v [n, G, dv] (k as the cache holds it), sink [H] or None -> [n, H, dv].
  One softmax over the window's tokens, the pooled blocks wholly before the window and the sink (which has no value)."""
  n, H, d = q.shape
  G = k.shape[1]
  rep = H // G
  out = torch.zeros(n, H, v.shape[-1], dtype=F64)
  nb = n // pool if pool else 0
  kp = k[:nb * pool].reshape(nb, pool, G, d).mean(1) if nb else None
  vp = v[:nb * pool].reshape(nb, pool, G, -1).mean(1) if nb else None
  for i in range(n):
    toks, blocks = visible_keys(i, window, pool)
    for h in range(H):
      g = h // rep
      ks = torch.cat([k[toks, g]] + ([kp[blocks, g]] if blocks else []))
      vs = torch.cat([v[toks, g]] + ([vp[blocks, g]] if blocks else []))
      s = ks @ q[i, h] * scale
      m = s.max() if sink is None else torch.maximum(s.max(), sink[h])
      e = torch.exp(s - m)
      den = e.sum() + (torch.exp(sink[h] - m) if sink is not None else 0.0)
      out[i, h] = (e[:, None] * vs).sum(0) / den
  return out


def attention_keys(h, m: dict, t: dict, p: str, eps: float, pos):
  """Keys (rotated, then divided by their rms) and values of a layer that has projections."""
  n = h.shape[0]
  G, d, dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
  k = (h @ t[p + "k"].to(F64).T + t[p + "k.b"].to(F64)).reshape(n, G, d)
  v = (h @ t[p + "v"].to(F64).T + t[p + "v.b"].to(F64)).reshape(n, G, dv)
  return rms_div(rotate(k, pos, m.get("rot")), eps), v


def attention_mixer(h, m: dict, t: dict, p: str, eps: float, kv, cache_round=None) -> torch.Tensor:
  """h [n, D] -> [n, D].  kv = (k, v) of this layer or of the layer named by kv_from."""
  n = h.shape[0]
  H, d = int(m["heads"]), int(m["dim"])
  pos = torch.arange(n)
  q = (h @ t[p + "q"].to(F64).T + t[p + "q.b"].to(F64)).reshape(n, H, d)
  q = rms_div(rotate(q, pos, m.get("rot")), eps)
  k, v = kv
  mask = m.get("mask") or {}
  sink = t[p + "sink"].to(F64) if p + "sink" in t else None
  o = window_pool_attention(q, k, v, sink, float(m["scale"]), int(mask.get("size", 0)), int(mask.get("pool", 0)))
  return o.reshape(n, -1) @ t[p + "o"].to(F64).T


# ------------------------------------------------------------------ mamba2
def causal_conv(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
  """x [n, C], w [C, taps] (last column: the current token), zeros before the start."""
  n, C = x.shape
  taps = w.shape[1]
  xp = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], 0)
  return sum(w[:, j] * xp[j:j + n] for j in range(taps)) + b


def ssd_scan(x, B, Cm, dt, A_log, Dskip) -> torch.Tensor:
  """x [n, H, dv], B / Cm [n, G, N], dt [n, H] (after softplus): S <- exp(-exp(A_log) dt) S + dt B x^T per head,
  y = S^T C + D x."""
  n, H, dv = x.shape
  G, N = B.shape[1], B.shape[2]
  rep = H // G
  y = torch.zeros(n, H, dv, dtype=F64)
  S = torch.zeros(H, N, dv, dtype=F64)
  for t in range(n):
    for h in range(H):
      g = h // rep
      S[h] = torch.exp(-torch.exp(A_log[h]) * dt[t, h]) * S[h] + dt[t, h] * torch.outer(B[t, g], x[t, h])
      y[t, h] = S[h].T @ Cm[t, g] + Dskip[h] * x[t, h]
  return y


def mamba2_mixer(h, m: dict, t: dict, p: str, eps: float) -> torch.Tensor:
  n = h.shape[0]
  H, dv, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
  inner = H * dv
  P = h @ t[p + "in"].to(F64).T
  z, xbc, dt = P[:, :inner], P[:, inner:2 * inner + 2 * G * N], P[:, 2 * inner + 2 * G * N:]
  xbc = silu(causal_conv(xbc, t[p + "conv"].to(F64), t[p + "conv.b"].to(F64)))
  x = xbc[:, :inner].reshape(n, H, dv)
  B = xbc[:, inner:inner + G * N].reshape(n, G, N)
  Cm = xbc[:, inner + G * N:].reshape(n, G, N)
  dt = softplus(dt + t[p + "dt_bias"].to(F64))
  y = ssd_scan(x, B, Cm, dt, t[p + "A_log"].to(F64), t[p + "D"].to(F64)).reshape(n, inner)
  y = y * silu(z)
  ng = int(m.get("norm_groups", 1))
  y = rms_div(y.reshape(n, ng, inner // ng), eps).reshape(n, inner) * t[p + "norm"].to(F64)
  return y @ t[p + "o"].to(F64).T


# ------------------------------------------------------------------ feed-forward
def polynorm(z, coef, eps: float):
  a, b, c, e = coef.to(F64).tolist()
  return a * rms_div(z, eps) + b * rms_div(z * z, eps) + c * rms_div(z * z * z, eps) + e


def dense_ff(h, t: dict, p: str, eps: float):
  return polynorm(h @ t[p + "up"].to(F64).T, t[p + "act"], eps) @ t[p + "down"].to(F64).T


def relu2_expert(h, t: dict, p: str):
  return torch.relu(h @ t[p + "up"].to(F64).T) ** 2 @ t[p + "down"].to(F64).T


def moe_ff(h, mlp: dict, t: dict, p: str):
  E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
  logits = h @ t[p + "router"].to(F64).T + t[p + "router.b"].to(F64)
  out = torch.zeros_like(h)
  for i in range(h.shape[0]):
    val, idx = torch.topk(logits[i], top)
    w = torch.softmax(val, 0)
    for j in range(top):
      out[i] += w[j] * relu2_expert(h[i:i + 1], t, p + f"e{int(idx[j])}.")[0]
  if mlp.get("shared"):
    gate = torch.sigmoid(h @ t[p + "shared.sg"].to(F64).T)  # [n, 1]
    out = out + gate * relu2_expert(h, t, p + "shared.")
  return out


def feed_forward(h, mlp: dict, t: dict, p: str, eps: float):
  return dense_ff(h, t, p, eps) if mlp.get("kind", "dense") == "dense" else moe_ff(h, mlp, t, p)


# ------------------------------------------------------------------ the model
def gated(y, h, t: dict, name: str):
  """y * sigmoid(W h + b) when the layer has that gate."""
  if name not in t:
    return y
  return y * torch.sigmoid(h @ t[name].to(F64).T + t[name + ".b"].to(F64))


def forward(cfg: dict, t: dict, tokens, return_layers: bool = False):
  """tokens: list of ids of ONE sequence -> logits [n, vocab] (and the residual stream after every layer)."""
  eps, alpha = float(cfg["norm"]["eps"]), float(cfg.get("postln_alpha", 1.0))
  x = t["embed"].to(F64)[torch.tensor(tokens, dtype=torch.long)]
  n = x.shape[0]
  pos = torch.arange(n)
  kvs, streams = {}, []
  for i, L in enumerate(cfg["layers"]):
    p, m = f"l{i}.", L["mixer"]
    if L["type"] == "attention":
      if "kv_from" in m and m["kv_from"] is not None:
        kv = kvs[int(m["kv_from"])]
      else:
        kv = kvs[i] = attention_keys(x, m, t, p + "mix.", eps, pos)
      y = attention_mixer(x, m, t, p + "mix.", eps, kv)
    elif L["type"] == "mamba2":
      y = mamba2_mixer(x, m, t, p + "mix.", eps)
    else:
      raise ValueError(L["type"])
    x = rms_div(alpha * x + gated(y, x, t, p + "rg1"), eps) * t[p + "norm1"].to(F64)
    if L.get("mlp"):
      y = feed_forward(x, L["mlp"], t, p + "mlp.", eps)
      x = rms_div(alpha * x + gated(y, x, t, p + "rg2"), eps) * t[p + "norm2"].to(F64)
    streams.append(x)
  logits = (rms_div(x, eps) * t["final.norm"].to(F64)) @ t["head"].to(F64).T
  return (logits, torch.stack(streams)) if return_layers else logits
