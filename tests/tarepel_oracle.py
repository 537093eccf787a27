"""A plain, slow Tarepel: one token at a time, float64, python lists as caches.  One function per mechanism.

It shares no code with the framework: it reads the same config dictionary (config.json's schema) and the same
name -> tensor dictionary a checkpoint holds, and keeps each sequence's memory in a dict of its own.

Notation: h is a layer's normed input (a vector), p the token's position in its sequence (from 0).
"""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
  return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
  return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(x):
  return x * torch.sigmoid(x)


def softplus(x):
  return torch.log1p(torch.exp(-x.abs())) + x.clamp(min=0)


def rotate(x, p, dims, base):
  """x [heads, dim]: dims i and i + dims/2 turn by the angle p * base^(-2i/dims); dims beyond `dims` pass."""
  half = dims // 2
  ang = p * base ** (-2.0 * torch.arange(half, dtype=F64) / dims)
  c, s = torch.cos(ang), torch.sin(ang)
  u, v = x[:, :half], x[:, half:dims]
  return torch.cat([u * c - v * s, v * c + u * s, x[:, dims:]], -1)


def chunk_gated_attention(W, pre, m, h, p, mem):
  """Keys of the query's own chunk up to the query; weights sigmoid(score + bias), not normalised; the value of a
  token is its key before rotation."""
  H, G, d = m["heads"], m["kv_heads"], m["dim"]
  q = rotate((W[pre + "q"] @ h).view(H, d), p, m["rot"]["dims"], m["rot"]["base"])
  k_raw = (W[pre + "k"] @ h).view(G, d)
  k = rotate(k_raw, p, m["rot"]["dims"], m["rot"]["base"])
  past = mem.setdefault(pre, [])
  past.append((k, k_raw))
  first = (p // m["mask"]["size"]) * m["mask"]["size"]
  out = torch.zeros(H, d, dtype=F64)
  for j in range(first, p + 1):
    kj, vj = past[j]
    for a in range(H):
      g = a // (H // G)
      out[a] += torch.sigmoid(torch.dot(q[a], kj[g]) * m["scale"] + W[pre + "pb"][a]) * vj[g]
  return W[pre + "o"] @ out.reshape(-1)


def short_conv(W, name, x, mem):
  """Causal convolution over time per channel (last tap = the current token), zeros before the start; then SiLU."""
  taps = W[name + ".conv"]
  hist = mem.setdefault(name, [torch.zeros_like(x) for _ in range(taps.shape[1] - 1)])
  window = hist + [x]
  y = sum(taps[:, j] * window[j] for j in range(taps.shape[1]))
  mem[name] = window[1:]
  return silu(y)


def gated_head_norm(o, weight, gate, eps):
  """Each head's read-out over its rms, times the shared weight, times SiLU of the gate."""
  return unit_rms(o, eps) * weight * silu(gate)


def gated_delta_rule(W, pre, m, h, mem, eps):
  H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
  q = short_conv(W, pre + "q", W[pre + "q"] @ h, mem).view(G, d)
  k = short_conv(W, pre + "k", W[pre + "k"] @ h, mem).view(G, d)
  v = short_conv(W, pre + "v", W[pre + "v"] @ h, mem).view(H, dv)
  q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) / math.sqrt(d)
  k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
  beta = torch.sigmoid(W[pre + "b"] @ h)
  g = torch.exp(-torch.exp(W[pre + "A_log"]) * softplus(W[pre + "a"] @ h + W[pre + "dt_bias"]))
  S = mem.setdefault(pre + "S", torch.zeros(H, d, dv, dtype=F64))
  o = torch.zeros(H, dv, dtype=F64)
  for a in range(H):
    kk, qq = k[a // (H // G)], q[a // (H // G)]
    S[a] = g[a] * S[a]
    u = beta[a] * (v[a] - S[a].t() @ kk)
    S[a] = S[a] + torch.outer(kk, u)
    o[a] = S[a].t() @ qq
  o = gated_head_norm(o, W[pre + "norm"], (W[pre + "g"] @ h).view(H, dv), eps)
  return W[pre + "o"] @ o.reshape(-1)


def gated_linear_attention(W, pre, m, h, mem, eps):
  H, d, dv = m["heads"], m["dim"], m["vdim"]
  q = (W[pre + "q"] @ h).view(H, d) / math.sqrt(d)
  k = (W[pre + "k"] @ h).view(H, d)
  v = (W[pre + "v"] @ h).view(H, dv)
  z = W[pre + "a2"] @ (W[pre + "a1"] @ h) + W[pre + "a2.b"]
  alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).view(H, d)
  S = mem.setdefault(pre + "S", torch.zeros(H, d, dv, dtype=F64))
  o = torch.zeros(H, dv, dtype=F64)
  for a in range(H):
    S[a] = alpha[a][:, None] * S[a] + torch.outer(k[a], v[a])
    o[a] = S[a].t() @ q[a]
  o = gated_head_norm(o, W[pre + "norm"], (W[pre + "g"] @ h).view(H, dv), eps)
  return W[pre + "o"] @ o.reshape(-1)


def feed_forward(W, pre, h):
  return W[pre + "down"] @ (gelu_tanh(W[pre + "gate"] @ h) * (W[pre + "up"] @ h))


def layer(W, i, L, x, p, mem, eps):
  """x + ls1 * mixer(h) + ls2 * ff(h), h = x / rms(x) * g: one norm, both sublayers read it."""
  pre = f"l{i}."
  h = unit_rms(x, eps) * W[pre + "norm1"]
  m = L["mixer"]
  if L["type"] == "parallel":
    y = m["left_scale"] * chunk_gated_attention(W, pre + "mix.left.", m["left"], h, p, mem) + \
        m["right_scale"] * gated_delta_rule(W, pre + "mix.right.", m["right"], h, mem, eps)
  else:
    y = gated_linear_attention(W, pre + "mix.", m, h, mem, eps)
  y = y * W[pre + "ls1"]
  if L["mlp"] is not None:
    y = y + feed_forward(W, pre + "mlp.", h) * W[pre + "ls2"]
  return x + y


class Oracle:
  def __init__(self, cfg: dict, tensors: dict):
    self.cfg = cfg
    self.W = {k: v.to(F64) for k, v in tensors.items()}
    self.eps = cfg["norm"]["eps"]

  def logits(self, tokens, want=None, residuals=None):
    """Logits [len(want), vocab] (all positions when want is None) of one sequence run from its start."""
    mem, out = {}, []
    for p, tok in enumerate(tokens):
      x = self.W["embed"][int(tok)].clone()
      for i, L in enumerate(self.cfg["layers"]):
        x = layer(self.W, i, L, x, p, mem, self.eps)
        if residuals is not None:
          residuals.append(x.clone())
      if want is None or p in want:
        out.append((self.W["head"] @ (unit_rms(x, self.eps) * self.W["final.norm"])) * self.cfg["logit_scale"])
    return torch.stack(out)
