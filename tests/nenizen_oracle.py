"""Plain float64 implementation of the Nenizen design over whole sequences: one function per mechanism, written from
the design's equations, sharing no code with the package.  `forward(cfg, tensors, tokens)` takes config.json's dict and
a {name: tensor} checkpoint and returns (logits [n, vocab], [residual stream after every layer run])."""
import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
  y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
  return y if w is None else y * w


def rotate(x, positions, dims, base, interleaved):
  """x [n, heads, d]: the first `dims` dims of every head turned by position * base^(-2i/dims); partner of dim 2i is
  2i + 1 (interleaved) or of dim i is i + dims/2."""
  if not dims:
    return x
  n = x.shape[0]
  half = dims // 2
  f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
  ang = positions.to(F64)[:, None] * f[None, :]
  c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
  out = x.clone()
  if interleaved:
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
  else:
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
  return out


def visible(n, window):
  i = torch.arange(n)[:, None]
  j = torch.arange(n)[None, :]
  m = j <= i
  if window:
    m = m & (i - j < window)
  return m


def softmax_with_sink(s, mask, sink):
  """s [H, n, n]; sink [H] or None: one more term exp(sink_h) in the denominator, with no value."""
  s = s.masked_fill(~mask[None], float("-inf"))
  if sink is not None:
    s = torch.cat([s, sink.to(F64)[:, None, None].expand(s.shape[0], s.shape[1], 1)], -1)
  w = torch.softmax(s, -1)
  return w[..., :mask.shape[1]]


def latent_attention(h, m, T, p, kind, eps):
  """One latent-attention mixer on the normed input h [n, D]; m: the layer's "mixer" dict; T: tensors; p: 'l<i>.mix.'."""
  n = h.shape[0]
  H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
  g = lambda name: T[p + name].to(F64)
  if kind == "latent_attention":
    q = h @ g("q").T
  else:
    q = rms_norm(h @ g("dq").T, g("dq.norm"), eps) @ g("uq").T
  q = q.reshape(n, H, dn + dr)
  ckv = h @ g("dkv").T
  c = rms_norm(ckv[:, :R], g("dkv.norm"), eps)
  kr = ckv[:, R:].reshape(n, 1, dr)
  pos = torch.arange(n)
  inter = kind == "latent_attention"
  rot = m["rot"]
  qr = rotate(q[..., dn:], pos, rot["dims"], rot["base"], inter)
  kr = rotate(kr, pos, rot["dims"], rot["base"], inter)
  kn = (c @ g("uk").T).reshape(n, H, dn)
  v = (c @ g("uv").T).reshape(n, H, dv)
  s = (torch.einsum("ihd,jhd->hij", q[..., :dn], kn) + torch.einsum("ihd,jd->hij", qr, kr[:, 0])) * m["scale"]
  window = m["mask"]["size"] if kind == "latent_attention_2" else 0
  sink = T[p + "sink"] if kind == "latent_attention_3" else None
  w = softmax_with_sink(s, visible(n, window), sink)
  o = torch.einsum("hij,jhd->ihd", w, v)
  if kind == "latent_attention":
    o = o * torch.sigmoid(h @ g("g").T).reshape(n, H, dv)
  elif kind == "latent_attention_2":
    o = o * torch.sigmoid(h @ g("g").T).reshape(n, H, 1)
  return o.reshape(n, H * dv) @ g("o").T


def dense_ff(h, f, T, p):
  lim = f["limit"]
  g = torch.clamp(h @ T[p + "gate"].to(F64).T, max=lim)
  u = torch.clamp(h @ T[p + "up"].to(F64).T, -lim, lim)
  return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ T[p + "down"].to(F64).T


def silu_expert(h, T, p):
  a = h @ T[p + "gate"].to(F64).T
  return (a * torch.sigmoid(a) * (h @ T[p + "up"].to(F64).T)) @ T[p + "down"].to(F64).T


def moe_ff(h, f, T, p):
  E, k = f["router"]["experts"], f["router"]["top"]
  # router in 32-bit, as the design computes it (so that ties break as in the product)
  z = (h.float() @ T[p + "router"].float().T)
  s = torch.softmax(z, -1)
  w, idx = torch.topk(s, k, dim=-1)
  out = torch.zeros(h.shape[0], T[p + "e0.down"].shape[0], dtype=F64)
  for e in range(E):
    for j in range(k):
      rows = (idx[:, j] == e).nonzero().view(-1)
      if rows.numel():
        out[rows] += w[rows, j].to(F64)[:, None] * silu_expert(h[rows], T, p + f"e{e}.")
  if f.get("shared"):
    out = out + silu_expert(h, T, p + "shared.")
  return out


def layer(x, L, T, i, eps):
  p = f"l{i}."
  g = lambda name: T[p + name].to(F64)
  y = latent_attention(rms_norm(x, g("norm1"), eps), L["mixer"], T, p + "mix.", L["type"], eps)
  x = x + rms_norm(y, g("norm1b"), eps)
  f = L.get("mlp")
  if f is not None:
    h = rms_norm(x, g("norm2"), eps)
    y = dense_ff(h, f, T, p + "mlp.") if f["kind"] == "dense" else moe_ff(h, f, T, p + "mlp.")
    x = x + rms_norm(y, g("norm2b"), eps)
  return x


def forward(cfg, T, tokens):
  eps = cfg["norm"]["eps"]
  emb = T["embed"].to(F64)
  x = emb[torch.as_tensor(tokens).long()] * cfg["embedding"]["scale"]
  x0 = x
  loop = cfg.get("loop")
  n = len(cfg["layers"])
  runs = []
  if loop:
    runs += [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
      runs += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    runs += [(i, None) for i in range(loop["stop"], n)]
  else:
    runs = [(i, None) for i in range(n)]
  trail = []
  for i, t in runs:
    if t is not None:
      x = torch.cat([x, x0], -1) @ T["loop.in"].to(F64).T + T["loop.step"].to(F64)[t]
    x = layer(x, cfg["layers"][i], T, i, eps)
    trail.append(x)
  y = rms_norm(x, T["final.norm"].to(F64), eps) @ emb.T
  cap = cfg.get("logit_softcap")
  if cap:
    y = cap * torch.tanh(y / cap)
  return y, trail
