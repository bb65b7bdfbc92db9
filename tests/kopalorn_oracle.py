"""Plain float64 implementation of the Kopalorn design: whole sequences, token by token where a state is carried, one
function per mechanism.  Written from the design's equations only; it shares no code with the package and is slow on
purpose.  `tensors` maps checkpoint names to torch tensors, `cfg` is the parsed config.json."""
import math

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
  mu = x.mean(-1, keepdim=True)
  var = ((x - mu) ** 2).mean(-1, keepdim=True)
  return (x - mu) / torch.sqrt(var + eps) * w + b


def rms(x, eps):
  return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rope_interleaved(x, base, dims):
  """x [n, heads, d]: dims (2i, 2i + 1), i < dims / 2, of the token at position p turn by p * base^(-2i / dims)."""
  if not dims:
    return x
  n = x.shape[0]
  i = torch.arange(dims // 2, dtype=F64)
  ang = torch.arange(n, dtype=F64)[:, None] * base ** (-2.0 * i / dims)[None, :]
  c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
  out = x.clone()
  u, v = x[..., 0:dims:2], x[..., 1:dims:2]
  out[..., 0:dims:2] = u * c - v * s
  out[..., 1:dims:2] = v * c + u * s
  return out


def softmax_attention(q, k, v, scale, window):
  """q [n, H, d], k [n, G, d], v [n, G, dv] -> [n, H, dv]; token i sees j with j <= i and (window > 0) i - j < window."""
  n, H, _ = q.shape
  G = k.shape[1]
  out = torch.zeros(n, H, v.shape[2], dtype=F64)
  for h in range(H):
    g = h // (H // G)
    for i in range(n):
      lo = max(0, i - window + 1) if window else 0
      s = (k[lo:i + 1, g] @ q[i, h]) * scale
      p = torch.softmax(s, 0)
      out[i, h] = p @ v[lo:i + 1, g]
  return out


def diff_attention(h, m, t, p, eps):
  """Differential attention with a sliding window, rotation, a per-head norm and a per-head output gate."""
  n = h.shape[0]
  H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
  q = (h @ t[p + "q"].T).reshape(n, H, 2, d)
  k = (h @ t[p + "k"].T).reshape(n, G, 2, d)
  v = (h @ t[p + "v"].T).reshape(n, G, dv)
  rot = m.get("rot") or {}
  window = int((m.get("mask") or {}).get("size", 0))
  maps = []
  for j in range(2):
    qj = rope_interleaved(q[:, :, j], float(rot.get("base", 1.0)), int(rot.get("dims", 0)))
    kj = rope_interleaved(k[:, :, j], float(rot.get("base", 1.0)), int(rot.get("dims", 0)))
    maps.append(softmax_attention(qj, kj, v, m["scale"], window))
  lam = math.exp(float((t[p + "lq1"] * t[p + "lk1"]).sum())) - math.exp(float((t[p + "lq2"] * t[p + "lk2"]).sum())) + m["diff"]
  o = rms(maps[0] - lam * maps[1], eps) * (1.0 - m["diff"])
  gate = torch.sigmoid(h @ t[p + "g"].T)  # [n, H]
  return (o * gate[:, :, None]).reshape(n, H * dv) @ t[p + "o"].T


def mlstm(h, m, t, p, eps):
  """Matrix-memory LSTM with a stabilising running maximum that starts at zero."""
  n = h.shape[0]
  H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
  q = (h @ t[p + "q"].T).reshape(n, H, d) * d ** -0.5
  k = (h @ t[p + "k"].T).reshape(n, H, d)
  v = (h @ t[p + "v"].T).reshape(n, H, dv)
  ig = cap * torch.tanh((h @ t[p + "i"].T + t[p + "i.b"]) / cap)
  fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ t[p + "f"].T + t[p + "f.b"]) / cap))
  out = torch.zeros(n, H, dv, dtype=F64)
  for hd in range(H):
    S = torch.zeros(d, dv, dtype=F64)
    nv = torch.zeros(d, dtype=F64)
    mx = 0.0
    for i in range(n):
      f, g = float(fg[i, hd]), float(ig[i, hd])
      new = max(f + mx, g)
      S = math.exp(f + mx - new) * S + math.exp(g - new) * torch.outer(k[i, hd], v[i, hd])
      nv = math.exp(f + mx - new) * nv + math.exp(g - new) * k[i, hd]
      mx = new
      out[i, hd] = (S.T @ q[i, hd]) / (max(abs(float(nv @ q[i, hd])), math.exp(-mx)) + 1e-6)
  o = rms(out, eps).reshape(n, H * dv) * t[p + "norm"]
  return (o * torch.sigmoid(h @ t[p + "g"].T)) @ t[p + "o"].T


def gated_attention(h, m, t, p):
  """Causal softmax attention with biased projections, no rotation, an element-wise output gate."""
  n = h.shape[0]
  H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
  q = (h @ t[p + "q"].T + t[p + "q.b"]).reshape(n, H, d)
  k = (h @ t[p + "k"].T + t[p + "k.b"]).reshape(n, G, d)
  v = (h @ t[p + "v"].T + t[p + "v.b"]).reshape(n, G, dv)
  o = softmax_attention(q, k, v, m["scale"], 0).reshape(n, H * dv)
  return (o * torch.sigmoid(h @ t[p + "g"].T)) @ t[p + "o"].T


def lightning(h, m, t, p, eps):
  """Linear attention with one fixed decay per head."""
  n = h.shape[0]
  H, d, dv = m["heads"], m["dim"], m["vdim"]
  silu = torch.nn.functional.silu
  q = silu(h @ t[p + "q"].T).reshape(n, H, d)
  k = silu(h @ t[p + "k"].T).reshape(n, H, d)
  v = silu(h @ t[p + "v"].T).reshape(n, H, dv)
  out = torch.zeros(n, H, dv, dtype=F64)
  for hd in range(H):
    S = torch.zeros(d, dv, dtype=F64)
    for i in range(n):
      S = float(m["decay"][hd]) * S + torch.outer(k[i, hd], v[i, hd])
      out[i, hd] = S.T @ q[i, hd]
  o = rms(out.reshape(n, H * dv), eps) * t[p + "norm"]
  return (o * torch.sigmoid(h @ t[p + "g"].T)) @ t[p + "o"].T


def parallel_mixer(h, m, t, p, eps):
  a = gated_attention(h, m["left"], t, p + "left.")
  b = lightning(h, m["right"], t, p + "right.", eps)
  return 0.5 * (rms(a, eps) * t[p + "left.out"] + rms(b, eps) * t[p + "right.out"])


def relu2_expert(h, t, p):
  return torch.relu(h @ t[p + "up"].T) ** 2 @ t[p + "down"].T


def route(z, corr, r):
  """Router logits z [E] -> (chosen experts, weights): sigmoid scores, group-limited choice on the corrected scores."""
  E, top = r["experts"], r["top"]
  s = torch.sigmoid(z)
  choice = s + corr
  gr = r.get("groups") or {"count": 1, "keep": 1}
  cnt, keep = int(gr["count"]), int(gr["keep"])
  per = E // cnt
  gscore = torch.stack([choice[g * per:(g + 1) * per].topk(min(2, per)).values.sum() for g in range(cnt)])
  kept = gscore.topk(keep).indices.tolist()
  masked = torch.full((E,), -math.inf, dtype=F64)
  for g in kept:
    masked[g * per:(g + 1) * per] = choice[g * per:(g + 1) * per]
  idx = masked.topk(top).indices
  w = s[idx]
  return idx.tolist(), (w / (w.sum() + 1e-20) * r["scale"]).tolist()


def moe(h, f, t, p):
  n = h.shape[0]
  z = h @ t[p + "router"].T
  out = torch.zeros(n, t[p + "e0.down"].shape[0], dtype=F64)
  for i in range(n):
    idx, w = route(z[i], t[p + "correction"], f["router"])
    for e, we in zip(idx, w):
      out[i] += we * relu2_expert(h[i], t, f"{p}e{e}.")
  if f.get("shared"):
    out = out + torch.sigmoid(h @ t[p + "shared.sg"].T) * relu2_expert(h, t, p + "shared.")
  return out


def forward(cfg, tensors, tokens, collect=None):
  """Logits [n, vocab] of one sequence; collect: a list that receives the residual stream after every layer run."""
  t = {k: v.to(F64) for k, v in tensors.items()}
  eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
  x0 = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
  x = x0.clone()
  L = len(cfg["layers"])
  lp = cfg.get("loop")
  runs = []
  if lp:
    runs += [(i, -1) for i in range(lp["start"])]
    for ps in range(lp["times"]):
      runs += [(i, ps if i == lp["start"] else -1) for i in range(lp["start"], lp["stop"])]
    runs += [(i, -1) for i in range(lp["stop"], L)]
  else:
    runs = [(i, -1) for i in range(L)]
  for i, ps in runs:
    if ps >= 0:
      if ps > 0:
        x = x + x0
      x = x + t["loop.step"][ps]
    lay, p = cfg["layers"][i], f"l{i}."

    def ln(name, y):
      return layer_norm(y, t[p + name], t[p + name + ".b"], eps)
    hin = ln("norm1", x)
    kind = lay["type"]
    if kind == "attention":
      y = diff_attention(hin, lay["mixer"], t, p + "mix.", eps)
    elif kind == "mlstm":
      y = mlstm(hin, lay["mixer"], t, p + "mix.", eps)
    elif kind == "parallel":
      y = parallel_mixer(hin, lay["mixer"], t, p + "mix.", eps)
    else:
      raise ValueError(kind)
    x = x + mult * ln("norm1b", y)
    if lay.get("mlp"):
      x = x + mult * ln("norm2b", moe(ln("norm2", x), lay["mlp"], t, p + "mlp."))
    if collect is not None:
      collect.append(x.clone())
  return layer_norm(x, t["final.norm"], t["final.norm.b"], eps) @ t["head"].T
