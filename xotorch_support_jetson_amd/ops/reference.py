"""Plain-PyTorch fp32 implementations of every kernel in the library.

These are (1) the numerical oracles the HIP kernels are tested against and (2) the compute path on
CPU-only hosts (BASELINE config 1: Llama-3.2-1B on the CPU engine).  Semantics match the kernels
exactly, including the paged KV layout (K [pages, Hkv, 64, Dh], V [pages, Hkv, Dh, 64] storage holding each page
chunk-major, see v_chunks).
"""
from __future__ import annotations

import os
import weakref

import torch
import torch.nn.functional as F

PAGE = 64


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, residual: torch.Tensor | None = None):
  """Returns (normed, new_residual). new_residual = bf16(x + residual) when residual is given."""
  if residual is not None:
    x = (x.float() + residual.float()).to(x.dtype)
  xf = x.float()
  y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
  return y.to(x.dtype), (x if residual is not None else None)


def rope(x: torch.Tensor, pos: torch.Tensor, cos_sin: torch.Tensor, inverse: bool = False) -> torch.Tensor:
  """x [T, nh, Dh]; HF rotate-half convention."""
  Dh = x.shape[-1]
  half = Dh // 2
  cs = cos_sin[pos.long()].to(x.device)  # [T, Dh]
  cos, sin = cs[:, None, :half], cs[:, None, half:]
  if inverse:
    sin = -sin
  xf = x.float()
  x0, x1 = xf[..., :half], xf[..., half:]
  return torch.cat([x0 * cos - x1 * sin, x1 * cos + x0 * sin], dim=-1).to(x.dtype)


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
  Fd = gu.shape[-1] // 2
  g, u = gu[..., :Fd].float(), gu[..., Fd:].float()
  return (F.silu(g) * u).to(gu.dtype)


# fp32 copies of low-precision CPU weights, made once per tensor and re-made when the tensor is written in place
# (its version counter moves) or re-pointed: without them every CPU token widened every weight again (~1 s per
# token for Llama-3.2-1B).  Tensors that require grad (trained parameters) are widened per call as before.
# at most this many bytes of fp32 copies live at once (XOT_CPU_F32_CACHE_GB): a model too large for it widens the
# rest per call, as before
_F32_BUDGET = int(float(os.environ.get("XOT_CPU_F32_CACHE_GB", "12")) * (1 << 30))
_f32_bytes = [0]


def _release(n: int) -> None:
  _f32_bytes[0] -= n


def _wide(w: torch.Tensor) -> torch.Tensor:
  if w.dtype == torch.float32 or w.device.type != "cpu" or w.requires_grad or w.grad_fn is not None:
    return w.float()
  key = (w._version, w.data_ptr(), tuple(w.shape), tuple(w.stride()))
  got = getattr(w, "_xot_f32", None)  # kept on the tensor: freed with it
  if got is not None and got[0] == key:
    return got[1]
  f = w.float()
  n = f.numel() * 4
  if got is None and _f32_bytes[0] + n > _F32_BUDGET:
    return f
  if got is None:
    _f32_bytes[0] += n
    weakref.finalize(w, _release, n)
  w._xot_f32 = (key, f)
  return f


def linear(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
  y = x.float() @ _wide(w).t()
  if bias is not None:
    y = y + bias.float()
  return y


def v_chunks(v_cache: torch.Tensor) -> torch.Tensor:
  """The V pool [pages, Hkv, Dh, BS] (storage shape) as the layout the kernels use: each page of a KV head
  chunk-major, [BS / 8 chunks][Dh][8 keys] (csrc/common.h v_page_off)."""
  nb, Hkv, Dh, BS = v_cache.shape
  return v_cache.view(nb, Hkv, BS // 8, Dh, 8)


def write_kv(k: torch.Tensor, v: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor):
  """k, v [T, Hkv, Dh] -> paged caches at global slots (slot < 0 skipped)."""
  BS = k_cache.shape[2]
  ok = slots >= 0
  s = slots[ok].long()
  blk, off = s // BS, s % BS
  k_cache[blk, :, off, :] = k[ok].to(k_cache.dtype)
  v_chunks(v_cache)[blk, :, off // 8, :, off % 8] = v[ok].to(v_cache.dtype)


def gather_kv(k_cache, v_cache, table, n):
  """Dense [n, Hkv, Dh] K and V for one sequence from its block table."""
  BS = k_cache.shape[2]
  npg = (n + BS - 1) // BS
  pages = table[:npg].long()
  k = k_cache[pages].permute(0, 2, 1, 3).reshape(npg * BS, k_cache.shape[1], k_cache.shape[3])[:n]
  v = v_chunks(v_cache)[pages].permute(0, 2, 4, 1, 3).reshape(npg * BS, v_cache.shape[1], v_cache.shape[2])[:n]
  return k, v


def _attend(q, k, v, scale, causal_offset: int | None):
  # q [S, H, Dh], k/v [T, Hkv, Dh]
  H, Hkv = q.shape[1], k.shape[1]
  G = H // Hkv
  kf = k.float().repeat_interleave(G, dim=1)
  vf = v.float().repeat_interleave(G, dim=1)
  s = torch.einsum("shd,thd->hst", q.float(), kf) * scale
  if causal_offset is not None:
    S, T = q.shape[0], k.shape[0]
    qpos = torch.arange(S, device=q.device)[:, None] + causal_offset
    kpos = torch.arange(T, device=q.device)[None, :]
    s = s.masked_fill(kpos > qpos, float("-inf"))
  p = torch.softmax(s, dim=-1)
  return torch.einsum("hst,thd->shd", p, vf)


def attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale):
  """q [B, H, Dh] -> [B, H, Dh]"""
  out = torch.empty_like(q)
  for b in range(q.shape[0]):
    n = int(ctx_lens[b])
    if n <= 0:
      out[b] = 0
      continue
    k, v = gather_kv(k_cache, v_cache, block_tables[b], n)
    out[b] = _attend(q[b:b + 1], k, v, scale, None)[0].to(q.dtype)
  return out


def attn_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, scale):
  """q [T, H, Dh] (new tokens of all sequences) -> [T, H, Dh]; causal against the cached context."""
  out = torch.empty_like(q)
  for b in range(ctx_lens.numel()):
    q0, q1 = int(cu_q[b]), int(cu_q[b + 1])
    if q1 <= q0:
      continue
    n = int(ctx_lens[b])
    k, v = gather_kv(k_cache, v_cache, block_tables[b], n)
    out[q0:q1] = _attend(q[q0:q1], k, v, scale, n - (q1 - q0)).to(q.dtype)
  return out


def sample_greedy(logits: torch.Tensor) -> torch.Tensor:
  return logits.float().argmax(dim=-1).to(torch.int32)


def topk_mask(logits: torch.Tensor, k: int) -> torch.Tensor:
  """Boolean mask of entries >= the k-th largest value (ties kept), per row."""
  kth = torch.topk(logits.float(), k, dim=-1).values[:, -1:]
  return logits.float() >= kth


def cross_entropy(logits: torch.Tensor, targets: torch.Tensor):
  """Per-row loss (0 where target < 0) and lse."""
  lf = logits.float()
  lse = torch.logsumexp(lf, dim=-1)
  valid = targets >= 0
  tgt = targets.clamp(min=0).long()
  picked = lf.gather(1, tgt[:, None])[:, 0]
  loss = torch.where(valid, lse - picked, torch.zeros_like(lse))
  return loss, lse


# ------------------------------------------------------------------ DeepSeek MLA / MoE routing
def mla_prep(ckv, kv_ln, q, qpe_off: int, H: int, pos, cos_sin, slots, cache, eps: float):
  """Latent rmsnorm (HF DeepseekV2RMSNorm rounding: normalise, cast, times weight) + rope of the shared
  key -> cache[slot] = [c | k_pe]; q_pe of every head rotated in place.  cache [pages, 64, DL + DR]."""
  DL = kv_ln.numel()
  DR = cos_sin.shape[1]
  T = ckv.shape[0]
  x = ckv[:, :DL].float()
  c = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)).to(ckv.dtype).float() * kv_ln.float()
  kpe = rope(ckv[:, DL:DL + DR].reshape(T, 1, DR), pos, cos_sin)[:, 0]
  qpe = q[:, qpe_off:qpe_off + H * DR].reshape(T, H, DR)
  q[:, qpe_off:qpe_off + H * DR] = rope(qpe, pos, cos_sin).reshape(T, H * DR)
  ok = slots >= 0
  flat = cache.view(-1, cache.shape[-1])
  row = torch.cat([c.to(cache.dtype), kpe.to(cache.dtype)], 1)
  flat[slots[ok].long()] = row[ok]


def mla_attn(q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, scale: float):
  """q_lat [H, T, DL], q_pe [T, >= H*DR] -> o_lat [H, T, DL]: causal multi-query attention over the latent."""
  H, T, DL = q_lat.shape
  DR = cache.shape[-1] - DL
  out = torch.zeros_like(q_lat)
  for b in range(ctx_lens.numel()):
    q0, q1 = int(cu_q[b]), int(cu_q[b + 1])
    n = int(ctx_lens[b])
    if q1 <= q0 or n <= 0:
      continue
    npg = -(-n // PAGE)
    lat = cache[block_tables[b, :npg].long()].reshape(npg * PAGE, -1)[:n].float()  # [n, DL + DR]
    qf = torch.cat([q_lat[:, q0:q1].float(), q_pe[q0:q1, :H * DR].reshape(q1 - q0, H, DR).permute(1, 0, 2).float()], 2)
    s = torch.einsum("hsd,td->hst", qf, lat) * scale
    qpos = torch.arange(q1 - q0)[:, None] + (n - (q1 - q0))
    s = s.masked_fill(torch.arange(n)[None, :] > qpos, float("-inf"))
    p = torch.softmax(s, -1)
    out[:, q0:q1] = torch.einsum("hst,td->hsd", p, lat[:, :DL]).to(out.dtype)
  return out


def moe_route_ds(logits, bias, k: int, n_group: int, topk_group: int, method: int, sigmoid: bool, norm: bool,
                 scale: float):
  """HF DeepseekV2TopkRouter / DeepseekV3TopkRouter -> (topw [T, k], topi [T, k])."""
  lf = logits.float()
  scores = torch.sigmoid(lf) if sigmoid else torch.softmax(lf, -1)
  choice = scores + bias.float() if bias is not None else scores
  T, E = lf.shape
  if n_group > 1 and topk_group < n_group:
    g = choice.view(T, n_group, E // n_group)
    gs = g.topk(2, -1).values.sum(-1) if method == 2 and E // n_group > 1 else g.max(-1).values
    keep = torch.zeros_like(gs).scatter_(1, gs.topk(topk_group, -1).indices, 1.0)
    mask = keep[:, :, None].expand(T, n_group, E // n_group).reshape(T, E).bool()
    choice = choice.masked_fill(~mask, float("-inf"))
  topi = choice.topk(k, -1).indices
  topw = scores.gather(1, topi)
  if norm:
    topw = topw / (topw.sum(-1, keepdim=True) + 1e-20)
  return topw * scale, topi


# ------------------------------------------------------------------ mixers on an fp32 residual stream
# Torch twins of csrc/mixers.hip.  P is a fused projection's output [T, n] (fp32 on a GPU; whatever the CPU GEMM
# returned here), addressed by column offsets.  Per-sequence loops are fine: this is the CPU path.
def resid_scale_norm(x, y1, s1, y2, s2, gain, eps, out):
  """x += s1 * y1 (+ s2 * y2) in place; out = x / sqrt(mean(x^2) + eps) * gain."""
  D = x.shape[1]
  if y1 is not None:
    a = s1.float() * y1[:, :D].float()
    if y2 is not None:
      a = a + s2.float() * y2[:, :D].float()
    x += a
  if out is not None:
    out[:, :D] = (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * gain.float()).to(out.dtype)


def gelu_mul(P, gate_off, up_off, Fd, out):
  z, u = P[:, gate_off:gate_off + Fd].float(), P[:, up_off:up_off + Fd].float()
  out[:, :Fd] = (0.5 * z * (1 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3))) * u).to(out.dtype)


def rope_kv_store(P, q_off, k_off, v_off, H, G, d, R, pos, cos_sin, slots, q_out, k_cache, v_cache):
  T = P.shape[0]
  q = P[:, q_off:q_off + H * d].float().reshape(T, H, d)
  k = P[:, k_off:k_off + G * d].float().reshape(T, G, d)
  v = k if v_off < 0 else P[:, v_off:v_off + G * d].float().reshape(T, G, d)
  half = R // 2

  def rot(x):
    if R == 0:
      return x
    cs = cos_sin[pos.long()]
    c, s = cs[:, None, :half], cs[:, None, half:]
    a, b = x[..., :half], x[..., half:R]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., R:]], -1)
  q_out.copy_(rot(q).to(q_out.dtype))
  ok = slots >= 0
  s = slots[ok].long()
  k_cache[s // PAGE, :, s % PAGE] = rot(k)[ok].to(k_cache.dtype)
  v_cache[s // PAGE, :, :, s % PAGE] = v[ok].to(v_cache.dtype)


def attn_gated_chunk(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, pb, scale, chunk, out_scale, out, max_qlen=0):
  T, H, d = q.shape
  G = k_cache.shape[1]
  for b in range(ctx_lens.numel()):
    t0, t1, n = int(cu_q[b]), int(cu_q[b + 1]), int(ctx_lens[b])
    if n <= 0 or t1 == t0:
      continue
    npg = -(-n // PAGE)
    pages = block_tables[b, :npg].long()
    k = k_cache[pages].permute(0, 2, 1, 3).reshape(npg * PAGE, G, d)[:n].float().repeat_interleave(H // G, 1)
    v = v_cache[pages].permute(0, 3, 1, 2).reshape(npg * PAGE, G, d)[:n].float().repeat_interleave(H // G, 1)
    qpos = torch.arange(n - (t1 - t0), n)[:, None]
    kpos = torch.arange(n)[None, :]
    vis = (kpos <= qpos) & (kpos // chunk == qpos // chunk)
    s = torch.einsum("shd,thd->hst", q[t0:t1].float(), k) * scale + pb.float()[:, None, None]
    w = torch.sigmoid(s) * vis
    o = torch.einsum("hst,thd->shd", w, v) * out_scale
    out[t0:t1] = o.reshape(t1 - t0, H * d).to(out.dtype)


def delta_prep(P, x_off, b_off, a_off, conv_w, conv_state, state_slots, cu_q, A_log, dt_bias, H, G, d, dv, qkv, beta, decay):
  C = 2 * G * d + H * dv
  taps = conv_w.shape[1]
  for b in range(state_slots.numel()):
    t0, t1, slot = int(cu_q[b]), int(cu_q[b + 1]), int(state_slots[b])
    if slot < 0 or t1 == t0:
      continue
    x = torch.cat([conv_state[slot], P[t0:t1, x_off:x_off + C].float()], 0)  # [taps - 1 + n, C]
    y = sum(conv_w[:, j].float() * x[j:j + t1 - t0] for j in range(taps))
    y = F.silu(y)
    qk = y[:, :2 * G * d].reshape(t1 - t0, 2 * G, d)
    qk = qk / torch.sqrt(qk.pow(2).sum(-1, keepdim=True) + 1e-6)
    qk[:, :G] *= d ** -0.5
    qkv[t0:t1] = torch.cat([qk.reshape(t1 - t0, -1), y[:, 2 * G * d:]], 1)
    conv_state[slot] = x[x.shape[0] - (taps - 1):]
    beta[t0:t1] = torch.sigmoid(P[t0:t1, b_off:b_off + H].float())
    decay[t0:t1] = torch.exp(-torch.exp(A_log.float()) * F.softplus(P[t0:t1, a_off:a_off + H].float() + dt_bias.float()))


def gla_prep(P, a1_off, a2, a2_b, tau, decay):
  z = P[:, a1_off:a1_off + a2.shape[1]].float() @ a2.float().t() + a2_b.float()
  decay.copy_(torch.exp(F.logsigmoid(z) / tau))


def linear_recurrence(q, k, v, decay, beta, q_scale, state, state_slots, cu_q, out):
  _, H, dv, d = state.shape  # stored transposed: S^T [dv, d] per head
  G = q.shape[1] // d
  rep = H // G
  if decay.dim() == 1 and decay.numel() == H and beta is None:  # one fixed decay per head
    decay = decay.reshape(1, H).expand(q.shape[0], H)
  norm_ch = v.shape[1] == H * (dv - 1)  # the state's last value channel is a normaliser fed with ones; beta: input scale
  if norm_ch:
    dv -= 1
  for b in range(state_slots.numel()):
    t0, t1, slot = int(cu_q[b]), int(cu_q[b + 1]), int(state_slots[b])
    if slot < 0 or t1 == t0:
      continue
    S = state[slot].transpose(1, 2)  # [H, d, dv] view; updates land in the slot
    for t in range(t0, t1):
      qt = (q[t].float() * q_scale).reshape(G, d).repeat_interleave(rep, 0)
      kt = k[t].float().reshape(G, d).repeat_interleave(rep, 0)
      vt = v[t].float().reshape(H, dv)
      if norm_ch:
        vt = torch.cat([vt, torch.ones(H, 1)], 1) * beta[t].reshape(H, 1)
        S *= decay[t].reshape(H, 1, 1)
        S += kt[:, :, None] * vt[:, None, :]
      elif beta is not None:
        S *= decay[t].reshape(H, 1, 1)
        u = beta[t].reshape(H, 1) * (vt - torch.einsum("hdv,hd->hv", S, kt))
        S += kt[:, :, None] * u[:, None, :]
      elif decay.numel() == decay.shape[0] * H:  # one decay per head
        S *= decay[t].reshape(H, 1, 1)
        S += kt[:, :, None] * vt[:, None, :]
      else:
        S *= decay[t].reshape(H, d, 1)
        S += kt[:, :, None] * vt[:, None, :]
      out[t] = torch.einsum("hdv,hd->hv", S, qt).reshape(-1)


def gated_rmsnorm(o, w, P, g_off, eps, out_scale, out):
  T = P.shape[0]
  dv = w.numel()
  x = o.reshape(T, -1, dv).float()
  gate = P[:, g_off:g_off + x.shape[1] * dv].float().reshape(T, -1, dv)
  y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float() * F.silu(gate) * out_scale
  out.copy_(y.reshape(T, -1).to(out.dtype))


# ------------------------------------------------------------------ post-norm blocks: window attention, SSD, feed-forwards
# Torch twins of csrc/hybrid.hip.
def gated_postnorm(x, y, P, g_off, gate_b, alpha, w, eps, out):
  """x <- (alpha x + y * sigmoid(P[:, g_off : +D] + gate_b)) / rms * w in place (P None: no gate); out[:, :D] = x."""
  D = x.shape[1]
  s = alpha * x
  if y is not None:
    yy = y[:, :D].float()
    if P is not None:
      yy = yy * torch.sigmoid(P[:, g_off:g_off + D].float() + gate_b.float())
    s = s + yy
  x.copy_(s / torch.sqrt(s.pow(2).mean(-1, keepdim=True) + eps) * w.float())
  if out is not None:
    out[:, :D] = x.to(out.dtype)


def pool_dims(pool: int) -> int:
  """Pooled entries per 64-token page: the most blocks of `pool` tokens whose last token lies in one page."""
  return -(-PAGE // pool)


def qk_norm_rope_store(P, bias, q_off, k_off, v_off, H, G, d, dv, R, pos, cos_sin, slots, eps, qk_norm, q_out, k_cache,
                       v_cache):
  T = P.shape[0]
  Gv = v_cache.shape[1] if k_off >= 0 else G  # value heads (fewer than key heads when key heads share values)
  Pb = P.float() if bias is None else P.float() + bias.float()
  half = R // 2

  def prep(x):
    if R:
      cs = cos_sin[pos.long()]
      c, s = cs[:, None, :half], cs[:, None, half:]
      a, b = x[..., :half], x[..., half:R]
      x = torch.cat([a * c - b * s, b * c + a * s, x[..., R:]], -1)
    if qk_norm:
      x = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return x
  q_out.copy_(prep(Pb[:, q_off:q_off + H * d].reshape(T, H, d)).to(q_out.dtype))
  if k_off < 0:
    return
  ok = slots >= 0
  s = slots[ok].long()
  k_cache[s // PAGE, :, s % PAGE] = prep(Pb[:, k_off:k_off + G * d].reshape(T, G, d))[ok].to(k_cache.dtype)
  v_cache[s // PAGE, :, :, s % PAGE] = Pb[:, v_off:v_off + Gv * dv].reshape(T, Gv, dv)[ok].to(v_cache.dtype)


def _pool_slot(blk: int, pool: int):
  """Pooled block blk lives with the page that holds its last token: (page index in the sequence, entry)."""
  pg = (blk * pool + pool - 1) // PAGE
  return pg, blk - (pg * PAGE) // pool


def kv_pool_update(k_cache, v_cache, kp, vp, block_tables, cu_q, ctx_lens, pool, max_qlen=0):
  """Mean key / value of every block of `pool` tokens whose last token arrived in this step -> the pooled caches
  kp [pages, G, per, d], vp [pages, G, per, dv]."""
  for b in range(ctx_lens.numel()):
    n, q = int(ctx_lens[b]), int(cu_q[b + 1]) - int(cu_q[b])
    if n <= 0 or q <= 0:
      continue
    for blk in range((n - q) // pool, (n - pool) // pool + 1):
      toks = torch.arange(blk * pool, blk * pool + pool)
      pages = block_tables[b, toks // PAGE].long()
      pg, e = _pool_slot(blk, pool)
      dst = int(block_tables[b, pg])
      kp[dst, :, e] = k_cache[pages, :, toks % PAGE].float().mean(0).to(kp.dtype)
      vp[dst, :, e] = v_cache[pages, :, :, toks % PAGE].float().mean(0).to(vp.dtype)


def attn_window_pool(q, k_cache, v_cache, kp, vp, block_tables, cu_q, ctx_lens, sink, scale, window, pool, out, max_qlen=0):
  T, H, d = q.shape
  G, dv = k_cache.shape[1], v_cache.shape[2]
  rep = H // G
  for b in range(ctx_lens.numel()):
    t0, t1, n = int(cu_q[b]), int(cu_q[b + 1]), int(ctx_lens[b])
    if n <= 0 or t1 == t0:
      continue
    npg = -(-n // PAGE)
    pages = block_tables[b, :npg].long()
    k = k_cache[pages].permute(0, 2, 1, 3).reshape(npg * PAGE, G, d)[:n].float()
    Gv = v_cache.shape[1]  # (key heads that share a value head: G / Gv neighbours)
    v = v_cache[pages].permute(0, 3, 1, 2).reshape(npg * PAGE, Gv, dv)[:n].float().repeat_interleave(G // Gv, 1)
    nb = n // pool if (pool and window) else 0
    if nb:
      loc = [_pool_slot(j, pool) for j in range(nb)]
      pk = torch.stack([kp[int(block_tables[b, pg]), :, e].float() for pg, e in loc])  # [nb, G, d]
      pv = torch.stack([vp[int(block_tables[b, pg]), :, e].float() for pg, e in loc])
      k, v = torch.cat([k, pk]), torch.cat([v, pv])
    qpos = torch.arange(n - (t1 - t0), n)[:, None]
    kpos = torch.arange(n)[None, :]
    vis = kpos <= qpos
    if window:
      vis = vis & (qpos - kpos < window)
    if nb:
      last = torch.arange(nb)[None, :] * pool + pool - 1
      vis = torch.cat([vis, last <= qpos - window], 1)
    s = torch.einsum("shd,thd->hst", q[t0:t1].float(), k.repeat_interleave(rep, 1)) * scale
    s = s.masked_fill(~vis[None], float("-inf"))
    if sink is not None:
      s = torch.cat([s, sink.float()[:, None, None].expand(H, t1 - t0, 1)], -1)
    w = torch.softmax(s, -1)[..., :k.shape[0]]
    o = torch.einsum("hst,thd->shd", w, v.repeat_interleave(rep, 1))
    out[t0:t1] = o.reshape(t1 - t0, H * dv).to(out.dtype)


def ssd_prep(P, x_off, dt_off, conv_w, conv_b, conv_state, state_slots, cu_q, A_log, dt_bias, H, dv, xbc, v, decay):
  C, taps = conv_w.shape
  for b in range(state_slots.numel()):
    t0, t1, slot = int(cu_q[b]), int(cu_q[b + 1]), int(state_slots[b])
    if slot < 0 or t1 == t0:
      continue
    x = torch.cat([conv_state[slot], P[t0:t1, x_off:x_off + C].float()], 0)
    y = F.silu(sum(conv_w[:, j].float() * x[j:j + t1 - t0] for j in range(taps)) + conv_b.float())
    xbc[t0:t1] = y
    if taps > 1:
      conv_state[slot] = x[x.shape[0] - (taps - 1):]
    dt = F.softplus(P[t0:t1, dt_off:dt_off + H].float() + dt_bias.float())
    decay[t0:t1] = torch.exp(-torch.exp(A_log.float()) * dt)
    v[t0:t1] = (y[:, :H * dv].reshape(-1, H, dv) * dt[:, :, None]).reshape(-1, H * dv)


def ssd_gate_norm(o, xbc, skip_d, P, z_off, w, groups, eps, out):
  T, inner = o.shape
  H = skip_d.numel()
  y = o.float() + (xbc[:, :inner].float().reshape(T, H, -1) * skip_d.float()[None, :, None]).reshape(T, inner)
  y = (y * F.silu(P[:, z_off:z_off + inner].float())).reshape(T, groups, -1)
  y = y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps)
  out[:, :inner] = (y.reshape(T, inner) * w.float()).to(out.dtype)


def polynorm_act(P, up_off, Fd, coef, eps, out):
  z = P[:, up_off:up_off + Fd].float()
  a, b, c, e = coef.float().tolist()

  def nrm(t):
    return t / torch.sqrt(t.pow(2).mean(-1, keepdim=True) + eps)
  out[:, :Fd] = (a * nrm(z) + b * nrm(z * z) + c * nrm(z * z * z) + e).to(out.dtype)


def relu2(P, off, Fd, out):
  out[:, :Fd] = torch.relu(P[:, off:off + Fd].float()).pow(2).to(out.dtype)


def moe_weighted_sum(y, slot_of, topw, k, sh_y, P, shg_off, out, splits=1):
  """out [T, D] = sum_j topw[t, j] y[slot_of[t, j]] (+ sigmoid(P[t, shg_off]) sh_y[t]); y [splits * T k, >= D] holds
  the down projection's K slices, summed first."""
  T, D = out.shape
  y = y.reshape(splits, T * k, -1).float().sum(0)
  acc = (y[slot_of.long().reshape(T, k), :D] * topw.reshape(T, k, 1)).sum(1)
  if sh_y is not None:
    sh = sh_y[:, :D].float()
    acc = acc + (sh if P is None else torch.sigmoid(P[:, shg_off:shg_off + 1].float()) * sh)
  out.copy_(acc)


# ------------------------------------------------------------------ sandwich blocks: latent attention, gated feed-forwards
# Torch twins of csrc/latent.hip.
def sandwich_add_norm(x, y, wb, wn, eps, out, bb=None, bn=None, mult=1.0):
  """x += mult * norm(y) in place (y None: nothing is added); with wn, out[:, :D] = norm(x).  norm(v) = v / rms(v) * w,
  or with a bias (bb / bn) the layer norm (v - mean) / sqrt(var + eps) * w + b."""
  D = x.shape[1]

  def norm(v, w, b):
    if b is None:
      return v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    c = v - v.mean(-1, keepdim=True)
    return c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w.float() + b.float()
  if y is not None:
    x += mult * norm(y[:, :D].float(), wb, bb)
  if wn is not None:
    out[:, :D] = norm(x, wn, bn).to(out.dtype)


def _rope_pairs(x, cs, R, interleaved):
  """x [T, heads, d]: the first R dims rotated by the table rows cs [T, R] = (cos | sin); partner of dim 2i is 2i + 1
  (interleaved) or of dim i is i + R / 2."""
  if not R:
    return x
  half = R // 2
  c, s = cs[:, None, :half], cs[:, None, half:]
  x = x.clone()
  if interleaved:
    a, b = x[..., 0:R:2].clone(), x[..., 1:R:2].clone()
    x[..., 0:R:2], x[..., 1:R:2] = a * c - b * s, b * c + a * s
  else:
    a, b = x[..., :half].clone(), x[..., half:R].clone()
    x[..., :half], x[..., half:R] = a * c - b * s, b * c + a * s
  return x


def latent_kv_store(P, ckv_off, R, dr, kv_norm, q_off, q_rank, q_norm, eps, rot_dims, interleaved, pos, cos_sin, slots,
                    cache, qa_out):
  T = P.shape[0]
  c = P[:, ckv_off:ckv_off + R].float()
  c = c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * kv_norm.float()
  kr = P[:, ckv_off + R:ckv_off + R + dr].float().reshape(T, 1, dr)
  kr = _rope_pairs(kr, cos_sin[pos.long()] if rot_dims else None, rot_dims, interleaved).reshape(T, dr)
  ok = slots >= 0
  s = slots[ok].long()
  cache[s // PAGE, 0, s % PAGE] = torch.cat([c, kr], 1)[ok].to(cache.dtype)
  if q_rank:
    q = P[:, q_off:q_off + q_rank].float()
    qa_out[:, :q_rank] = (q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm.float()).to(qa_out.dtype)


def latent_q_rope(Q, q_off, H, dn, dr, rot_dims, interleaved, pos, cos_sin, qn_out, qpe_out):
  T = Q.shape[0]
  q = Q[:, q_off:q_off + H * (dn + dr)].float().reshape(T, H, dn + dr)
  qn_out.copy_(q[..., :dn].transpose(0, 1).to(qn_out.dtype))
  qpe_out.copy_(_rope_pairs(q[..., dn:], cos_sin[pos.long()] if rot_dims else None, rot_dims, interleaved).to(qpe_out.dtype))


def latent_attn(q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, sink, scale, window, out, max_qlen=0):
  H, T, R = q_lat.shape
  for b in range(ctx_lens.numel()):
    t0, t1, n = int(cu_q[b]), int(cu_q[b + 1]), int(ctx_lens[b])
    if n <= 0 or t1 == t0:
      continue
    npg = -(-n // PAGE)
    rows = cache[block_tables[b, :npg].long(), 0].reshape(npg * PAGE, -1)[:n].float()
    qpos = torch.arange(n - (t1 - t0), n)[:, None]
    kpos = torch.arange(n)[None, :]
    vis = kpos <= qpos
    if window:
      vis = vis & (qpos - kpos < window)
    s = (torch.einsum("htr,jr->htj", q_lat[:, t0:t1].float(), rows[:, :R]) +
         torch.einsum("thr,jr->htj", q_pe[t0:t1].float(), rows[:, R:])) * scale
    s = s.masked_fill(~vis[None], float("-inf"))
    if sink is not None:
      s = torch.cat([s, sink.float()[:, None, None].expand(H, t1 - t0, 1)], -1)
    w = torch.softmax(s, -1)[..., :n]
    out[:, t0:t1] = torch.einsum("htj,jr->htr", w, rows[:, :R]).to(out.dtype)


def latent_out_gate(o, P, g_off, gate, out):
  """o [H, T, dv] -> out[:, :H dv] token-major, times sigmoid of P's gate columns: gate 1 one per element, 2 one per head."""
  H, T, dv = o.shape
  y = o.float().transpose(0, 1)
  if gate == 1:
    y = y * torch.sigmoid(P[:, g_off:g_off + H * dv].float()).reshape(T, H, dv)
  elif gate == 2:
    y = y * torch.sigmoid(P[:, g_off:g_off + H].float()).reshape(T, H, 1)
  out[:, :H * dv] = y.reshape(T, H * dv).to(out.dtype)


def glu_act(P, gate_off, up_off, Fd, clamped, limit, out):
  g, u = P[:, gate_off:gate_off + Fd].float(), P[:, up_off:up_off + Fd].float()
  if clamped:
    g, u = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1)
  else:
    y = F.silu(g) * u
  out[:, :Fd] = y.to(out.dtype)


# ------------------------------------------------------------------ layer-norm sandwich blocks: differential attention, mlstm, lightning
# Torch twins of csrc/recurrent_gates.hip.
def diff_attn_out(a, P, g_off, H, G, lam, post, eps, out):
  """a [T, 2 H dv]: the two maps' attention outputs, heads ordered (kv head, map, head of the group) -> out[:, :H dv] =
  rms_norm(a_1 - lam a_2) * post * sigmoid(P[:, g_off + head]), heads in their own order."""
  T = a.shape[0]
  rep = H // G
  x = a.float().reshape(T, G, 2, rep, -1)
  o = (x[:, :, 0] - lam * x[:, :, 1]).reshape(T, H, -1)
  o = o / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps) * post
  o = o * torch.sigmoid(P[:, g_off:g_off + H].float())[:, :, None]
  out[:, :o.shape[1] * o.shape[2]] = o.reshape(T, -1).to(out.dtype)


def sigmoid_gate_mul(a, P, g_off, out):
  """out[:, :n] = a * sigmoid(P[:, g_off : +n]), n = a's row."""
  n = a.shape[1]  # (a may be out's own rows)
  out[:, :n] = (a.float() * torch.sigmoid(P[:, g_off:g_off + n].float())).to(out.dtype)


def silu_cols(P, off, n, out):
  """out [T, n] fp32 = silu(P[:, off : +n])."""
  out.copy_(F.silu(P[:, off:off + n].float()))


def mlstm_gates(P, i_off, f_off, gate_b, cap, mstate, state_slots, cu_q, decay, inscale, mout):
  """Per head and token: i = cap tanh((P[i_off + h] + b_i) / cap), f = logsigmoid(cap tanh((P[f_off + h] + b_f) / cap)),
  m_t = max(f + m_(t-1), i) from the slot's running maximum mstate [slots, H] (updated); decay = e^(f + m_(t-1) - m_t),
  inscale = e^(i - m_t), mout = m_t, each [T, H]."""
  H = mstate.shape[1]
  gi = cap * torch.tanh((P[:, i_off:i_off + H].float() + gate_b[:H].float()) / cap)
  gf = F.logsigmoid(cap * torch.tanh((P[:, f_off:f_off + H].float() + gate_b[H:].float()) / cap))
  for b in range(state_slots.numel()):
    t0, t1, slot = int(cu_q[b]), int(cu_q[b + 1]), int(state_slots[b])
    if slot < 0 or t1 == t0:
      continue
    m = mstate[slot].clone()
    for t in range(t0, t1):
      new = torch.maximum(gf[t] + m, gi[t])
      decay[t], inscale[t], mout[t] = torch.exp(gf[t] + m - new), torch.exp(gi[t] - new), new
      m = new
    mstate[slot] = m


def gated_group_norm(o, m, w, P, g_off, groups, eps, out):
  """o [T, groups * gs] (m None) or [T, groups * (gs + 1)] with m [T, groups]: each group's last channel is then a
  normaliser n and its values are divided by max(|n|, e^(-m)) + 1e-6 first.  out[:, :groups gs] = the values divided by
  their group's RMS, times w [groups gs], times sigmoid(P[:, g_off : +groups gs])."""
  T = o.shape[0]
  x = o.float().reshape(T, groups, -1)
  if m is not None:
    den = torch.maximum(x[..., -1].abs(), torch.exp(-m.float())) + 1e-6
    x = x[..., :-1] / den[..., None]
  x = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
  n = x.shape[1] * x.shape[2]
  out[:, :n] = (x.reshape(T, n) * w.float() * torch.sigmoid(P[:, g_off:g_off + n].float())).to(out.dtype)


def pair_norm_mean(y1, y2, w, eps, out):
  """out [T, D] fp32 = (y1 / rms(y1) * w[0] + y2 / rms(y2) * w[1]) / 2 (y rows may be wider than D)."""
  D = out.shape[1]
  a, b = y1[:, :D].float(), y2[:, :D].float()
  out.copy_(0.5 * (a / torch.sqrt(a.pow(2).mean(-1, keepdim=True) + eps) * w[0].float() +
                   b / torch.sqrt(b.pow(2).mean(-1, keepdim=True) + eps) * w[1].float()))
