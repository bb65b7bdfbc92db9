"""Python entry points of the gfx950 kernel library.

Each function takes torch tensors, allocates outputs when the caller did not preallocate them, and
dispatches to the HIP kernel for GPU tensors or to the fp32 torch reference (`ops.reference`) for
CPU tensors.  GPU tensors never take the reference path: if the extension is missing the call
raises (see `ops._ext.require`).
"""
from __future__ import annotations

import os

import torch

from . import reference as ref
from ._ext import require

EPI = {"none": 0, "resid": 1, "silu": 2}
PAGE = 64


def _gpu(t: torch.Tensor) -> bool:
  if t.is_cuda:
    require()
    return True
  return False


# ------------------------------------------------------------------ norms / elementwise
def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, residual: torch.Tensor | None = None,
            out: torch.Tensor | None = None, residual_out: torch.Tensor | None = None):
  """Returns (out, residual_out).  With `residual`, residual_out = x + residual (the new stream)."""
  if not _gpu(x):
    y, r = ref.rmsnorm(x, w, eps, residual)
    if out is not None:
      out.copy_(y)
      y = out
    if residual_out is not None and r is not None:
      residual_out.copy_(r)
      r = residual_out
    return y, r
  out = torch.empty_like(x) if out is None else out
  if residual is not None and residual_out is None:
    residual_out = torch.empty_like(x)
  require().rmsnorm(x, w, out, residual, residual_out, float(eps))
  return out, residual_out


def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
  if not _gpu(table):
    y = table[ids.long().clamp(0, table.shape[0] - 1)]
    if out is not None:
      out.copy_(y.reshape(out.shape))
      return out
    return y
  ids32 = ids.to(torch.int32).contiguous()
  out = torch.empty(ids32.numel(), table.shape[1], dtype=table.dtype, device=table.device) if out is None else out
  require().embedding(ids32, table, out)
  return out


def silu_mul(gu: torch.Tensor, out: torch.Tensor | None = None, interleaved16: bool = False) -> torch.Tensor:
  """silu(gate) * up.  gu = [gate | up] halves, or 16-column interleaved tiles (fused gate_up layout)."""
  if not _gpu(gu):
    if interleaved16:
      M, N = gu.shape
      g = gu.view(M, N // 32, 2, 16)
      y = (torch.nn.functional.silu(g[:, :, 0].float()) * g[:, :, 1].float()).reshape(M, N // 2).to(gu.dtype)
    else:
      y = ref.silu_mul(gu)
    if out is not None:
      out.copy_(y)
      return out
    return y
  Fd = gu.shape[-1] // 2
  out = torch.empty(*gu.shape[:-1], Fd, dtype=gu.dtype, device=gu.device) if out is None else out
  require().silu_mul(gu.contiguous(), out, bool(interleaved16))
  return out


# ------------------------------------------------------------------ GEMM
def gemm(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None, residual: torch.Tensor | None = None,
         epi: str = "none", out: torch.Tensor | None = None, out_dtype: torch.dtype | None = None, algo: int = 0,
         nt: int = 0) -> torch.Tensor:
  """y = x @ w.T (+bias) with fused epilogue: 'none' | 'resid' (y += residual) | 'silu'.

  For 'silu' the weight rows must be gate/up interleaved in 16-row tiles (see
  models.weights.interleave_gate_up); the output has w.shape[0] // 2 columns.
  """
  M, N = x.shape[0], w.shape[0]
  ncol = N // 2 if epi == "silu" else N
  if not _gpu(x):
    y = ref.linear(x, w, bias)
    if epi == "silu":
      y = y.view(M, N // 32, 2, 16)
      y = (torch.nn.functional.silu(y[:, :, 0]) * y[:, :, 1]).reshape(M, ncol)
    elif epi == "resid":
      y = y + residual.float()
    dt = out_dtype or (out.dtype if out is not None else x.dtype)
    if out is not None:
      out.copy_(y.to(out.dtype))
      return out
    return y.to(dt)
  if out is None:
    out = torch.empty(M, ncol, dtype=out_dtype or x.dtype, device=x.device)
  if nt == 0:
    nt = 2 if (N // 32) >= 1024 else 1
  if algo == 0 and epi != "silu" and N % 16:  # the skinny kernel tiles 16 output columns; the tiled one masks
    algo = 2
  require().gemm(x, w, out, bias, residual, EPI[epi], int(algo), int(nt))
  return out


# ------------------------------------------------------------------ RoPE + paged KV
def rope_kv_write(qkv: torch.Tensor, pos: torch.Tensor, cos_sin: torch.Tensor, slots: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, H: int, Hkv: int,
                  q_out: torch.Tensor | None = None) -> torch.Tensor:
  """qkv [T, (H+2Hkv)*Dh] -> rotated q [T, H, Dh]; rotated k and v written into the paged caches."""
  T = qkv.shape[0]
  Dh = k_cache.shape[-1]
  if not _gpu(qkv):
    x = qkv.view(T, H + 2 * Hkv, Dh)
    q = ref.rope(x[:, :H], pos, cos_sin)
    k = ref.rope(x[:, H:H + Hkv], pos, cos_sin)
    ref.write_kv(k, x[:, H + Hkv:], slots, k_cache, v_cache)
    if q_out is not None:
      q_out.copy_(q.view(q_out.shape))
      return q_out
    return q
  q_out = torch.empty(T, H, Dh, dtype=qkv.dtype, device=qkv.device) if q_out is None else q_out
  require().rope_kv_write(qkv, pos, cos_sin, slots, q_out, k_cache, v_cache, int(H), int(Hkv))
  return q_out


def rope_apply(x: torch.Tensor, pos: torch.Tensor, cos_sin: torch.Tensor, nh: int, Dh: int, inverse: bool = False,
               out: torch.Tensor | None = None) -> torch.Tensor:
  """x [T, >= nh*Dh] (2-D rows) -> rotated copy (or into `out`)."""
  if not _gpu(x):
    y = ref.rope(x[:, :nh * Dh].reshape(-1, nh, Dh), pos, cos_sin, inverse).reshape(x.shape[0], nh * Dh)
    if out is not None:
      out[:, :nh * Dh].copy_(y)
      return out
    return y
  out = torch.empty(x.shape[0], nh * Dh, dtype=x.dtype, device=x.device) if out is None else out
  require().rope_apply(x, out, pos, cos_sin, int(nh), int(Dh), bool(inverse))
  return out


# ------------------------------------------------------------------ attention
# 0: workgroup per (sequence, KV head, partition), waves split pages + LDS combine
# 1 / 2: wave per (sequence, KV head, partition), transposed S^T (lane = query head), no LDS;
#        2 prefetches the next page under the current one
# 3: 2 with non-temporal K / V loads (neutral in round 3, profiles/r3/s3/; on the chunk-major V cache of round 6
#        the KV stream runs 5-13 % faster in isolation -- B 512: 183.9 vs 193.7 us per layer, B 256 / ctx 1040:
#        166.6 vs 185.1, B 128 / ctx 2048: 156.2 vs 177.3 -- and the 70B headline step 74.6-74.7 vs 75.4-75.7 ms,
#        profiles/r6/headline/attn_nt/)
# -1 (default): 0 below 64 (sequence, KV head) pairs -- few long sequences, where the workgroup
#        kernel's 4-wave page split needs fewer partitions; else 3 once a layer's K / V pages (batch x block-table
#        width) outgrow the 256 MB last-level cache, 2 below (B 16 / ctx 530: 15.1 vs 13.5 us, B 64 / ctx 530: 29.3 vs
#        24.8 with nt; B 16 / ctx 8192: 85.7 vs 97.1, B 64 / ctx 2048: 85.1 vs 97.2; tools/bench_attn_small.py,
#        profiles/r6/headline/attn_nt/attn_small.log)
# (4, an 8-wave workgroup over one partition for short tables at small batch, measured 1 % slower at 8B batch 1 --
#  3.55 vs 3.52 ms, profiles/r3/s3/ -- and was removed in round 6)
DECODE_ALGO = int(os.environ.get("XOT_ATTN_DECODE", "-1"))


NT_MIN_KV_BYTES = 256 << 20  # K / V bytes per layer from which the page loads go non-temporal (algo 3)


def resolve_decode_algo(batch: int, Hkv: int, algo: int | None = None, kv_bytes: int | None = None) -> int:
  algo = DECODE_ALGO if algo is None else algo
  if algo < 0:
    if batch * Hkv < 64:
      return 0
    return 3 if kv_bytes is None or kv_bytes >= NT_MIN_KV_BYTES else 2
  return algo


def choose_pages_per_part(batch: int, Hkv: int, max_ctx: int, algo: int | None = None) -> int:
  """KV pages per split-KV partition for a decode step of `batch` sequences."""
  algo = resolve_decode_algo(batch, Hkv, algo)
  pages = max(1, -(-max_ctx // PAGE))
  if algo == 0:  # enough workgroups to cover 256 CUs several times, >= 4 pages (one per wave) each
    for ppp in (16, 8, 4):
      if batch * Hkv * -(-pages // ppp) >= 1024:
        return ppp
    return 4
  # one wave per unit: ~1024 waves (4 per CU), partitions of 2..32 pages (tools/bench_attn_small.py,
  # profiles/bench_attn_small_r1.json: 2048 waves of shorter partitions lose to the extra merge work)
  nparts = max(1, min(max(pages // 2, 1), -(-1024 // max(batch * Hkv, 1))))
  nparts = max(nparts, -(-pages // 32))
  return -(-pages // nparts)


class DecodeWorkspace:
  """Split-KV scratch for attn_decode, sized for every batch up to max_batch at this context bound.
  The partitioning is chosen per call from the actual batch (static per captured graph)."""

  def __init__(self, max_batch: int, H: int, Dh: int, max_ctx: int, device, pages_per_part: int | None = None,
               algo: int | None = None):
    self.algo = DECODE_ALGO if algo is None else algo
    self.max_ctx = max_ctx
    self.Hkv_hint = None
    self.Dh = Dh
    self.fixed_ppp = pages_per_part
    pages = max(1, -(-max_ctx // PAGE))
    worst = 1
    for b in range(1, max_batch + 1):
      for hkv in (1, 2, 4, 8, 16):
        ppp = pages_per_part or choose_pages_per_part(b, hkv, max_ctx, self.algo)
        worst = max(worst, b * -(-pages // ppp))
    self.units = worst  # max over batch of batch * nparts
    self.o = torch.empty(worst * H * Dh, dtype=torch.float32, device=device)
    self.ml = torch.empty(worst * H * 2, dtype=torch.float32, device=device)

  def partition(self, batch: int, Hkv: int, width_pages: int):
    """(pages per partition, partitions, kernel) for this call."""
    algo = resolve_decode_algo(batch, Hkv, self.algo, kv_bytes=batch * Hkv * width_pages * PAGE * self.Dh * 4)
    ppp = self.fixed_ppp or choose_pages_per_part(batch, Hkv, width_pages * PAGE, algo)
    nparts = max(1, -(-width_pages // ppp))
    if batch * nparts > self.units:
      raise RuntimeError(f"decode workspace sized for {self.units} units, need {batch * nparts}")
    return ppp, nparts, algo


class PendingMerge:
  """A batch-1 split-KV decode attention whose partition merge was left to its consumer: o_proj merges the
  partitions of its K slice in its GEMM prologue (linear_resid_norm -> gemm_stream_merge), one launch less per
  layer.  materialize() runs the merge kernel into `out` instead."""

  __slots__ = ("o", "ml", "ctx_lens", "ppp", "nparts", "out")

  def __init__(self, o, ml, ctx_lens, ppp, nparts, out):
    self.o, self.ml, self.ctx_lens, self.ppp, self.nparts, self.out = o, ml, ctx_lens, ppp, nparts, out

  def materialize(self) -> torch.Tensor:
    require().attn_decode_merge(self.o, self.ml, self.ctx_lens, self.out, self.ppp, self.nparts)
    return self.out


def attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale: float, ws: DecodeWorkspace | None = None,
                out: torch.Tensor | None = None, defer_merge: bool = False):
  """defer_merge (one sequence): return a PendingMerge when the context is split over partitions."""
  if not _gpu(q):
    y = ref.attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale)
    if out is not None:
      out.copy_(y.view(out.shape))
      return out
    return y
  B, H, Dh = q.shape
  width = block_tables.shape[1]
  if ws is None:
    ws = DecodeWorkspace(B, H, Dh, width * PAGE, q.device)
  ppp, nparts, algo = ws.partition(B, k_cache.shape[1], width)
  out = torch.empty_like(q) if out is None else out
  defer = defer_merge and B == 1 and nparts > 1
  require().attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, out, ws.o, ws.ml, ppp, nparts, float(scale),
                        algo, not defer)
  return PendingMerge(ws.o, ws.ml, ctx_lens, ppp, nparts, out) if defer else out


# XOT_PREFILL_ATTN: 2 = 256-row workgroups, LDS-DMA page ring, in-register softmax (default); 1 = the
# first 64-row kernel (register-staged pages, P through LDS)
PREFILL_ALGO = int(os.environ.get("XOT_PREFILL_ATTN", "2"))


def attn_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, max_qlen: int, scale: float,
                 out: torch.Tensor | None = None) -> torch.Tensor:
  if not _gpu(q):
    y = ref.attn_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, scale)
    if out is not None:
      out.copy_(y)
      return out
    return y
  out = torch.empty_like(q) if out is None else out
  require().attn_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, out, int(max_qlen), float(scale),
                         PREFILL_ALGO)
  return out


# ------------------------------------------------------------------ sampling
def attention_bidir(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, B: int, L: int, H: int, Dh: int,
                    scale: float) -> torch.Tensor:
  """Bidirectional (unmasked) multi-head attention over B sequences of L tokens: q / k / v [B*L, H*Dh] token-major
  (row views with unit inner stride) -> o [B*L, H*Dh].  GPU: the flash-style forward of the training kernels with
  the causal mask off (csrc/attention_train.hip; V transposed per head first) for Dh 64 / 128; CPU and other
  head sizes (the tiny test towers): fp32 reference."""
  if not _gpu(q) or Dh not in (64, 128):
    qh, kh, vh = (t.float().reshape(B, L, H, Dh).transpose(1, 2) for t in (q, k, v))
    a = torch.softmax((qh @ kh.transpose(-1, -2)) * scale, -1) @ vh
    return a.transpose(1, 2).reshape(B * L, H * Dh).to(q.dtype)
  C = require()
  Lp = -(-L // 64) * 64
  vt = torch.empty(B, H, Dh, Lp, dtype=v.dtype, device=v.device)
  C.attn_train_transpose(v, vt, B, L, Lp, H, Dh)
  o = torch.empty(B * L, H * Dh, dtype=q.dtype, device=q.device)
  lse2 = torch.empty(B * H * L, dtype=torch.float32, device=q.device)
  C.attn_train_fwd(q, k, vt, o, lse2, B, L, Lp, H, H, Dh, float(scale), False)
  return o


def sample(logits: torch.Tensor, temps: torch.Tensor, top_k: int, seed_off: torch.Tensor,
           out: torch.Tensor | None = None) -> torch.Tensor:
  """Greedy when temp <= 1e-5, else top-k + exponential-race sampling (all on device)."""
  if not _gpu(logits):
    B = logits.shape[0]
    res = torch.empty(B, dtype=torch.int32)
    g = torch.Generator().manual_seed(int(seed_off[0]) * 1000003 + int(seed_off[1]))
    for b in range(B):
      t = float(temps[b])
      row = logits[b].float()
      if t <= 1e-5 or top_k == 1:
        res[b] = int(row.argmax())
        continue
      row = row / max(t, 1e-5)
      if 0 < top_k < row.numel():
        kth = torch.topk(row, top_k).values[-1]
        row = row.masked_fill(row < kth, float("-inf"))
      probs = torch.softmax(row, -1)
      q = torch.empty_like(probs).exponential_(1, generator=g)
      res[b] = int((probs / q).argmax())
    if out is not None:
      out.copy_(res)
      return out
    return res
  out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device) if out is None else out
  require().sample(logits, temps, int(top_k), seed_off, out)
  return out


def topk_cand(logits: torch.Tensor, top_k: int, kc: int = 64) -> tuple:
  """Each row's top_k (value, index) candidates in [B, kc] buffers (unused slots -inf / -1): one vocab
  slice's contribution to a sampler that runs on another stage."""
  B = logits.shape[0]
  if not _gpu(logits):
    v, i = torch.topk(logits.float(), top_k, dim=-1)
    vals = torch.full((B, kc), float("-inf"))
    idx = torch.full((B, kc), -1, dtype=torch.int32)
    vals[:, :top_k] = v
    idx[:, :top_k] = i.int()
    return vals, idx
  vals = torch.empty(B, kc, dtype=torch.float32, device=logits.device)
  idx = torch.empty(B, kc, dtype=torch.int32, device=logits.device)
  require().topk_cand(logits, int(top_k), vals, idx)
  return vals, idx


# ------------------------------------------------------------------ DeepSeek MLA
def mla_prep(ckv, kv_ln, q, qpe_off: int, H: int, pos, cos_sin, slots, cache, eps: float) -> None:
  """ckv [T, >= DL+DR] (rows may be strided), q [T, ldq]: latent norm + rope + cache write, q_pe rotated
  in place."""
  if not _gpu(ckv):
    ref.mla_prep(ckv, kv_ln, q, qpe_off, H, pos, cos_sin, slots, cache, eps)
    return
  require().mla_prep(ckv, kv_ln, q, int(qpe_off), int(H), pos, cos_sin, slots, cache, float(eps))


class MLAWorkspace:
  """Split-KV scratch of the MLA attention kernel."""

  def __init__(self, max_tokens: int, H: int, DL: int, max_ctx: int, device):
    self.max_tokens, self.H, self.DL = max_tokens, H, DL
    self.pages = max(1, -(-max_ctx // PAGE))
    self.max_parts = max(self.partition(1, self.pages)[1], self.partition(8, self.pages)[1])
    units = max(max_tokens * self.max_parts, 1)
    self.o = torch.empty(units * H * DL, dtype=torch.float32, device=device)
    self.ml = torch.empty(units * H * 2, dtype=torch.float32, device=device)

  def wide(self, T: int) -> bool:
    """Many-head kernel (one workgroup covers up to 128 heads, each page loaded once for all of them) for
    >= 64 heads at batch sizes that fill the chip; the narrow kernel (a workgroup per 16 heads) keeps more
    workgroups in flight for a handful of tokens.  XOT_MLA_WIDE=0/1 forces either."""
    force = os.environ.get("XOT_MLA_WIDE")
    if force in ("0", "1"):
      return force == "1"
    return self.H >= 64 and T >= 8

  def partition(self, T: int, width_pages: int):
    """(pages per partition, partitions, wide): enough workgroups for 256 CUs (one per CU: the kernels
    hold two 73 KB pages in LDS); narrow-kernel partitions of at least 2 pages."""
    nhb = -(-self.H // 16)
    wide = self.wide(T)
    units = T * -(-nhb // 8) if wide else T * nhb
    want = max(1, -(-256 // max(units, 1)))
    cap = width_pages if wide else (width_pages // 2 if width_pages >= 2 else 1)
    nparts = max(1, min(want, cap))
    ppp = -(-width_pages // nparts)
    return ppp, -(-width_pages // ppp), wide


def mla_attn(q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, scale: float, ws: MLAWorkspace | None = None,
             out: torch.Tensor | None = None) -> torch.Tensor:
  """q_lat [H, T, DL], q_pe [T, >= H*DR] (row-major, strided rows ok) -> o_lat [H, T, DL]."""
  if not _gpu(q_lat):
    y = ref.mla_attn(q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, scale)
    if out is not None:
      out.copy_(y)
      return out
    return y
  H, T, DL = q_lat.shape
  width = block_tables.shape[1]
  if ws is None:
    ws = MLAWorkspace(T, H, DL, width * PAGE, q_lat.device)
  ppp, nparts, wide = ws.partition(T, width)
  if T * nparts > ws.max_tokens * ws.max_parts:
    ppp, nparts = width, 1
  out = torch.empty_like(q_lat) if out is None else out
  require().mla_attn(q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, out, ws.o, ws.ml, int(ppp), int(nparts),
                     float(scale), int(wide))
  return out


_ROUTE_CNT = {}


def _route_counters(device) -> torch.Tensor:
  """Per-device expert counters of moe_route_ds: zero between launches (the kernel resets them)."""
  key = str(device)
  if key not in _ROUTE_CNT:
    _ROUTE_CNT[key] = torch.zeros(256, dtype=torch.int32, device=device)
  return _ROUTE_CNT[key]


def moe_route_ds(logits, bias, k: int, n_group: int, topk_group: int, method: int, sigmoid: bool, norm: bool,
                 scale: float, outs: tuple | None = None):
  """DeepSeekMoE routing.  GPU: (topw, topi, slot_of, sorted_tok, off) device tensors (graph-capturable;
  launches on one stream reuse the per-device counters in order); CPU: (topw [T, k], topi [T, k])."""
  if not _gpu(logits):
    return ref.moe_route_ds(logits, bias, k, n_group, topk_group, method, sigmoid, norm, scale)
  T, E = logits.shape
  dev = logits.device
  if outs is None:
    outs = (torch.empty(T * k, dtype=torch.float32, device=dev), torch.empty(T * k, dtype=torch.int32, device=dev),
            torch.empty(T * k, dtype=torch.int32, device=dev), torch.empty(T * k, dtype=torch.int32, device=dev),
            torch.empty(E + 1, dtype=torch.int32, device=dev))
  require().moe_route_ds(logits.contiguous(), bias, int(k), int(n_group), int(topk_group), int(method), bool(sigmoid),
                         bool(norm), float(scale), _route_counters(dev), *outs)
  return outs


# ------------------------------------------------------------------ mixers on an fp32 residual stream (csrc/mixers.hip)
# P is a fused projection's fp32 output [T, n]; *_off are column offsets into it.  Outputs are preallocated by the
# caller (graph-capturable); activation outputs may be column slices of a wider row buffer.
def _mix(name: str, on_gpu: bool):
  return getattr(require(), name) if on_gpu else getattr(ref, name)


def resid_scale_norm(x, y1=None, s1=None, y2=None, s2=None, gain=None, eps: float = 1e-5, out=None) -> None:
  """fp32 residual rows x [T, D] += s1 * y1 (+ s2 * y2) in place (per-channel scales; y rows may be wider than
  D), then, with `out`, out[:, :D] = x / sqrt(mean(x^2) + eps) * gain (gain: one fp32 number on the device)."""
  _mix("resid_scale_norm", _gpu(x))(x, y1, s1, y2, s2, gain, float(eps), out)


def gelu_mul(P, gate_off: int, up_off: int, F: int, out) -> None:
  """out[:, :F] = gelu_tanh(P[:, gate_off : +F]) * P[:, up_off : +F]  (out rows may be wider: K padding)."""
  _mix("gelu_mul", _gpu(P))(P, int(gate_off), int(up_off), int(F), out)


def rope_kv_store(P, q_off: int, k_off: int, v_off: int, H: int, G: int, d: int, R: int, pos, cos_sin, slots, q_out,
                  k_cache, v_cache) -> None:
  """Rotate-half RoPE on the first R dims of every q / k head (pairs (i, i + R/2)); q -> q_out [T, H, d], the
  rotated key -> k_cache [pages, G, 64, d], the value (v_off < 0: the key before rotation) -> v_cache [pages, G, d, 64],
  both at `slots`."""
  _mix("rope_kv_store", _gpu(P))(P, int(q_off), int(k_off), int(v_off), int(H), int(G), int(d), int(R), pos, cos_sin,
                                 slots, q_out, k_cache, v_cache)


def attn_gated_chunk(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, pb, scale: float, chunk: int, out_scale: float,
                     out, max_qlen: int = 0) -> None:
  """out [T, H d] = out_scale * sum over the keys j <= i of query i's chunk (floor(i / chunk) == floor(j / chunk))
  of sigmoid(q_i . k_j * scale + pb[head]) v_j; positions count from each sequence's start.  Caches: K [pages, G, 64,
  d], V [pages, G, d, 64].  max_qlen: the step's longest run of new tokens of one sequence (0: unknown -> the total);
  bf16 steps with runs above one token take the MFMA kernel; single tokens, fp32 and head sizes that are no
  multiple of 32 a (token, kv head, key split) kernel that scores each key once for all query heads of its group."""
  _mix("attn_gated_chunk", _gpu(q))(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, pb, float(scale), int(chunk),
                                    float(out_scale), out, int(max_qlen) or int(q.shape[0]))


def delta_prep(P, x_off: int, b_off: int, a_off: int, conv_w, conv_state, state_slots, cu_q, A_log, dt_bias, H: int,
               G: int, d: int, dv: int, qkv, beta, decay) -> None:
  """Delta-rule inputs of a step and the convolution state's update (see csrc/mixers.hip delta_prep)."""
  _mix("delta_prep", _gpu(P))(P, int(x_off), int(b_off), int(a_off), conv_w, conv_state, state_slots, cu_q, A_log, dt_bias,
                              int(H), int(G), int(d), int(dv), qkv, beta, decay)


def gla_prep(P, a1_off: int, a2, a2_b, tau: float, decay) -> None:
  """decay [T, H d] = sigmoid(z)^(1/tau), z = a2 P[:, a1_off : +rank] + a2_b."""
  _mix("gla_prep", _gpu(P))(P, int(a1_off), a2, a2_b, float(tau), decay)


def linear_recurrence(q, k, v, decay, beta, q_scale: float, state, state_slots, cu_q, out) -> None:
  """Per sequence and value head, token by token on the fp32 state, stored S^T [slots, H, dv, d] (updated in place):
  beta given (delta rule, decay [T, H]):  S *= g; u = beta (v - S^T k); S += k u^T; o = S^T q
  else (decay [T, H d] per key channel, [T, H] per head, or a 1-D [H]: fixed per head):  S = diag(a) S + k v^T; o = S^T q.
  q is scaled by q_scale.
  A state with one value channel more than v has (decay [T, H], beta [T, H] an input scale): S = g S + k (beta [v | 1])^T,
  the last channel being a normaliser n = g n + beta k; out [T, H (dv + 1)] then ends each head with n . q."""
  _mix("linear_recurrence", _gpu(q))(q, k, v, decay, beta, float(q_scale), state, state_slots, cu_q, out)


def gated_rmsnorm(o, w, P, g_off: int, eps: float, out_scale: float, out) -> None:
  """out [T, H dv] = o / rms(o per head) * w * silu(P[:, g_off : +H dv]) * out_scale."""
  _mix("gated_rmsnorm", _gpu(o))(o, w, P, int(g_off), float(eps), float(out_scale), out)


# ------------------------------------------------------------------ post-norm blocks (csrc/hybrid.hip)
pool_dims = ref.pool_dims


def gated_postnorm(x, y, P, g_off: int, gate_b, alpha: float, w, eps: float, out=None) -> None:
  """fp32 stream rows x [T, D] <- (alpha x + y * sigmoid(P[:, g_off : +D] + gate_b)) / rms * w in place (P None: the
  sublayer's result y is not gated); with `out`, out[:, :D] = the new x in out's dtype (the next GEMM's operand)."""
  _mix("gated_postnorm", _gpu(x))(x, y, P, int(g_off), gate_b, float(alpha), w, float(eps), out)


def qk_norm_rope_store(P, bias, q_off: int, k_off: int, v_off: int, H: int, G: int, d: int, dv: int, R: int, pos, cos_sin,
                       slots, eps: float, qk_norm: bool, q_out, k_cache, v_cache) -> None:
  """q / k / v = P's columns (+ bias, one fp32 number per column of P); rotate-half RoPE on the first R dims of every
  q / k head, then (qk_norm) each head divided by its RMS; q -> q_out [T, H, d], k -> k_cache [pages, G, 64, d],
  v -> v_cache [pages, Gv, dv, 64] at `slots` (Gv = v_cache's heads: G, or fewer when neighbouring key heads share a
  value head).  k_off < 0: the layer has no keys and values of its own."""
  _mix("qk_norm_rope_store", _gpu(P))(P, bias, int(q_off), int(k_off), int(v_off), int(H), int(G), int(d), int(dv), int(R),
                                      pos, cos_sin, slots, float(eps), bool(qk_norm), q_out, k_cache, v_cache)


def kv_pool_update(k_cache, v_cache, kp, vp, block_tables, cu_q, ctx_lens, pool: int, max_qlen: int) -> None:
  """Mean key and value of every block of `pool` consecutive tokens whose last token is among the step's new ones,
  read from the paged caches as they hold them, into the pooled caches kp [pages, G, per, d] / vp [pages, G, per, dv]
  (entry of block b: with the page of its last token, see pool_dims)."""
  _mix("kv_pool_update", _gpu(k_cache))(k_cache, v_cache, kp, vp, block_tables, cu_q, ctx_lens, int(pool), int(max_qlen))


def attn_window_pool(q, k_cache, v_cache, kp, vp, block_tables, cu_q, ctx_lens, sink, scale: float, window: int,
                     pool: int, out, max_qlen: int = 0) -> None:
  """out [T, H dv] = softmax attention of each new token over the tokens at most window - 1 places back (window 0:
  all), the pooled blocks that end at or before position - window (pool 0: none), and the per-head sink logit.  Key
  head g reads value head g / (G / Gv) (the caches' head counts); out may be fp32 beside bf16 caches."""
  _mix("attn_window_pool", _gpu(q))(q, k_cache, v_cache, kp, vp, block_tables, cu_q, ctx_lens, sink, float(scale),
                                    int(window), int(pool), out, int(max_qlen) or int(q.shape[0]))


def ssd_prep(P, x_off: int, dt_off: int, conv_w, conv_b, conv_state, state_slots, cu_q, A_log, dt_bias, H: int, dv: int,
             xbc, v, decay) -> None:
  """SSD inputs of a step: xbc [T, C] = silu(causal conv of P[:, x_off : +C] + conv_b) (x | B | C channels),
  dt = softplus(P[:, dt_off : +H] + dt_bias), v [T, H dv] = dt * x, decay [T, H] = exp(-exp(A_log) dt); the
  convolution state [slots, taps - 1, C] takes the step's last inputs."""
  _mix("ssd_prep", _gpu(P))(P, int(x_off), int(dt_off), conv_w, conv_b, conv_state, state_slots, cu_q, A_log, dt_bias,
                            int(H), int(dv), xbc, v, decay)


def ssd_gate_norm(o, xbc, skip_d, P, z_off: int, w, groups: int, eps: float, out) -> None:
  """out[:, :inner] = group_rms_norm((o + D[head] * x) * silu(P[:, z_off : +inner])) * w, in `groups` equal parts."""
  _mix("ssd_gate_norm", _gpu(o))(o, xbc, skip_d, P, int(z_off), w, int(groups), float(eps), out)


def polynorm_act(P, up_off: int, F: int, coef, eps: float, out) -> None:
  """out[:, :F] = a N(z) + b N(z^2) + c N(z^3) + e, z = P[:, up_off : +F], N = division by the row's RMS, coef = (a, b, c, e)."""
  _mix("polynorm_act", _gpu(P))(P, int(up_off), int(F), coef, float(eps), out)


def relu2(P, off: int, F: int, out) -> None:
  """out[:, :F] = relu(P[:, off : +F])^2."""
  _mix("relu2", _gpu(P))(P, int(off), int(F), out)


def moe_weighted_sum(y, slot_of, topw, k: int, sh_y, P, shg_off: int, out, splits: int = 1) -> None:
  """out [T, D] fp32 = sum_j topw[t, j] * y[slot_of[t, j]] (+ sigmoid(P[t, shg_off]) * sh_y[t] for a shared expert);
  y [splits * T k, >= D]: the experts' down projections, K slice after K slice."""
  _mix("moe_weighted_sum", _gpu(y))(y, slot_of, topw, int(k), sh_y, P, int(shg_off), out, int(splits))


# ------------------------------------------------------------------ sandwich blocks (csrc/latent.hip)
def sandwich_add_norm(x, y, wb, wn, eps: float, out=None, bb=None, bn=None, mult: float = 1.0) -> None:
  """fp32 stream rows x [T, D] += mult * norm(y) * wb in place (y None: nothing is added); with wn, out[:, :D] =
  norm(x) * wn in out's dtype (the next GEMM's operand).  norm = division by the RMS, or, with the biases bb / bn, the
  layer norm (v - mean) / sqrt(var + eps) * w + b."""
  _mix("sandwich_add_norm", _gpu(x))(x, y, wb, wn, float(eps), out, bb, bn, float(mult))


def latent_kv_store(P, ckv_off: int, R: int, dr: int, kv_norm, q_off: int, q_rank: int, q_norm, eps: float, rot_dims: int,
                    interleaved: bool, pos, cos_sin, slots, cache, qa_out) -> None:
  """Per token: the latent rms_norm(P[:, ckv_off : +R]) * kv_norm and the rotated key part rope(P[:, ckv_off + R : +dr])
  -> cache [pages, 1, 64, R + dr] at `slots`; q_rank > 0: qa_out[:, :q_rank] = rms_norm(P[:, q_off : +q_rank]) * q_norm
  (the query latent, operand of the query up-projection).  RoPE on the first rot_dims dims of the rotated part, pairs
  (2i, 2i + 1) (interleaved) or (i, i + rot_dims / 2); cos_sin [rows, rot_dims] = (cos | sin)."""
  _mix("latent_kv_store", _gpu(P))(P, int(ckv_off), int(R), int(dr), kv_norm, int(q_off), int(q_rank), q_norm, float(eps),
                                   int(rot_dims), bool(interleaved), pos, cos_sin, slots, cache, qa_out)


def latent_q_rope(Q, q_off: int, H: int, dn: int, dr: int, rot_dims: int, interleaved: bool, pos, cos_sin, qn_out,
                  qpe_out) -> None:
  """Queries Q[:, q_off : +H (dn + dr)], head by head [dn unrotated | dr rotated]: the unrotated parts -> qn_out
  [H, T, dn] (operand of the per-head product with W_uk), the rotated parts after RoPE -> qpe_out [T, H, dr]."""
  _mix("latent_q_rope", _gpu(Q))(Q, int(q_off), int(H), int(dn), int(dr), int(rot_dims), bool(interleaved), pos, cos_sin,
                                 qn_out, qpe_out)


def latent_attn(q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, sink, scale: float, window: int, out,
                max_qlen: int = 0) -> None:
  """out [H, T, R] = softmax attention of every head's absorbed query (q_lat [H, T, R] against the cached latents, q_pe
  [T, H, dr] against the cached rotated key parts, times scale) over the tokens at most window - 1 places back
  (window 0: all earlier ones), the values being the latents themselves; sink [H] (or None): one more logit per head in
  the denominator.  cache [pages, 1, 64, R + dr]."""
  _mix("latent_attn", _gpu(q_lat))(q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, sink, float(scale), int(window), out,
                                   int(max_qlen) or int(q_lat.shape[1]))


def latent_out_gate(o, P, g_off: int, gate: int, out) -> None:
  """o [H, T, dv] -> out[:, :H dv] (token-major, out's dtype) times sigmoid(P[:, g_off : ...]): gate 0 none, 1 one
  gate per element, 2 one per head."""
  _mix("latent_out_gate", _gpu(o))(o, P, int(g_off), int(gate), out)


def glu_act(P, gate_off: int, up_off: int, F: int, clamped: bool, limit: float, out) -> None:
  """out[:, :F] = silu(g) * u, or (clamped) g' sigmoid(1.702 g') (u' + 1) with g' = min(g, limit), u' = clamp(u,
  -limit, limit); g = P[:, gate_off : +F], u = P[:, up_off : +F]."""
  _mix("glu_act", _gpu(P))(P, int(gate_off), int(up_off), int(F), bool(clamped), float(limit), out)


# ------------------------------------------------------------------ layer-norm sandwich blocks (csrc/recurrent_gates.hip)
def diff_attn_out(a, P, g_off: int, H: int, G: int, lam: float, post: float, eps: float, out) -> None:
  """Differential attention's combination: a [T, 2 H dv] fp32, the two maps' outputs with heads ordered (kv head, map, head
  of the group) -> out[:, :H dv] = rms_norm(a_1 - lam a_2) * post * sigmoid(P[:, g_off + head])."""
  _mix("diff_attn_out", _gpu(a))(a, P, int(g_off), int(H), int(G), float(lam), float(post), float(eps), out)


def sigmoid_gate_mul(a, P, g_off: int, out) -> None:
  """out[:, :n] = a * sigmoid(P[:, g_off : +n]) for a [T, n], fp32 or of out's dtype (out's own rows: in place)."""
  _mix("sigmoid_gate_mul", _gpu(a))(a, P, int(g_off), out)


def silu_cols(P, off: int, n: int, out) -> None:
  """out [T, n] fp32 = silu(P[:, off : +n])."""
  _mix("silu_cols", _gpu(P))(P, int(off), int(n), out)


def mlstm_gates(P, i_off: int, f_off: int, gate_b, cap: float, mstate, state_slots, cu_q, decay, inscale, mout) -> None:
  """The mlstm's gates of a step, per head: i = cap tanh((P[i_off + h] + gate_b[h]) / cap), f = logsigmoid(cap tanh((P[f_off
  + h] + gate_b[H + h]) / cap)), the running maximum m_t = max(f + m_(t-1), i) continued from mstate [slots, H] (updated
  in place); decay [T, H] = e^(f + m_(t-1) - m_t), inscale = e^(i - m_t), mout = m_t."""
  _mix("mlstm_gates", _gpu(P))(P, int(i_off), int(f_off), gate_b, float(cap), mstate, state_slots, cu_q, decay, inscale, mout)


def gated_group_norm(o, m, w, P, g_off: int, groups: int, eps: float, out) -> None:
  """out[:, :groups gs] = o's values divided by their group's RMS, times w, times sigmoid(P[:, g_off : ...]).  With m
  [T, groups] every group of o carries one channel more, a normaliser n, and its values are first divided by max(|n|,
  e^(-m)) + 1e-6."""
  _mix("gated_group_norm", _gpu(o))(o, m, w, P, int(g_off), int(groups), float(eps), out)


def pair_norm_mean(y1, y2, w, eps: float, out) -> None:
  """out [T, D] fp32 = (rms_norm(y1) * w[0] + rms_norm(y2) * w[1]) / 2."""
  _mix("pair_norm_mean", _gpu(y1))(y1, y2, w, float(eps), out)
