"""Forward pass of one pipeline shard of a dense (Llama/Qwen2/Mistral) or MoE (Mixtral) decoder.

Per layer, all on the kernel library (ops.*), with the residual stream `h` carried in place:
  xn  = rmsnorm(h, ln1)
  qkv = xn @ qkv_w.T (+b)                          fused QKV GEMM
  q   = rope(qkv.q); cache <- rope(qkv.k), qkv.v   one kernel, paged write (slot mapping)
  a   = attention(q, paged cache)                  decode: split-KV GQA; prefill: causal varlen
  h   = h + a @ o_w.T                              residual add in the GEMM epilogue
  xn  = rmsnorm(h, ln2)
  act = silu(xn @ gate.T) * (xn @ up.T)            one GEMM (interleaved gate/up), SiLU in the epilogue
  h   = h + act @ down.T                           residual add in the GEMM epilogue
Last shard: rmsnorm + LM head on each sequence's LAST row only (the reference computes the head over
every prompt row and keeps [:, -1], sharded_inference_engine.py:366), fp32 logits for the sampler.

Hidden-state contract between shards: the output of this shard's end_layer (fixing the reference's
off-by-one that returns the *input* of the last layer and IndexErrors on middle shards,
llm_utils.py:404-440 / general_mha.py:209).
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch

from ..inference.shard import Shard
from ..ops import kernels as K
from ..ops._ext import require
from ..ops.linear import FUSE_MERGE, FUSE_NORM, PendingNorm, layout_of, linear, linear_resid_norm, linear_rope_kv, scratch
from ..ops.rope import longrope_window, rope_shift, rope_table
from .config import ModelConfig
from .weights import ShardWeights, expert

# average rows per expert above which the grouped expert GEMMs run on gemm_big tiles
MOE_BIG_MIN_ROWS = float(os.environ.get("XOT_MOE_BIG_MIN_ROWS", "24"))
# K splits of the grouped gate/up GEMM for decode-sized batches (1: fused SiLU epilogue, no slabs)
MOE_GU_SPLITS = int(os.environ.get("XOT_MOE_GU_SPLITS", "4"))
MOE_BM = int(os.environ.get("XOT_MOE_BM", "0"))  # force the grouped gemm_big tile code (tests, A/B)
MOE_DN_SPLITS = int(os.environ.get("XOT_MOE_DN_SPLITS", "0"))  # force the grouped down GEMM's K split on gemm_big tiles
MOE_PP2 = os.environ.get("XOT_MOE_PP2", "1") == "1"  # 256-row expert tiles on the two-phase ping-pong schedule
PAGE = 64


def moe_tiles(rows: float, E: int) -> Tuple[int, int, int]:
  """(gate/up tile code, down tile code, down K split) of the grouped expert GEMMs on gemm_big tiles at `rows`
  average rows per expert.  Tile code = row tile + 1000 for the deeper LDS pipeline (three 64-deep stages for
  128 rows: more expert-weight bytes in flight, which is what the HBM-bound small groups need).  Measured at
  Mixtral shapes (tools/bench_moe.py, profiles/r3/moe_tiles/): ~32 rows gate/up 315 us (1128) vs 356 (128),
  down 144 (1128, S 2) vs 166; ~64 rows gate/up 441 (1128) vs 566 (128), down 178 (256, S 2) vs 288 (128, S 2);
  ~128 rows 192-row tiles (gate/up 439 us, down 254 at S 4).  Many small experts (DeepSeek-V2-Lite, 64 x ~24
  rows) keep 256-row tiles (11.0 vs 12.6 ms per step with 128)."""
  if rows <= 96 and E > 16:
    return 256, 256, 2
  if rows <= 48:
    return 1128, 1128, 2
  if rows <= 96:
    return 1128, 256, 2
  if rows <= 160:
    return 192, 192, 4
  return 256, 256, 2


@dataclass
class StepInputs:
  """Device-side description of one forward step over a batch of sequences (all int tensors)."""
  positions: torch.Tensor  # [T] int32 absolute position of each new token
  slots: torch.Tensor  # [T] int64 global KV slot of each new token (-1: do not write)
  block_tables: torch.Tensor  # [B, max_blocks] int32
  ctx_lens: torch.Tensor  # [B] int32 context length INCLUDING the new tokens
  cu_q: torch.Tensor  # [B+1] int32 offsets of each sequence's new tokens in T
  last_idx: torch.Tensor  # [B] int64 row of each sequence's last new token
  max_qlen: int
  decode: bool  # every sequence has exactly one new token
  image_embeds: Optional[torch.Tensor] = None  # LLaVA: [n image-token rows, D], in token order (first shard)
  # models with recurrent layers: [B] int32 state slot of each sequence (-1: padding row, nothing is read or written)
  state_slots: Optional[torch.Tensor] = None

  @property
  def num_tokens(self) -> int:
    return int(self.positions.numel())

  @property
  def batch(self) -> int:
    return int(self.ctx_lens.numel())


class KVCache:
  """Per-shard paged KV pool: K [L, pages, Hkv, 64, Dh] and V [L, pages, Hkv, Dh, 64] (V storage: each page chunk-major,
  [8 chunks][Dh][8 keys], ops/reference.py v_chunks).
  MLA models (DeepSeek) keep one latent row per token instead: k = C [L, pages, 64, kv_lora + rope], v None."""

  def __init__(self, c: ModelConfig, n_layers: int, num_pages: int, device, dtype=torch.bfloat16, layer_ids=None):
    self.num_pages = num_pages
    self.device = torch.device(device)
    if c.is_mixed:
      # one K [pages, G, 64, d] and one V [pages, G, d, 64] pool per layer that has an attention mixer (None for the others):
      # layers may differ in heads and sizes; the value pool holds whatever the layer's mixer stores as values
      # (one entry per layer RUN: a looped layer has a cache of its own in every pass, config.layer_runs)
      ids = [i for i, _ in c.layer_runs(layer_ids if layer_ids is not None else range(n_layers))]
      dims = [c.layer_specs[i].kv_dims for i in ids]
      self.k = [None if a is None else torch.zeros(num_pages, a[0], PAGE, a[1], device=device, dtype=dtype) for a in dims]
      # (latent attention keeps no value pool: the cached latent is key and value, value dim 0)
      # (key heads that share values: a fourth entry gives the value heads)
      self.v = [None if a is None or not a[2] else
                torch.zeros(num_pages, a[3] if len(a) > 3 else a[0], a[2], PAGE, device=device, dtype=dtype) for a in dims]
      # window attention with pooled blocks: per layer the (source layer, block size) pooled caches it reads, K
      # [pages, G, per, d] and V [pages, G, per, dv]; entries live with the page of a block's last token, so they are
      # handed out and returned with the sequence's pages.  pool_owner[j]: this layer fills them (the first layer of
      # the shard that reads this source with this block size); a layer that borrows another's keys and values aliases
      # that layer's pools.
      self.kp: List[Optional[torch.Tensor]] = [None] * len(ids)
      self.vp: List[Optional[torch.Tensor]] = [None] * len(ids)
      self.pool_owner = [False] * len(ids)
      made = {}
      for j, i in enumerate(ids):
        a = c.layer_specs[i].wattn
        if a is None:
          continue
        src = i if a.kv_from < 0 else a.kv_from
        if src not in ids:
          raise ValueError(f"layer {i} reads the keys and values of layer {src}, which is not on this shard")
        # (the source's run that this run follows: a looped layer has a cache of its own in every pass)
        js = j if src == i else max([jj for jj in range(j) if ids[jj] == src], default=ids.index(src))
        self.k[j], self.v[j] = self.k[js], self.v[js]
        src = js  # pooled caches belong to the run, too
        if a.pool > 0 and a.window > 0:
          if (src, a.pool) not in made:
            per = K.pool_dims(a.pool)
            made[(src, a.pool)] = (torch.zeros(num_pages, a.kv_heads, per, a.dim, device=device, dtype=dtype),
                                   torch.zeros(num_pages, a.kv_heads, per, a.vdim, device=device, dtype=dtype))
            self.pool_owner[j] = True
          self.kp[j], self.vp[j] = made[(src, a.pool)]
      return
    if c.is_mla:
      self.k = torch.zeros(n_layers, num_pages, PAGE, c.mla_dim, device=device, dtype=dtype)
      self.v = None
      return
    self.k = torch.zeros(n_layers, num_pages, c.num_kv_heads, PAGE, c.head_dim, device=device, dtype=dtype)
    self.v = torch.zeros(n_layers, num_pages, c.num_kv_heads, c.head_dim, PAGE, device=device, dtype=dtype)

  @staticmethod
  def bytes_per_page(c: ModelConfig, n_layers: int, layer_ids=None, itemsize: int = 2) -> int:
    if c.is_mixed:
      ids = [i for i, _ in c.layer_runs(layer_ids if layer_ids is not None else range(n_layers))]
      n, seen = 0, set()
      for j, i in enumerate(ids):
        a, w = c.layer_specs[i].kv_dims, c.layer_specs[i].wattn
        if a is not None:
          n += PAGE * (a[0] * a[1] + (a[3] if len(a) > 3 else a[0]) * a[2]) * itemsize
        if w is not None and w.pool > 0 and w.window > 0:
          # (pooled caches: one per run of the source layer and block size)
          js = j if w.kv_from < 0 else max([jj for jj in range(j) if ids[jj] == w.kv_from], default=-1)
          if (js, w.pool) not in seen:
            seen.add((js, w.pool))
            n += w.kv_heads * K.pool_dims(w.pool) * (w.dim + w.vdim) * itemsize
      return max(1, n)
    if c.is_mla:
      return n_layers * PAGE * c.mla_dim * 2
    return 2 * n_layers * c.num_kv_heads * PAGE * c.head_dim * 2

  def nbytes(self) -> int:
    ts = (self.k + self.v + getattr(self, "kp", []) + getattr(self, "vp", [])) if isinstance(self.k, list) else (self.k, self.v)
    seen, n = set(), 0
    for t in ts:
      if t is not None and t.data_ptr() not in seen:
        seen.add(t.data_ptr())
        n += t.numel() * t.element_size()
    return n


class StatePool:
  """Recurrent state of a shard's layers, one slot per live request (models.config.LinearRecurrenceSpec): per layer
  with a recurrence S^T [slots, H, dv, d] fp32 (a value channel's key rows contiguous) and, for rules with short convolutions, the last taps - 1 convolution
  inputs [slots, taps - 1, channels] fp32; rules that carry scalars per head beside the matrix (the mlstm's running maximum)
  keep them in aux [slots, H, n] fp32.  A slot is cleared when a request is admitted to it."""

  def __init__(self, c: ModelConfig, layer_ids, slots: int, device):
    self.slots = slots
    self.S: List[Optional[torch.Tensor]] = []
    self.conv: List[Optional[torch.Tensor]] = []
    self.aux: List[Optional[torch.Tensor]] = []
    for i, _ in c.layer_runs(layer_ids):  # (a looped layer: a state of its own in every pass)
      sd = c.layer_specs[i].state_dims  # (heads, value channels, key dim, taps, convolution channels, scalars per head)
      self.S.append(None if sd is None else torch.zeros(slots, sd[0], sd[1], sd[2], device=device, dtype=torch.float32))
      self.conv.append(torch.zeros(slots, max(sd[3] - 1, 0), sd[4], device=device, dtype=torch.float32)
                       if sd is not None and sd[4] else None)
      self.aux.append(torch.zeros(slots, sd[0], sd[5], device=device, dtype=torch.float32) if sd is not None and sd[5] else None)

  def clear(self, slot: int) -> None:
    for t in self.S + self.conv + self.aux:
      if t is not None:
        t[slot].zero_()

  def nbytes(self) -> int:
    return sum(t.numel() * 4 for t in self.S + self.conv + self.aux if t is not None)


class ShardModel:
  def __init__(self, weights: ShardWeights, kv: KVCache, max_batch: int = 256, max_ctx: int = 8192):
    self.w = weights
    self.c: ModelConfig = weights.config
    self.shard: Shard = weights.shard
    self.kv = kv
    self.device = kv.device if hasattr(kv, "device") else kv.k.device
    c = self.c
    self.state: Optional[StatePool] = None  # set by the runner for models with recurrent layers
    if c.is_mixed:
      self.layer_ids = list(self.shard.layers())
      self.max_batch, self.max_ctx, self.ws = max_batch, max_ctx, None
      self.rope_rows, self.rope_window = max(max_ctx, 16), None
      self.head_rows, self._head_cache = None, None
      # one [rows, R] (cos | sin) table per distinct (rotary dims, base) among the attention mixers
      self.rope_tabs = {}
      from ..ops.rope import build_cos_sin
      for i in self.layer_ids:
        a = c.layer_specs[i].attn
        if a is not None and a.rot_dims and (a.rot_dims, a.rot_base) not in self.rope_tabs:
          self.rope_tabs[(a.rot_dims, a.rot_base)] = build_cos_sin(a.rot_dims, self.rope_rows, a.rot_base, None, self.device)
        a = c.layer_specs[i].wattn
        if a is not None and a.rot_dims and (a.rot_dims, a.rot_base, a.rot_scaling) not in self.rope_tabs:
          sc = a.rot_scaling and dict(rope_type="llama3", factor=a.rot_scaling[0], low_freq_factor=a.rot_scaling[1],
                                      high_freq_factor=a.rot_scaling[2], original_max_position_embeddings=a.rot_scaling[3])
          self.rope_tabs[(a.rot_dims, a.rot_base, a.rot_scaling)] = build_cos_sin(a.rot_dims, self.rope_rows, a.rot_base,
                                                                                 sc, self.device)
        a = c.layer_specs[i].lattn or c.layer_specs[i].dattn
        if a is not None and a.rot_dims and (a.rot_dims, a.rot_base) not in self.rope_tabs:
          self.rope_tabs[(a.rot_dims, a.rot_base)] = build_cos_sin(a.rot_dims, self.rope_rows, a.rot_base, None, self.device)
      self.runs = c.layer_runs(self.layer_ids)
      return
    self.scale = 1.0 / math.sqrt(c.head_dim)
    max_pos = max(max_ctx, 16)
    self.cos_sin = rope_table(c, max_pos, self.device)
    self.rope_rows, self.rope_window = max_pos, longrope_window(c)
    self.layer_ids: List[int] = list(self.shard.layers())
    self.max_batch = max_batch
    self.max_ctx = max_ctx
    self.ws = None
    if self.device.type == "cuda":
      if c.is_mla:
        self.ws = K.MLAWorkspace(max_batch, c.num_heads, c.kv_lora_rank, max_ctx, self.device)
      else:
        self.ws = K.DecodeWorkspace(max_batch, c.num_heads, c.head_dim, max_ctx, self.device)
    if c.is_mla:
      self.scale = c.attn_scale()
    # last shard with the LM head split across two ring stages: logits of vocab rows [0, head_rows) only,
    # and forward returns (logits, normed hidden)
    self.head_rows: Optional[int] = None
    self._head_cache = None

  def rope_pos(self, start: int, n: int) -> range:
    """RoPE table rows of a step's n new tokens at positions start.. (LongRoPE: the long-factor half
    once the sequence outgrows the pretraining window; positions only feed the RoPE kernels)."""
    o = rope_shift(self.rope_window, self.rope_rows, start + n)
    return range(start + o, start + n + o)

  # ------------------------------------------------------------------ helpers
  def _attention(self, q: torch.Tensor, li: int, inp: StepInputs, ws=None, defer_merge: bool = False):
    kc, vc = self.kv.k[li], self.kv.v[li]
    if inp.decode:
      return K.attn_decode(q, kc, vc, inp.block_tables, inp.ctx_lens, self.scale, ws or self.ws,
                           defer_merge=defer_merge)
    return K.attn_prefill(q, kc, vc, inp.block_tables, inp.cu_q, inp.ctx_lens, inp.max_qlen, self.scale)

  def _mla(self, xn: torch.Tensor, lw, li: int, inp: StepInputs) -> torch.Tensor:
    """DeepSeek multi-head latent attention -> [T, H * v_head_dim] (before o_proj).
    A = xn @ [q_a | kv_a]^T; q = rmsnorm(q_a) @ q_b^T (or A's q part); latent norm + rope + cache write;
    absorbed query q_lat = q_nope . W_UK per head; attention over the latent cache (csrc/mla.hip);
    o = o_lat . W_UV^T per head."""
    c = self.c
    T = xn.shape[0]
    H, dn, dr, dv, L = c.num_heads, c.qk_nope_head_dim, c.qk_rope_head_dim, c.v_head_dim, c.kv_lora_rank
    A = linear(xn, lw.qkv_w)
    nq = c.q_lora_rank or H * (dn + dr)
    if c.q_lora_rank:
      qa, _ = K.rmsnorm(A[:, :nq].contiguous(), lw.q_ln, c.rms_norm_eps)
      q = linear(qa, lw.qb_w)  # [T, H dn | H dr]
    else:
      q = A  # q = A[:, :nq], rows of stride A.shape[1]
    ckv = A[:, nq:]
    cache = self.kv.k[li]
    K.mla_prep(ckv, lw.kv_ln, q, H * dn, H, inp.positions, self.cos_sin, inp.slots, cache, c.rms_norm_eps)
    dt = q.dtype
    q_pe = q[:, H * dn:]
    if getattr(lw.wuk, "xot_layout", "rowmajor") == "stream_t":
      # absorbed projections on the batched stream GEMM (pre-shuffled per head, csrc/gemm.hip MOE==3 mode):
      # head h reads q[:, h dn:(h+1) dn] in place and writes q_lat[h]; o_lat[h] . W_UV[h]^T lands in o[:, h dv:]
      KC = require()
      q_lat = torch.empty(H, T, L, device=q.device, dtype=dt)
      KC.gemm_batched(q[:, :H * dn], dn, dn, lw.wuk, q_lat, T * L, L, T)
      o_lat = K.mla_attn(q_lat, q_pe, cache, inp.block_tables, inp.cu_q, inp.ctx_lens, self.scale, self.ws)
      o = torch.empty(T, H * dv, device=q.device, dtype=dt)
      KC.gemm_batched(o_lat.view(H * T, L), T * L, L, lw.wuv, o, dv, H * dv, T)
      return o
    q_nope = q[:, :H * dn].view(T, H, dn).transpose(0, 1)  # [H, T, dn]
    if xn.is_cuda:
      q_lat = torch.bmm(q_nope, lw.wuk)  # [H, T, L] (row-major weights: shapes gemm_batched does not tile)
    else:  # CPU reference path: fp32 math whatever the shard's storage dtypes
      q_lat = torch.bmm(q_nope.float(), lw.wuk.float()).to(dt)
    o_lat = K.mla_attn(q_lat, q_pe, cache, inp.block_tables, inp.cu_q, inp.ctx_lens, self.scale, self.ws)
    if xn.is_cuda:
      o = torch.bmm(o_lat, lw.wuv.transpose(1, 2))  # [H, T, dv]
    else:
      o = torch.bmm(o_lat.float(), lw.wuv.float().transpose(1, 2)).to(dt)
    return o.transpose(0, 1).reshape(T, H * dv)

  def _mlp(self, xn: torch.Tensor, lw, h: torch.Tensor, next_norm: Optional[torch.Tensor], li: int = -1,
           defer_to: Optional[torch.Tensor] = None):
    """h += MLP(xn) in place; returns rmsnorm(h) * next_norm (None if there is no following norm), or a
    PendingNorm whose residual continues in defer_to (see linear_resid_norm)."""
    c = self.c
    if lw.router is None:
      act = linear(xn, lw.gu_w, epi="silu")
      if next_norm is not None:
        return linear_resid_norm(act, lw.down_w, h, next_norm, c.rms_norm_eps, defer_to=defer_to)
      linear(act, lw.down_w, residual=h, epi="resid", out=h)
      return None
    if isinstance(xn, PendingNorm):
      xn = xn.materialize()
    out = self._moe(xn, lw, h, next_norm)
    if out is not None:  # the combine kernel also applied the following RMSNorm
      return out
    return K.rmsnorm(h, next_norm, c.rms_norm_eps)[0] if next_norm is not None else None

  @property
  def _ds_route(self) -> bool:
    """DeepSeekMoE routing (groups / sigmoid / bias / unnormalised scaled weights) vs Mixtral's."""
    c = self.c
    return not (c.topk_method == "greedy" and c.scoring_func == "softmax" and c.norm_topk_prob
                and c.routed_scaling_factor == 1.0)

  def _route_args(self):
    c = self.c
    method = {"greedy": 0, "group_limited_greedy": 1, "noaux_tc": 2}[c.topk_method]
    return (c.num_experts_per_tok, c.n_group if method else 1, c.topk_group if method else 1, method,
            c.scoring_func == "sigmoid", c.norm_topk_prob, c.routed_scaling_factor)

  def _moe(self, xn: torch.Tensor, lw, h: torch.Tensor, next_norm: Optional[torch.Tensor] = None):
    """Sparse MoE: top-k routing (Mixtral softmax, or DeepSeek's grouped / sigmoid-with-bias rules), shared
    experts (DeepSeek) added as a dense SwiGLU, tokens grouped per expert, expert GEMMs on the kernel library
    (gate/up with fused SiLU epilogue), weighted scatter-add back into h."""
    c = self.c
    if lw.sh_gu_w is not None:  # shared experts: h += down(silu(gate) * up) of every token
      linear(linear(xn, lw.sh_gu_w, epi="silu"), lw.sh_down_w, residual=h, epi="resid", out=h)
    if xn.is_cuda and (c.num_experts in (4, 8, 16) or (c.num_experts in (32, 64, 128, 160, 256)
                                                       and c.hidden_size % 512 == 0)) and layout_of(lw.router) == "rowmajor":
      # fp32 router logits, one small kernel (instead of a bf16 library GEMM + cast)
      logits = torch.empty(xn.shape[0], c.num_experts, dtype=torch.float32, device=xn.device)
      require().router_logits(xn.contiguous(), lw.router.contiguous(), logits)
    else:
      logits = linear(xn, lw.router, out_dtype=torch.float32)  # [T, E]
    if xn.is_cuda:
      return self._moe_gpu(xn, lw, h, logits, next_norm)
    if self._ds_route:
      topw, topi = K.moe_route_ds(logits, lw.router_bias, *self._route_args())
    else:
      probs = torch.softmax(logits, dim=-1)
      topw, topi = torch.topk(probs, c.num_experts_per_tok, dim=-1)
      topw = topw / topw.sum(-1, keepdim=True)
    T = xn.shape[0]
    flat_e = topi.reshape(-1)
    order = torch.argsort(flat_e, stable=True)
    tok = order // c.num_experts_per_tok
    counts = torch.bincount(flat_e, minlength=c.num_experts).tolist()
    out = torch.zeros(T, c.hidden_size, device=xn.device, dtype=torch.float32)
    start = 0
    wflat = topw.reshape(-1)[order]
    for e, n in enumerate(counts):
      if n == 0:
        continue
      idx = tok[start:start + n]
      xe = xn.index_select(0, idx)  # (expert weights of Fe = c.expert_dim rows)
      act = linear(xe, expert(lw.gu_w, e), epi="silu")
      ye = linear(act, expert(lw.down_w, e), out_dtype=torch.float32)
      out.index_add_(0, idx, ye * wflat[start:start + n, None])
      start += n
    h += out.to(h.dtype)
    return None

  def _moe_gpu(self, xn: torch.Tensor, lw, h: torch.Tensor, logits: torch.Tensor,
               next_norm: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """Device-only MoE (graph-capturable): routing kernel (softmax top-k, per-expert slot order),
    grouped gate/up GEMM gathering token rows with the SiLU*mul epilogue, grouped down GEMM into fp32
    slots, combine kernel adding sum_j w_j * y_slot(j) into the residual stream."""
    c = self.c
    T, D = xn.shape
    k, E, F = c.num_experts_per_tok, c.num_experts, c.expert_dim
    dev = xn.device
    C = require()
    topw = torch.empty(T * k, dtype=torch.float32, device=dev)
    topi = torch.empty(T * k, dtype=torch.int32, device=dev)
    slot_of = torch.empty(T * k, dtype=torch.int32, device=dev)
    sorted_tok = torch.empty(T * k, dtype=torch.int32, device=dev)
    off = torch.empty(E + 1, dtype=torch.int32, device=dev)
    if self._ds_route:
      K.moe_route_ds(logits, lw.router_bias, *self._route_args(), outs=(topw, topi, slot_of, sorted_tok, off))
    else:
      C.moe_route(logits.contiguous(), k, topw, topi, slot_of, sorted_tok, off)
    shuffled = layout_of(lw.gu_w) == "stream" and layout_of(lw.down_w) == "stream"
    # rows per expert decide the kernel: the weight-streaming GEMM for decode-sized groups, gemm_big
    # tiles (128 or 256 rows) once the groups are compute-bound
    rows = T * k / E
    bm, bm_dn, S_dn = (0, 0, 0) if not shuffled or rows < MOE_BIG_MIN_ROWS else moe_tiles(rows, E)
    if MOE_PP2:  # 256- / 192-row expert tiles on the two-phase ping-pong schedule (csrc/gemm_big.hip 2256 / 2192)
      bm, bm_dn = ({256: 2256, 192: 2192}.get(b, b) for b in (bm, bm_dn))
    if MOE_BM and bm:
      bm = bm_dn = MOE_BM
    if MOE_DN_SPLITS and bm:
      S_dn = MOE_DN_SPLITS
    act = torch.empty(T * k, F, dtype=torch.bfloat16, device=dev)
    Sg = MOE_GU_SPLITS if (bm == 0 and T * k <= 32 and D % (256 * MOE_GU_SPLITS) == 0) else 1
    if Sg > 1:
      # decode-sized groups: the weight-streaming gate/up split over K into fp32 slabs (k experts x N/128
      # column blocks alone leave the last wave of workgroups short, e.g. 448 on 512 slots at batch 1),
      # SiLU*mul applied by the slab reduce
      ys = torch.empty(Sg * T * k, 2 * F, dtype=torch.float32, device=dev)
      C.gemm_moe(xn, lw.gu_w, ys, off, sorted_tok, K.EPI["none"], T, layout_of(lw.gu_w) == "stream", Sg, 0)
      C.splitk_silu(ys, Sg, act)
    else:
      C.gemm_moe(xn, lw.gu_w, act, off, sorted_tok, K.EPI["silu"], T, layout_of(lw.gu_w) == "stream", 1, bm)
    # down projection split over K (fp32 partial slabs summed by the combine): the grouped GEMM only has
    # (experts hit) x N/tile workgroups with work, too few to stream the expert weights at full HBM rate
    S = (4 if T * k <= 64 else 2) if bm == 0 else S_dn
    if F % (256 * S):
      S = 1
    y = torch.empty(S * T * k, D, dtype=torch.float32, device=dev)
    C.gemm_moe(act, lw.down_w, y, off, None, K.EPI["none"], T, layout_of(lw.down_w) == "stream", S, bm_dn)
    if next_norm is not None:  # combine + the following RMSNorm in one kernel
      out = torch.empty_like(h)
      C.moe_combine_norm(y, slot_of, topw, h, S, next_norm, out, float(c.rms_norm_eps))
      return out
    C.moe_combine(y, slot_of, topw, h, S)
    return None

  # ------------------------------------------------------------------ layers of differing mixers
  @staticmethod
  def _proj(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """fp32 x @ w^T: the kernel library's bf16 GEMMs (fp32 accumulate and output), or the vendor SGEMM for an
    all-fp32 run."""
    if x.dtype == torch.float32:
      return torch.matmul(x, w.t())
    return linear(x, w, out_dtype=torch.float32)

  def _gated_attn(self, P: torch.Tensor, lw, j: int, inp: StepInputs, mix: torch.Tensor) -> None:
    """Chunk-local sigmoid attention: RoPE + paged write of (rotated key, key as projected), then the gated sum
    over the query's chunk, scaled into the mixers' output row."""
    a = lw.spec.attn
    q = torch.empty(P.shape[0], a.heads, a.dim, dtype=mix.dtype, device=P.device)
    tab = self.rope_tabs.get((a.rot_dims, a.rot_base))
    K.rope_kv_store(P, lw.cols["aq"][0], lw.cols["ak"][0], -1 if a.values_are_keys else lw.cols["av"][0], a.heads,
                    a.kv_heads, a.dim, a.rot_dims if tab is not None else 0,
                    inp.positions, tab if tab is not None else torch.zeros(1, 0, device=P.device), inp.slots, q,
                    self.kv.k[j], self.kv.v[j])
    off, n = lw.mix_cols["attn"]
    K.attn_gated_chunk(q, self.kv.k[j], self.kv.v[j], inp.block_tables, inp.cu_q, inp.ctx_lens, lw.attn_pb, a.scale,
                       a.chunk, lw.spec.attn_scale, mix[:, off:off + n], max_qlen=inp.max_qlen)

  def _recurrence(self, P: torch.Tensor, lw, j: int, inp: StepInputs, mix: torch.Tensor) -> None:
    """Linear-attention recurrence over each sequence's state slot (delta rule or per-channel decay), then the
    per-head gated RMS norm, scaled into the mixers' output row."""
    r, st, dev = lw.spec.rec, self.state, P.device
    T = P.shape[0]
    H, G, d, dv = r.heads, r.kv_heads, r.dim, r.vdim
    o = torch.empty(T, H * dv, dtype=torch.float32, device=dev)
    if r.rule == "delta":
      C = 2 * G * d + H * dv
      qkv = torch.empty(T, C, dtype=torch.float32, device=dev)
      beta = torch.empty(T, H, dtype=torch.float32, device=dev)
      decay = torch.empty(T, H, dtype=torch.float32, device=dev)
      K.delta_prep(P, lw.cols["rq"][0], lw.cols["rb"][0], lw.cols["ra"][0], lw.conv_w, st.conv[j], inp.state_slots,
                   inp.cu_q, lw.A_log, lw.dt_bias, H, G, d, dv, qkv, beta, decay)
      K.linear_recurrence(qkv[:, :G * d], qkv[:, G * d:2 * G * d], qkv[:, 2 * G * d:], decay, beta, 1.0, st.S[j],
                          inp.state_slots, inp.cu_q, o)
    else:
      decay = torch.empty(T, H * d, dtype=torch.float32, device=dev)
      K.gla_prep(P, lw.cols["ra1"][0], lw.a2_w, lw.a2_b, r.tau, decay)
      (qo, qn), (ko, kn), (vo, vn) = lw.cols["rq"], lw.cols["rk"], lw.cols["rv"]
      K.linear_recurrence(P[:, qo:qo + qn], P[:, ko:ko + kn], P[:, vo:vo + vn], decay, None, d ** -0.5, st.S[j],
                          inp.state_slots, inp.cu_q, o)
    off, n = lw.mix_cols["rec"]
    K.gated_rmsnorm(o, lw.rec_norm, P, lw.cols["rg"][0], self.c.rms_norm_eps, lw.spec.rec_scale, mix[:, off:off + n])

  def _forward_mixed(self, x: torch.Tensor, inp: StepInputs) -> torch.Tensor:
    """Layers of config.layer_specs on an fp32 residual stream h:
      hn = h / rms(h) * g                       one scalar gain per norm (fused into the previous layer's residual add)
      P  = hn @ in_w^T                          every projection of the layer in one GEMM, fp32 result
      mix = [attn_scale * attention | rec_scale * recurrence]    both mixers read hn; outputs side by side along K
      h += ls1 * (mix @ out_w^T) + ls2 * (gelu_tanh(gate) * up) @ down_w^T
    Returns h (non-last shard) or logit_scale * head(norm(h rows inp.last_idx))."""
    c, w = self.c, self.w
    if c.has_state and (self.state is None or inp.state_slots is None):
      raise RuntimeError("a model with recurrent layers needs a state pool and the step's state slots")
    if self.shard.is_first_layer():
      h = w.embed.index_select(0, x.view(-1).long().clamp(0, w.embed.shape[0] - 1))
    else:
      h = x.to(torch.float32).contiguous().clone()
    T, D = h.shape
    n = len(self.layer_ids)
    last = self.shard.is_last_layer()
    adt = (w.layers[self.layer_ids[0]].in_w if n else w.lm_head).dtype
    if c.block == "postln":
      return self._forward_postln(h, inp, adt)
    if c.block == "sandwich":
      return self._forward_sandwich(h, inp, adt)
    bufs = {}

    def rows(name: str, live: int, padded: int) -> torch.Tensor:
      # activation rows whose K-padding columns stay zero: kernels only write the first `live` columns
      key = (name, live, padded)
      if key not in bufs:
        bufs[key] = (torch.zeros if padded > live else torch.empty)(T, padded, dtype=adt, device=h.device)
      return bufs[key]
    hn = rows("hn", D, -(-D // 128) * 128)
    if n:
      K.resid_scale_norm(h, gain=w.layers[self.layer_ids[0]].norm_g, eps=c.rms_norm_eps, out=hn)
    for j, li in enumerate(self.layer_ids):
      lw = w.layers[li]
      s = lw.spec
      P = self._proj(hn, lw.in_w)
      live = sum(sz for _, sz in lw.mix_cols.values())
      mix = rows("mix", live, lw.out_w.shape[1])
      if s.attn is not None:
        self._gated_attn(P, lw, j, inp, mix)
      if s.rec is not None:
        self._recurrence(P, lw, j, inp, mix)
      y1 = self._proj(mix, lw.out_w)
      y2 = None
      if s.ff:
        act = rows("act", s.ff, lw.down_w.shape[1])
        K.gelu_mul(P, lw.cols["gate"][0], lw.cols["up"][0], s.ff, act)
        y2 = self._proj(act, lw.down_w)
      nxt = w.layers[self.layer_ids[j + 1]].norm_g if j + 1 < n else None
      K.resid_scale_norm(h, y1, lw.ls1, y2, lw.ls2 if y2 is not None else None, gain=nxt, eps=c.rms_norm_eps,
                         out=hn if nxt is not None else None)
    if not last:
      return h
    hl = h.index_select(0, inp.last_idx)
    xn = torch.zeros(hl.shape[0], hn.shape[1], dtype=adt, device=h.device)
    K.resid_scale_norm(hl, gain=w.norm, eps=c.rms_norm_eps, out=xn)
    logits = self._proj(xn, w.lm_head)[:, :c.vocab_size]
    return logits * c.logit_scale

  # ------------------------------------------------------------------ post-norm blocks (window attention / SSD, MoE)
  def _window_attn(self, P: torch.Tensor, lw, j: int, inp: StepInputs, mix: torch.Tensor) -> None:
    """Softmax attention over a sliding window, pooled blocks before it and a sink: biases + RoPE + per-head RMS
    division + paged write, the pooled caches' update for blocks that this step completed, then the attention."""
    a = lw.spec.wattn
    q = torch.empty(P.shape[0], a.heads, a.dim, dtype=mix.dtype, device=P.device)
    tab = self.rope_tabs.get((a.rot_dims, a.rot_base, a.rot_scaling))
    own = a.kv_from < 0
    K.qk_norm_rope_store(P, lw.in_b, lw.cols["q"][0], lw.cols["k"][0] if own else -1, lw.cols["v"][0] if own else -1,
                         a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims if tab is not None else 0, inp.positions,
                         tab if tab is not None else torch.zeros(1, 0, device=P.device), inp.slots, self.c.rms_norm_eps,
                         a.qk_norm, q, self.kv.k[j], self.kv.v[j])
    if self.kv.pool_owner[j]:
      K.kv_pool_update(self.kv.k[j], self.kv.v[j], self.kv.kp[j], self.kv.vp[j], inp.block_tables, inp.cu_q, inp.ctx_lens,
                       a.pool, inp.max_qlen)
    pool = a.pool if self.kv.kp[j] is not None else 0
    o = mix[:, :a.heads * a.vdim]
    K.attn_window_pool(q, self.kv.k[j], self.kv.v[j], self.kv.kp[j], self.kv.vp[j], inp.block_tables, inp.cu_q,
                       inp.ctx_lens, lw.sink, a.scale, a.window, pool, o, max_qlen=inp.max_qlen)
    if a.gate != "none":  # one sigmoid gate per element, from the mixer's input, applied in place
      K.sigmoid_gate_mul(o, P, lw.cols["gate"][0], mix)

  def _diff_attn(self, P: torch.Tensor, lw, j: int, inp: StepInputs, mix: torch.Tensor) -> None:
    """Differential attention on the window-attention kernels: the two maps of every head are query heads of their own
    (the fused projection orders them kv head, map, head of the group) over 2 G key heads that share G value heads;
    then a_1 - lam a_2, the per-head RMS division and the per-head gate."""
    a = lw.spec.dattn
    T, dev = P.shape[0], P.device
    q = torch.empty(T, 2 * a.heads, a.dim, dtype=mix.dtype, device=dev)
    tab = self.rope_tabs.get((a.rot_dims, a.rot_base))
    K.qk_norm_rope_store(P, None, lw.cols["q"][0], lw.cols["k"][0], lw.cols["v"][0], 2 * a.heads, 2 * a.kv_heads, a.dim, a.vdim,
                         a.rot_dims if tab is not None else 0, inp.positions,
                         tab if tab is not None else torch.zeros(1, 0, device=dev), inp.slots, self.c.rms_norm_eps, False, q,
                         self.kv.k[j], self.kv.v[j])
    o = torch.empty(T, 2 * a.heads * a.vdim, dtype=torch.float32, device=dev)
    K.attn_window_pool(q, self.kv.k[j], self.kv.v[j], None, None, inp.block_tables, inp.cu_q, inp.ctx_lens, None, a.scale,
                       a.window, 0, o, max_qlen=inp.max_qlen)
    K.diff_attn_out(o, P, lw.cols["gate"][0], a.heads, a.kv_heads, lw.lam, 1.0 - a.lam_init, self.c.rms_norm_eps, mix)

  def _mlstm(self, P: torch.Tensor, lw, j: int, inp: StepInputs, mix: torch.Tensor) -> None:
    """The xLSTM matrix memory on the state slots: gates and the running maximum per head, the framework's linear
    recurrence with one decay per head and an input scale (the normaliser is the state's last value channel), then the
    stabilised division, the per-head norm, the weight and the sigmoid gate."""
    r, st, dev = lw.spec.rec, self.state, P.device
    T, H = P.shape[0], r.heads
    decay, inscale, m = (torch.empty(T, H, dtype=torch.float32, device=dev) for _ in range(3))
    K.mlstm_gates(P, lw.cols["ri"][0], lw.cols["rf"][0], lw.gate_b, r.gate_cap, st.aux[j].view(-1, H), inp.state_slots, inp.cu_q, decay,
                  inscale, m)
    o = torch.empty(T, H * (r.vdim + 1), dtype=torch.float32, device=dev)
    (qo, qn), (ko, kn), (vo, vn) = lw.cols["rq"], lw.cols["rk"], lw.cols["rv"]
    K.linear_recurrence(P[:, qo:qo + qn], P[:, ko:ko + kn], P[:, vo:vo + vn], decay, inscale, r.dim ** -0.5, st.S[j],
                        inp.state_slots, inp.cu_q, o)
    K.gated_group_norm(o, m, lw.rec_norm, P, lw.cols["rg"][0], H, self.c.rms_norm_eps, mix)

  def _lightning(self, P: torch.Tensor, lw, j: int, inp: StepInputs, mix: torch.Tensor) -> None:
    """Lightning attention on the state slots: SiLU on q, k, v, the linear recurrence with one fixed decay per head, the
    norm over all heads together, the weight and the sigmoid gate."""
    r, st, dev = lw.spec.rec, self.state, P.device
    T, H = P.shape[0], r.heads
    nq, nv = H * r.dim, H * r.vdim
    qkv = torch.empty(T, 2 * nq + nv, dtype=torch.float32, device=dev)
    K.silu_cols(P, lw.cols["rq"][0], 2 * nq + nv, qkv)  # (q | k | v are neighbours in the fused projection)
    o = torch.empty(T, nv, dtype=torch.float32, device=dev)
    K.linear_recurrence(qkv[:, :nq], qkv[:, nq:2 * nq], qkv[:, 2 * nq:], lw.decay, None, 1.0,
                        st.S[j], inp.state_slots, inp.cu_q, o)
    K.gated_group_norm(o, None, lw.rec_norm, P, lw.cols["rg"][0], 1, self.c.rms_norm_eps, mix)

  def _ssd(self, P: torch.Tensor, lw, j: int, inp: StepInputs, mix: torch.Tensor) -> None:
    """Mamba-2 mixer on the state slots: convolution + SiLU, step sizes and decays, the recurrence on the fp32 state
    (the framework's linear recurrence with one decay per head: q = C, k = B, v = dt x), skip, gate, grouped norm."""
    m, st, dev = lw.spec.ssd, self.state, P.device
    T = P.shape[0]
    inner, gn = m.inner, m.groups * m.state
    xbc = torch.empty(T, m.conv_channels, dtype=torch.float32, device=dev)
    v = torch.empty(T, inner, dtype=torch.float32, device=dev)
    decay = torch.empty(T, m.heads, dtype=torch.float32, device=dev)
    o = torch.empty(T, inner, dtype=torch.float32, device=dev)
    i0 = lw.cols["in"][0]
    K.ssd_prep(P, i0 + inner, i0 + 2 * inner + 2 * gn, lw.conv_w, lw.conv_b, st.conv[j], inp.state_slots, inp.cu_q,
               lw.A_log, lw.dt_bias, m.heads, m.vdim, xbc, v, decay)
    K.linear_recurrence(xbc[:, inner + gn:], xbc[:, inner:inner + gn], v, decay, None, 1.0, st.S[j], inp.state_slots,
                        inp.cu_q, o)
    K.ssd_gate_norm(o, xbc, lw.skip_d, P, i0, lw.ssd_norm, m.norm_groups, self.c.rms_norm_eps, mix)

  def _relu2_moe(self, hn: torch.Tensor, P: torch.Tensor, lw, rows) -> torch.Tensor:
    """Routed relu^2 experts + the gated shared expert -> fp32 [T, D].  Routing on the framework's top-k kernels (the
    softmax over the chosen logits, or the grouped sigmoid rule with a correction), experts on the grouped GEMMs (bf16)
    or per expert on the vendor SGEMM (fp32)."""
    f, dev = lw.spec.ffn, P.device
    T, D = hn.shape[0], self.c.hidden_size
    E, k = f.experts, f.top
    r0 = lw.ff_cols["router"][0]
    grouped = f.route == "sigmoid_groups"  # sigmoid scores, choice among the best groups on the corrected scores
    logits = P[:, r0:r0 + E].contiguous() if grouped else (P[:, r0:r0 + E] + lw.router_b).contiguous()
    if P.is_cuda:
      topw = torch.empty(T * k, dtype=torch.float32, device=dev)
      topi, slot_of, sorted_tok = (torch.empty(T * k, dtype=torch.int32, device=dev) for _ in range(3))
      off = torch.empty(E + 1, dtype=torch.int32, device=dev)
      if grouped:
        K.moe_route_ds(logits, lw.router_b, k, f.groups, f.keep, 2, True, True, f.route_scale,
                       outs=(topw, topi, slot_of, sorted_tok, off))
      elif E <= 64 and k <= 8:
        require().moe_route(logits, k, topw, topi, slot_of, sorted_tok, off)
      else:
        K.moe_route_ds(logits, None, k, 1, 1, 0, False, True, 1.0, outs=(topw, topi, slot_of, sorted_tok, off))
    else:
      if grouped:
        topw, idx = K.moe_route_ds(logits, lw.router_b, k, f.groups, f.keep, 2, True, True, f.route_scale)
        topw, topi = topw.reshape(-1), idx.reshape(-1).int()
      else:
        val, idx = torch.topk(logits, k, dim=-1)
        topw, topi = torch.softmax(val, -1).reshape(-1), idx.reshape(-1).int()
      order = torch.argsort(topi, stable=True)
      slot_of = torch.empty_like(order)
      slot_of[order] = torch.arange(T * k)
      sorted_tok = (order // k).int()
      off = torch.cat([torch.zeros(1, dtype=torch.long), torch.bincount(topi.long(), minlength=E).cumsum(0)]).int()
    Fp, Dq, S = lw.ex_up_w.shape[1], lw.ex_down_w.shape[1], 1
    if hn.dtype == torch.bfloat16 and hn.is_cuda:
      # rows per expert decide the kernel as for the framework's other expert layers: the weight-streaming grouped GEMM
      # for decode-sized groups (down projection split over K), gemm_big tiles once the groups are compute-bound
      C = require()
      sh_up, sh_dn = layout_of(lw.ex_up_w) == "stream", layout_of(lw.ex_down_w) == "stream"
      per_expert = T * k / E
      big = sh_up and sh_dn and per_expert >= MOE_BIG_MIN_ROWS and Fp % 256 == 0 and Dq % 256 == 0
      bm, bm_dn, S_dn = moe_tiles(per_expert, E) if big else (0, 0, 0)
      if MOE_PP2:
        bm, bm_dn = ({256: 2256, 192: 2192}.get(t, t) for t in (bm, bm_dn))
      S = S_dn if big else (4 if T * k <= 64 else 2)
      if Fp % (256 * S):
        S = 1
      up = torch.empty(T * k, Fp, dtype=torch.float32, device=dev)
      C.gemm_moe(hn, lw.ex_up_w, up, off, sorted_tok, K.EPI["none"], T, sh_up, 1, bm)
      act = torch.empty(T * k, Fp, dtype=torch.bfloat16, device=dev)
      K.relu2(up, 0, Fp, act)
      y = torch.empty(S * T * k, Dq, dtype=torch.float32, device=dev)
      C.gemm_moe(act, lw.ex_down_w, y, off, None, K.EPI["none"], T, sh_dn, S, bm_dn)
    else:
      # all-fp32 run: one vendor SGEMM pair per expert that has rows (the offsets come to the host)
      y = torch.zeros(T * k, lw.ex_down_w.shape[1], dtype=torch.float32, device=dev)
      offs = off.tolist()
      for e in range(E):
        if offs[e + 1] > offs[e]:
          xe = hn.index_select(0, sorted_tok[offs[e]:offs[e + 1]].long()).float()
          y[offs[e]:offs[e + 1]] = torch.relu(xe @ lw.ex_up_w[e].float().t()).pow(2) @ lw.ex_down_w[e].float().t()
    sh_y = None
    if f.shared_ff:
      act = rows("sh_act", f.shared_ff, lw.down_w.shape[1])
      K.relu2(P, lw.ff_cols["sh_up"][0], f.shared_ff, act)
      sh_y = self._proj(act, lw.down_w)
    out = torch.empty(T, D, dtype=torch.float32, device=dev)
    K.moe_weighted_sum(y, slot_of, topw, k, sh_y, P, lw.ff_cols["sh_gate"][0] if f.shared_ff else 0, out, splits=S)
    return out

  def _forward_postln(self, h: torch.Tensor, inp: StepInputs, adt) -> torch.Tensor:
    """Layers of post-norm blocks on the fp32 stream h (hn: its copy in the GEMMs' operand dtype):
      P = hn @ in_w^T                              the mixer's input projections and the mixer gate in one GEMM
      h <- norm1(alpha h + sigmoid(gate + b) * (mixer(P) @ out_w^T))
      P = hn @ ff_w^T                              feed-forward up (or router, shared up, shared gate) and its gate
      h <- norm2(alpha h + sigmoid(gate + b) * ff(P))
    Returns h (non-last shard) or head(norm(h rows inp.last_idx))."""
    c, w = self.c, self.w
    T, D = h.shape
    Dp = -(-D // 128) * 128
    bufs = {}

    def rows(name: str, live: int, padded: int) -> torch.Tensor:
      key = (name, live, padded)
      if key not in bufs:
        bufs[key] = (torch.zeros if padded > live else torch.empty)(T, padded, dtype=adt, device=h.device)
      return bufs[key]
    hn = rows("hn", D, Dp)
    hn[:, :D] = h.to(adt)
    for j, li in enumerate(self.layer_ids):
      lw = w.layers[li]
      s = lw.spec
      P = self._proj(hn, lw.in_w)
      mix = rows("mix", lw.mix_cols["mix"][1], lw.out_w.shape[1])
      if s.wattn is not None:
        self._window_attn(P, lw, j, inp, mix)
      else:
        self._ssd(P, lw, j, inp, mix)
      y = self._proj(mix, lw.out_w)
      K.gated_postnorm(h, y, P, lw.cols["gate"][0], lw.gate1_b, c.postln_alpha, lw.norm1, c.rms_norm_eps, hn)
      f = s.ffn
      if f is None:
        continue
      P = self._proj(hn, lw.ff_w)
      if f.kind == "polynorm":
        act = rows("act", f.ff, lw.down_w.shape[1])
        K.polynorm_act(P, lw.ff_cols["up"][0], f.ff, lw.act, c.rms_norm_eps, act)
        y = self._proj(act, lw.down_w)
      else:
        y = self._relu2_moe(hn, P, lw, rows)
      K.gated_postnorm(h, y, P, lw.ff_cols["gate"][0], lw.gate2_b, c.postln_alpha, lw.norm2, c.rms_norm_eps, hn)
    if not self.shard.is_last_layer():
      return h
    hl = h.index_select(0, inp.last_idx)
    xn = torch.zeros(hl.shape[0], Dp, dtype=adt, device=h.device)
    K.gated_postnorm(hl, None, None, 0, None, 1.0, w.norm, c.rms_norm_eps, xn)
    return self._proj(xn, w.lm_head)[:, :c.vocab_size]

  # ------------------------------------------------------------------ sandwich blocks (latent attention, gated feed-forwards)
  def _latent_attn(self, P: torch.Tensor, lw, j: int, inp: StepInputs, mix: torch.Tensor, rows) -> None:
    """Attention through the cached latent (one row [latent | rotated key part] per token): norms + RoPE + paged write,
    the query up-projection (queries with a latent of their own), the unrotated query parts absorbed into the latent
    space per head (q_lat = q W_uk), attention over the latent rows, the heads' values out of the latent space
    (o = o_lat W_uv^T), the output gate."""
    a, c, dev = lw.spec.lattn, self.c, P.device
    T, adt = P.shape[0], mix.dtype
    H, dn, dr, dv, R = a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank
    tab = self.rope_tabs.get((a.rot_dims, a.rot_base))
    rd = a.rot_dims if tab is not None else 0
    tab = tab if tab is not None else torch.zeros(1, 0, device=dev)
    qa = rows("qa", a.q_rank, lw.uq_w.shape[1]) if a.q_rank else None
    K.latent_kv_store(P, lw.cols["ckv"][0], R, dr, lw.kv_norm, lw.cols["q"][0], a.q_rank, lw.q_norm, c.rms_norm_eps, rd,
                      a.rot_interleaved, inp.positions, tab, inp.slots, self.kv.k[j], qa)
    Q, q_off = (self._proj(qa, lw.uq_w), 0) if a.q_rank else (P, lw.cols["q"][0])
    qn = torch.empty(H, T, dn, dtype=adt, device=dev)
    qpe = torch.empty(T, H, dr, dtype=adt, device=dev)
    K.latent_q_rope(Q, q_off, H, dn, dr, rd, a.rot_interleaved, inp.positions, tab, qn, qpe)
    q_lat = self._bmm(qn, lw.uk_w)  # [H, T, R]
    o_lat = torch.empty(H, T, R, dtype=adt, device=dev)
    K.latent_attn(q_lat, qpe, self.kv.k[j], inp.block_tables, inp.cu_q, inp.ctx_lens, lw.sink, a.scale, a.window, o_lat,
                  max_qlen=inp.max_qlen)
    o = self._bmm(o_lat, lw.uv_w)  # [H, T, dv]
    K.latent_out_gate(o, P, lw.cols["gate"][0] if a.gate != "none" else 0, {"none": 0, "elem": 1, "head": 2}[a.gate], mix)

  @staticmethod
  def _bmm(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """Per-head products [H, T, k] x [H, k, n] on the vendor library (the CPU path multiplies in fp32)."""
    if x.is_cuda:
      return torch.bmm(x, w)
    return torch.bmm(x.float(), w.float()).to(x.dtype)

  def _silu_moe(self, hn: torch.Tensor, P: torch.Tensor, lw, rows) -> torch.Tensor:
    """SiLU-gated experts chosen by the softmax scores' top-k (weights: the scores as they are) + the ungated shared
    expert -> fp32 [T, D].  Routing on the framework's grouped top-k kernel, experts on the grouped GEMMs (bf16) or per
    expert on the vendor SGEMM (fp32)."""
    f, dev = lw.spec.ffn, P.device
    T, D = hn.shape[0], self.c.hidden_size
    E, k = f.experts, f.top
    r0 = lw.ff_cols["router"][0]
    logits = P[:, r0:r0 + E].contiguous()
    Fp, Dq, S = lw.ex_down_w.shape[2], lw.ex_down_w.shape[1], 1
    if P.is_cuda:
      topw = torch.empty(T * k, dtype=torch.float32, device=dev)
      topi, slot_of, sorted_tok = (torch.empty(T * k, dtype=torch.int32, device=dev) for _ in range(3))
      off = torch.empty(E + 1, dtype=torch.int32, device=dev)
      K.moe_route_ds(logits, None, k, 1, 1, 0, False, False, 1.0, outs=(topw, topi, slot_of, sorted_tok, off))
    else:
      topw, idx = torch.topk(torch.softmax(logits.float(), -1), k, dim=-1)
      topw, topi = topw.reshape(-1), idx.reshape(-1).int()
      order = torch.argsort(topi, stable=True)
      slot_of = torch.empty_like(order)
      slot_of[order] = torch.arange(T * k)
      sorted_tok = (order // k).int()
      off = torch.cat([torch.zeros(1, dtype=torch.long), torch.bincount(topi.long(), minlength=E).cumsum(0)]).int()
    if hn.dtype == torch.bfloat16 and hn.is_cuda:
      C = require()
      sh_up, sh_dn = layout_of(lw.ex_up_w) == "stream", layout_of(lw.ex_down_w) == "stream"
      per_expert = T * k / E
      big = sh_up and sh_dn and per_expert >= MOE_BIG_MIN_ROWS and Fp % 256 == 0 and Dq % 256 == 0
      bm, bm_dn, S_dn = moe_tiles(per_expert, E) if big else (0, 0, 0)
      if MOE_PP2:
        bm, bm_dn = ({256: 2256, 192: 2192}.get(t, t) for t in (bm, bm_dn))
      S = S_dn if big else (4 if T * k <= 64 else 2)
      if Fp % (256 * S):
        S = 1
      act = torch.empty(T * k, Fp, dtype=torch.bfloat16, device=dev)  # silu(gate) * up in the GEMM's epilogue
      C.gemm_moe(hn, lw.ex_up_w, act, off, sorted_tok, K.EPI["silu"], T, sh_up, 1, bm)
      y = torch.empty(S * T * k, Dq, dtype=torch.float32, device=dev)
      C.gemm_moe(act, lw.ex_down_w, y, off, None, K.EPI["none"], T, sh_dn, S, bm_dn)
    else:
      # all-fp32 run (and the CPU path): one vendor SGEMM pair per expert that has rows (the offsets come to the host)
      y = torch.zeros(T * k, Dq, dtype=torch.float32, device=dev)
      offs = off.tolist()
      for e in range(E):
        if offs[e + 1] > offs[e]:
          xe = hn.index_select(0, sorted_tok[offs[e]:offs[e + 1]].long()).float()
          gu = (xe @ lw.ex_up_w[e].float().t()).reshape(xe.shape[0], Fp // 16, 2, 16)  # (gate | up tiles of 16)
          act = (torch.nn.functional.silu(gu[:, :, 0]) * gu[:, :, 1]).reshape(xe.shape[0], Fp)
          y[offs[e]:offs[e + 1]] = act @ lw.ex_down_w[e].float().t()
    sh_y = None
    if f.shared_ff:
      act = rows("sh_act", f.shared_ff, lw.down_w.shape[1])
      K.glu_act(P, lw.ff_cols["sh_gate"][0], lw.ff_cols["sh_up"][0], f.shared_ff, False, 0.0, act)
      sh_y = self._proj(act, lw.down_w)
    out = torch.empty(T, D, dtype=torch.float32, device=dev)
    K.moe_weighted_sum(y, slot_of, topw, k, sh_y, None, 0, out, splits=S)
    return out

  def _forward_sandwich(self, h: torch.Tensor, inp: StepInputs, adt) -> torch.Tensor:
    """Layer runs (a looped layer once per pass, each pass with caches and states of its own) of sandwich blocks on the
    fp32 stream h (hn: the normed sublayer input in the GEMMs' operand dtype):
      pass start:  h <- [h | embedding output] @ loop_in^T + step[pass]       (loop_input "linear")
                   h <- h + embedding output (passes after the first) + step[pass]       ("add")
      P = hn @ in_w^T                    every projection that reads the mixer's input
      h += mult * norm1b(mixer(P) @ out_w^T);  hn = norm2(h)
      P = hn @ ff_w^T                    gate | up, or router | shared expert's projections
      h += mult * norm2b(ff(P));  hn = the next run's norm1(h)
    The norms are RMS norms with a weight, or (norm_kind "layer") layer norms with weight and bias.  Mixers: latent
    attention; differential attention; mlstm; gated attention beside lightning attention, each projected to the width,
    RMS-normed with its own weight and averaged.
    Returns h (non-last shard) or softcap(head(final_norm(h rows inp.last_idx)))."""
    c, w = self.c, self.w
    T, D = h.shape
    Dp = -(-D // 128) * 128
    bufs = {}

    def rows(name: str, live: int, padded: int) -> torch.Tensor:
      key = (name, live, padded)
      if key not in bufs:
        bufs[key] = (torch.zeros if padded > live else torch.empty)(T, padded, dtype=adt, device=h.device)
      return bufs[key]
    hn = rows("hn", D, Dp)
    x0 = None
    if w.loop_in is not None:  # the embedding output in the operand dtype, second half of every pass's input rows
      xx = torch.zeros(T, 2 * Dp, dtype=adt, device=h.device)
      xx[:, Dp:Dp + D] = h.to(adt)
    elif w.loop_step is not None:
      x0 = h.clone()
    runs = self.runs
    eps, mult = c.rms_norm_eps, c.residual_mult
    fresh = True  # hn does not hold this run's normed input yet
    for j, (li, t) in enumerate(runs):
      lw = w.layers[li]
      s = lw.spec
      if t >= 0 and w.loop_in is not None:
        xx[:, :D] = h.to(adt)
        h = self._proj(xx, w.loop_in)[:, :D] + w.loop_step[t]
        fresh = True
      elif t >= 0:
        if t > 0:
          h += x0
        h += w.loop_step[t]
        fresh = True
      if fresh:
        K.sandwich_add_norm(h, None, None, lw.norm1, eps, hn, bn=lw.norm1_b)
      P = self._proj(hn, lw.in_w)
      mix = rows("mix", lw.mix_cols["mix"][1], lw.out_w.shape[1])
      if s.lattn is not None:
        self._latent_attn(P, lw, j, inp, mix, rows)
      elif s.dattn is not None:
        self._diff_attn(P, lw, j, inp, mix)
      elif s.wattn is not None:
        self._window_attn(P, lw, j, inp, mix)
      else:
        self._mlstm(P, lw, j, inp, mix)
      y = self._proj(mix, lw.out_w)
      if s.wattn is not None and s.rec is not None:  # the second mixer of a parallel layer, then the mean of the normed pair
        mix2 = rows("mix2", lw.mix_cols["mix2"][1], lw.out2_w.shape[1])
        self._lightning(P, lw, j, inp, mix2)
        y2 = self._proj(mix2, lw.out2_w)
        y1, y = y, torch.empty(T, D, dtype=torch.float32, device=h.device)
        K.pair_norm_mean(y1, y2, lw.pair_w, eps, y)
      f = s.ffn
      # the norm that follows this run: the next run's input norm unless a pass starts there
      nl = w.layers[runs[j + 1][0]] if j + 1 < len(runs) and runs[j + 1][1] < 0 else None
      nxt, nxt_b = (nl.norm1, nl.norm1_b) if nl is not None else (None, None)
      if f is None:
        K.sandwich_add_norm(h, y, lw.norm1b, nxt, eps, hn, bb=lw.norm1b_b, bn=nxt_b, mult=mult)
      else:
        K.sandwich_add_norm(h, y, lw.norm1b, lw.norm2, eps, hn, bb=lw.norm1b_b, bn=lw.norm2_b, mult=mult)
        P = self._proj(hn, lw.ff_w)
        if f.kind == "clamped_glu":
          act = rows("act", f.ff, lw.down_w.shape[1])
          K.glu_act(P, lw.ff_cols["gate"][0], lw.ff_cols["up"][0], f.ff, True, f.limit, act)
          y = self._proj(act, lw.down_w)
        elif f.kind == "relu2_moe":
          y = self._relu2_moe(hn, P, lw, rows)
        else:
          y = self._silu_moe(hn, P, lw, rows)
        K.sandwich_add_norm(h, y, lw.norm2b, nxt, eps, hn, bb=lw.norm2b_b, bn=nxt_b, mult=mult)
      fresh = nxt is None
    if not self.shard.is_last_layer():
      return h
    hl = h.index_select(0, inp.last_idx)
    xn = torch.zeros(hl.shape[0], Dp, dtype=adt, device=h.device)
    K.sandwich_add_norm(hl, None, None, w.norm, eps, xn, bn=w.norm_b)
    logits = self._proj(xn, w.lm_head)[:, :c.vocab_size]
    if c.logit_softcap > 0:
      logits = torch.tanh(logits / c.logit_softcap) * c.logit_softcap
    return logits

  # ------------------------------------------------------------------ forward
  @torch.inference_mode()
  def forward(self, x: torch.Tensor, inp: StepInputs) -> torch.Tensor:
    """x: token ids [T] (first shard) or hidden [T, D] bf16.  Returns hidden [T, D] (non-last shard)
    or fp32 logits [B, V] of each sequence's last token (last shard)."""
    c, w = self.c, self.w
    if c.is_mixed:
      return self._forward_mixed(x, inp)
    if self.shard.is_first_layer():
      h = K.embedding(x, w.embed)
      if inp.image_embeds is not None:  # LLaVA: projected image features replace the image-token rows
        rows = (x.view(-1) == c.image_token_id).nonzero().view(-1)
        if rows.numel() != inp.image_embeds.shape[0]:
          raise ValueError(f"{rows.numel()} image tokens but {inp.image_embeds.shape[0]} image feature rows")
        h.index_copy_(0, rows, inp.image_embeds.to(h.dtype))
    else:
      h = x.contiguous().clone() if x.dtype == torch.bfloat16 else x.to(torch.bfloat16).contiguous()
    last = self.shard.is_last_layer()
    n = len(self.layer_ids)
    xn, _ = K.rmsnorm(h, w.layers[self.layer_ids[0]].ln1, c.rms_norm_eps) if n else (None, None)
    # batch-1 decode: the split-K reduce + residual + RMSNorm after o_proj / down_proj is deferred into the next
    # GEMM's prologue (ops.linear.PendingNorm); the residual stream then alternates between two row buffers
    fuse = FUSE_NORM and h.is_cuda and h.shape[0] == 1 and not c.is_mla and n > 0
    hb = (h, torch.empty_like(h)) if fuse else None
    other = (lambda t: hb[1] if t is hb[0] else hb[0]) if fuse else (lambda t: None)
    for j, li in enumerate(self.layer_ids):
      lw = w.layers[li]
      if c.is_mla:
        a = self._mla(xn, lw, j, inp)
      else:
        # QKV projection + RoPE + paged KV write (split-K slabs reduced inside the RoPE kernel)
        q = linear_rope_kv(xn, lw.qkv_w, lw.qkv_b, inp.positions, self.cos_sin, inp.slots, self.kv.k[j],
                           self.kv.v[j], c.num_heads, c.num_kv_heads)
        if isinstance(xn, PendingNorm):
          h = xn.dst
        a = self._attention(q, j, inp, defer_merge=fuse and FUSE_MERGE and lw.router is None)
        if not isinstance(a, K.PendingMerge):  # (a pending merge is finished inside o_proj's prologue)
          a = a.view(h.shape[0], c.num_heads * c.head_dim)
      # o_proj + residual + post-attention norm (one fused pass when the projection runs split-K)
      xn = linear_resid_norm(a, lw.o_w, h, lw.ln2, c.rms_norm_eps,
                             defer_to=other(h) if lw.router is None else None)
      if isinstance(xn, PendingNorm):
        h = xn.dst  # gate/up's prologue stores the summed residual there
      # the norm that follows this layer: the next layer's input norm, or the final norm (decode: every row
      # is a sequence's last token) -- fused into the down projection's reduce the same way
      nxt = w.layers[self.layer_ids[j + 1]].ln1 if j + 1 < n else (w.norm if last and inp.decode else None)
      xn = self._mlp(xn, lw, h, nxt, li, defer_to=other(h) if j + 1 < n else None)
    if not last:
      return h
    if not inp.decode or n == 0:
      hl = h.index_select(0, inp.last_idx) if not inp.decode else h
      xn, _ = K.rmsnorm(hl, w.norm, c.rms_norm_eps)
    if self.head_rows is None:
      return linear(xn, w.lm_head, out_dtype=torch.float32)
    # LM head split with another stage (parallel/pipeline.py): logits of vocab rows [0, head_rows) and
    # the normed hidden state the other stage applies the remaining rows to
    return linear(xn, self._head_slice(), out_dtype=torch.float32), xn

  def _head_slice(self) -> torch.Tensor:
    w = self.w.lm_head
    if self._head_cache is None or self._head_cache[0] != self.head_rows:
      # rows [0, r) of the pre-shuffled layout (16-row groups) are a storage prefix: a view, no copy
      hs = w[: self.head_rows]
      if layout_of(w) != "rowmajor":
        hs.xot_layout = layout_of(w)
      self._head_cache = (self.head_rows, hs)
    return self._head_cache[1]


def make_step_inputs(seqs: List[tuple], device, block_width: Optional[int] = None) -> StepInputs:
  """Host helper: seqs = [(positions list, slots list, block_table list, ctx_len)] -> StepInputs."""
  pos, slots, cu, last = [], [], [0], []
  width = block_width or max(1, max(len(s[2]) for s in seqs))
  tables = torch.zeros(len(seqs), width, dtype=torch.int32)
  ctx = torch.zeros(len(seqs), dtype=torch.int32)
  for b, (p, s, bt, n) in enumerate(seqs):
    pos += list(p)
    slots += list(s)
    cu.append(cu[-1] + len(p))
    last.append(cu[-1] - 1)
    tables[b, :len(bt)] = torch.tensor(bt, dtype=torch.int32)
    ctx[b] = n
  qlens = [cu[i + 1] - cu[i] for i in range(len(seqs))]
  return StepInputs(
    positions=torch.tensor(pos, dtype=torch.int32, device=device),
    slots=torch.tensor(slots, dtype=torch.int64, device=device),
    block_tables=tables.to(device),
    ctx_lens=ctx.to(device),
    cu_q=torch.tensor(cu, dtype=torch.int32, device=device),
    last_idx=torch.tensor(last, dtype=torch.int64, device=device),
    max_qlen=max(qlens),
    decode=all(q == 1 for q in qlens),
  )
