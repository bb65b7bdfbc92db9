"""Per-shard weights in the fused device layout, built from HF safetensors or random init.

Device layout per decoder layer (all bf16, nn.Linear [out, in] rows):
  qkv_w  [(H + 2 Hkv) Dh, D]   = cat(q_proj, k_proj, v_proj)     (+ qkv_b for Qwen2)
  o_w    [D, H Dh]
  gu_w   [2F, D]               gate/up interleaved in 16-row tiles (one MFMA n-tile each), so the
                               GEMM epilogue computes silu(gate)*up without another pass
  down_w [D, F]
  ln1, ln2 [D]
MoE (Mixtral): router [E, D], gu_w [E, 2F, D], down_w [E, D, F].
Only this shard's layers are materialised (the reference allocates every shard's full embedding and
LM head, general_mha.py:124-128; here the embedding lives on the first shard and the head on the last).
HF names are kept for loading and checkpointing so any shard checkpoint can be re-partitioned.
Reference parity: load_model_weights_torchtune (llm_utils.py:136-284) — without the q/k permute,
because the RoPE kernel uses the HF rotate-half convention directly.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from pathlib import Path
from typing import Dict, Iterable, Optional

import torch

from ..inference.shard import Shard
from .config import ModelConfig

TILE = 16


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
  """[F, D] x2 -> [2F, D] with rows [g0..g15, u0..u15, g16..g31, u16..u31, ...]."""
  Fd, D = gate.shape
  assert Fd % TILE == 0, "intermediate size must be a multiple of 16"
  return torch.stack([gate.view(Fd // TILE, TILE, D), up.view(Fd // TILE, TILE, D)], dim=1).reshape(2 * Fd, D)


def split_gate_up(gu: torch.Tensor):
  n2, D = gu.shape[-2], gu.shape[-1]
  v = gu.reshape(*gu.shape[:-2], n2 // (2 * TILE), 2, TILE, D)
  return v[..., 0, :, :].reshape(*gu.shape[:-2], n2 // 2, D), v[..., 1, :, :].reshape(*gu.shape[:-2], n2 // 2, D)


@dataclass
class LayerWeights:
  qkv_w: torch.Tensor
  o_w: torch.Tensor
  gu_w: torch.Tensor
  down_w: torch.Tensor
  ln1: torch.Tensor
  ln2: torch.Tensor
  qkv_b: Optional[torch.Tensor] = None
  router: Optional[torch.Tensor] = None  # MoE
  # DeepSeek MLA: qkv_w is the fused A projection [q_a (or q) | kv latent | shared rope key]
  q_ln: Optional[torch.Tensor] = None  # [q_lora_rank]
  kv_ln: Optional[torch.Tensor] = None  # [kv_lora_rank]
  qb_w: Optional[torch.Tensor] = None  # [H (dn + dr), q_lora_rank], rows [all heads' nope | all heads' rope]
  wuk: Optional[torch.Tensor] = None  # [H, dn, kv_lora_rank]  (kv_b_proj's key rows, absorbed into q)
  wuv: Optional[torch.Tensor] = None  # [H, dv, kv_lora_rank]  (kv_b_proj's value rows)
  # DeepSeekMoE
  router_bias: Optional[torch.Tensor] = None  # [E] fp32 selection bias (V3 e_score_correction_bias)
  sh_gu_w: Optional[torch.Tensor] = None  # shared experts, gate/up interleaved [2 Fs, D]
  sh_down_w: Optional[torch.Tensor] = None  # [D, Fs]

  def tensors(self) -> Dict[str, torch.Tensor]:
    return {k: v for k, v in self.__dict__.items() if isinstance(v, torch.Tensor)}


@dataclass
class ShardWeights:
  config: ModelConfig
  shard: Shard
  layers: Dict[int, LayerWeights] = field(default_factory=dict)
  embed: Optional[torch.Tensor] = None  # first shard (and last, when tied)
  norm: Optional[torch.Tensor] = None  # last shard
  norm_b: Optional[torch.Tensor] = None  # last shard, models whose norms are layer norms with a bias
  lm_head: Optional[torch.Tensor] = None  # last shard (aliases embed when tied)
  vision: Optional[Dict[str, torch.Tensor]] = None  # LLaVA tower + projector (first shard), HF names
  # looped layers (config.loop): the pass input mix [Dn, 2 D padded] over [x | embedding output] and the vector added
  # at the start of each pass [times, D] fp32
  loop_in: Optional[torch.Tensor] = None
  loop_step: Optional[torch.Tensor] = None

  def nbytes(self) -> int:
    seen, total = set(), 0
    for t in self.all_tensors():
      if t.data_ptr() not in seen:
        seen.add(t.data_ptr())
        total += t.numel() * t.element_size()
    return total

  def all_tensors(self) -> Iterable[torch.Tensor]:
    for lw in self.layers.values():
      yield from lw.tensors().values()
    for t in (self.embed, self.norm, self.norm_b, self.lm_head, self.loop_in, self.loop_step):
      if t is not None:
        yield t
    if self.vision:
      yield from self.vision.values()

  # ---------------------------------------------------------------- HF naming (checkpoints)
  def to_hf_state_dict(self) -> Dict[str, torch.Tensor]:
    c = self.config
    H, Hkv, Dh = c.num_heads, c.num_kv_heads, c.head_dim
    sd: Dict[str, torch.Tensor] = {}
    from ..ops.rope import permute_qk_rows
    fused = c.model_type == "phi3"  # Phi-3 checkpoints keep qkv_proj / gate_up_proj fused
    for i, lw in self.layers.items():
      p = f"model.layers.{i}."
      if c.is_mla:
        _mla_to_hf(c, lw, p, sd)
        continue
      qkv_w = permute_qk_rows(_rowmajor(lw.qkv_w), H, Hkv, Dh, c.rotary_dim, inverse=True)
      if fused:
        sd[p + "self_attn.qkv_proj.weight"] = qkv_w
      else:
        q, k, v = qkv_w.split([H * Dh, Hkv * Dh, Hkv * Dh], 0)
        sd[p + "self_attn.q_proj.weight"], sd[p + "self_attn.k_proj.weight"], sd[p + "self_attn.v_proj.weight"] = q, k, v
      if lw.qkv_b is not None:
        qkv_b = permute_qk_rows(lw.qkv_b, H, Hkv, Dh, c.rotary_dim, inverse=True)
        qb, kb, vb = qkv_b.split([H * Dh, Hkv * Dh, Hkv * Dh], 0)
        sd[p + "self_attn.q_proj.bias"], sd[p + "self_attn.k_proj.bias"], sd[p + "self_attn.v_proj.bias"] = qb, kb, vb
      sd[p + "self_attn.o_proj.weight"] = _rowmajor(lw.o_w)
      sd[p + "input_layernorm.weight"] = lw.ln1
      sd[p + "post_attention_layernorm.weight"] = lw.ln2
      gu, down = _rowmajor(lw.gu_w), _rowmajor(lw.down_w)
      if c.is_moe:
        sd[p + "block_sparse_moe.gate.weight"] = lw.router
        g, u = split_gate_up(gu)
        for e in range(c.num_experts):
          sd[p + f"block_sparse_moe.experts.{e}.w1.weight"] = g[e]
          sd[p + f"block_sparse_moe.experts.{e}.w3.weight"] = u[e]
          sd[p + f"block_sparse_moe.experts.{e}.w2.weight"] = down[e]
      else:
        g, u = split_gate_up(gu)
        if fused:
          sd[p + "mlp.gate_up_proj.weight"] = torch.cat([g, u], 0)
        else:
          sd[p + "mlp.gate_proj.weight"], sd[p + "mlp.up_proj.weight"] = g, u
        sd[p + "mlp.down_proj.weight"] = down
    if self.embed is not None:
      sd["model.embed_tokens.weight"] = self.embed
    if self.norm is not None:
      sd["model.norm.weight"] = self.norm
    if self.lm_head is not None and not c.tie_word_embeddings:
      sd["lm_head.weight"] = _rowmajor(self.lm_head)
    elif self.lm_head is not None and self.embed is None:
      sd["model.embed_tokens.weight"] = _rowmajor(self.lm_head)  # tied head on a shard without the embedding
    if self.vision:
      sd.update(self.vision)
    return {k: v.contiguous() for k, v in sd.items()}


def _mla_q_order(c: ModelConfig) -> torch.Tensor:
  """Device row r of the q projection <- HF row: all heads' nope dims, then all heads' rope dims with the
  interleaved pairs de-interleaved (ops.rope.interleave_perm)."""
  from ..ops.rope import interleave_perm
  H, dn, dr = c.num_heads, c.qk_nope_head_dim, c.qk_rope_head_dim
  hd = dn + dr
  nope = (torch.arange(H)[:, None] * hd + torch.arange(dn)[None, :]).reshape(-1)
  rope = (torch.arange(H)[:, None] * hd + dn + interleave_perm(dr)[None, :]).reshape(-1)
  return torch.cat([nope, rope])


def _mla_kv_order(c: ModelConfig) -> torch.Tensor:
  from ..ops.rope import interleave_perm
  L = c.kv_lora_rank
  return torch.cat([torch.arange(L), L + interleave_perm(c.qk_rope_head_dim)])


def _mla_from_hf(c: ModelConfig, get, has, p: str) -> dict:
  """HF DeepSeek attention tensors -> device layout fields of LayerWeights."""
  a = p + "self_attn."
  qo = _mla_q_order(c)
  kv_a = get(a + "kv_a_proj_with_mqa.weight")
  kv_a = kv_a.index_select(0, _mla_kv_order(c).to(kv_a.device))
  out = {}
  if c.q_lora_rank:
    q_a = get(a + "q_a_proj.weight")
    out["q_ln"] = get(a + "q_a_layernorm.weight")
    qb = get(a + "q_b_proj.weight")
    out["qb_w"] = qb.index_select(0, qo.to(qb.device)).contiguous()
  else:
    q = get(a + "q_proj.weight")
    q_a = q.index_select(0, qo.to(q.device))
  out["qkv_w"] = torch.cat([q_a, kv_a], 0).contiguous()
  out["kv_ln"] = get(a + "kv_a_layernorm.weight")
  kvb = get(a + "kv_b_proj.weight").view(c.num_heads, c.qk_nope_head_dim + c.v_head_dim, c.kv_lora_rank)
  out["wuk"] = kvb[:, :c.qk_nope_head_dim].contiguous()
  out["wuv"] = kvb[:, c.qk_nope_head_dim:].contiguous()
  out["o_w"] = get(a + "o_proj.weight")
  return out


def _mla_to_hf(c: ModelConfig, lw: "LayerWeights", p: str, sd: Dict[str, torch.Tensor]) -> None:
  a = p + "self_attn."
  qo = torch.argsort(_mla_q_order(c))
  ko = torch.argsort(_mla_kv_order(c))
  A = _rowmajor(lw.qkv_w)
  nq = c.q_lora_rank or c.num_heads * (c.qk_nope_head_dim + c.qk_rope_head_dim)
  q_a, kv_a = A[:nq], A[nq:]
  sd[a + "kv_a_proj_with_mqa.weight"] = kv_a.index_select(0, ko.to(kv_a.device))
  if c.q_lora_rank:
    sd[a + "q_a_proj.weight"] = q_a
    sd[a + "q_a_layernorm.weight"] = lw.q_ln
    qb = _rowmajor(lw.qb_w)
    sd[a + "q_b_proj.weight"] = qb.index_select(0, qo.to(qb.device))
  else:
    sd[a + "q_proj.weight"] = q_a.index_select(0, qo.to(q_a.device))
  sd[a + "kv_a_layernorm.weight"] = lw.kv_ln
  sd[a + "kv_b_proj.weight"] = torch.cat([_rowmajor(lw.wuk), _rowmajor(lw.wuv)], 1).reshape(-1, c.kv_lora_rank)
  sd[a + "o_proj.weight"] = _rowmajor(lw.o_w)
  sd[p + "input_layernorm.weight"] = lw.ln1
  sd[p + "post_attention_layernorm.weight"] = lw.ln2
  gu, down = _rowmajor(lw.gu_w), _rowmajor(lw.down_w)
  g, u = split_gate_up(gu)
  if lw.router is not None:
    m = p + "mlp."
    sd[m + "gate.weight"] = lw.router
    if lw.router_bias is not None:
      sd[m + "gate.e_score_correction_bias"] = lw.router_bias
    for e in range(c.num_experts):
      sd[m + f"experts.{e}.gate_proj.weight"], sd[m + f"experts.{e}.up_proj.weight"] = g[e], u[e]
      sd[m + f"experts.{e}.down_proj.weight"] = down[e]
    if lw.sh_gu_w is not None:
      sg, su = split_gate_up(_rowmajor(lw.sh_gu_w))
      sd[m + "shared_experts.gate_proj.weight"], sd[m + "shared_experts.up_proj.weight"] = sg, su
      sd[m + "shared_experts.down_proj.weight"] = _rowmajor(lw.sh_down_w)
  else:
    sd[p + "mlp.gate_proj.weight"], sd[p + "mlp.up_proj.weight"] = g, u
    sd[p + "mlp.down_proj.weight"] = down


def _rowmajor(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
  """Row-major view of a possibly pre-shuffled device weight (2-D, or 3-D expert stacks), without the zero
  padding a tiled layout may carry (`xot_logical`: see pad_ffn_for_tiles)."""
  logical = getattr(t, "xot_logical", None)
  if logical is not None:
    full = _rowmajor_full(t)
    return full[:logical[0], :logical[1]].contiguous()
  return _rowmajor_full(t)


def _rowmajor_full(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
  if t is not None and getattr(t, "xot_layout", "rowmajor") == "stream8":
    from ..ops.weights_layout import dequant_stream8
    return dequant_stream8(t, t.xot_scale)
  if t is not None and getattr(t, "xot_layout", "rowmajor") == "stream_t":  # per-head shuffled W^T (MLA W_UK)
    from ..ops.weights_layout import unshuffle_from_stream
    return torch.stack([unshuffle_from_stream(t[h]).t() for h in range(t.shape[0])])
  if t is None or getattr(t, "xot_layout", "rowmajor") != "stream":
    return t
  from ..ops.weights_layout import unshuffle_from_stream
  if t.dim() == 3:
    return torch.stack([unshuffle_from_stream(t[e]) for e in range(t.shape[0])])
  return unshuffle_from_stream(t)


def expert(t: torch.Tensor, e: int) -> torch.Tensor:
  """Expert e's [rows, K] weight, keeping the storage-layout tag of the stack."""
  v = t[e]
  if hasattr(t, "xot_layout"):
    v.xot_layout = t.xot_layout
  return v


def _pad_to(t: torch.Tensor, shape) -> torch.Tensor:
  """Zero-pad the trailing rows / columns of a 2-D tensor up to `shape`."""
  return torch.nn.functional.pad(t, (0, shape[1] - t.shape[1], 0, shape[0] - t.shape[0]))


def pad_ffn_for_tiles(lw: "LayerWeights") -> None:
  """A dense SwiGLU whose intermediate size F is not a multiple of 128 (DeepSeek-V2-Lite's first layer:
  10944) cannot take the down projection (K = F) on the 128-deep pre-shuffled tiles.  Pad F to F' = 128k
  with zero features instead: gate/up gain zero rows (interleaved groups past F, so silu(0) * 0 = 0 columns
  in the activation) and down gains zero columns -- the same products, every GEMM on the tiled kernels.
  `xot_logical` records the unpadded shape for _rowmajor / assign_weight (training, export)."""
  gu, down = lw.gu_w, lw.down_w
  if gu is None or down is None or gu.dim() != 2 or lw.router is not None or not gu.is_cuda:
    return
  if getattr(gu, "xot_layout", "rowmajor") != "rowmajor" or getattr(down, "xot_layout", "rowmajor") != "rowmajor":
    return
  F = down.shape[1]
  if F % 128 == 0 or F % TILE or gu.shape[0] != 2 * F:
    return
  Fp = -(-F // 128) * 128
  lw.gu_w = _pad_to(gu, (2 * Fp, gu.shape[1]))  # pad rows after the last interleaved (gate, up) group pair
  lw.down_w = _pad_to(down, (down.shape[0], Fp))
  lw.gu_w.xot_logical, lw.down_w.xot_logical = tuple(gu.shape), tuple(down.shape)


def prepare_for_decode(sw: "ShardWeights", keep_rowmajor: Iterable[str] = (), fp8: bool = False) -> "ShardWeights":
  """Convert the projection weights of a GPU shard to the pre-shuffled stream layout (in place).
  The embedding stays row-major (it is gathered); a tied LM head gets its own shuffled copy.
  `keep_rowmajor` names projections ("qkv", "o", "gu", "down") left row-major: at decode batches of
  ~256 rows hipBLASLt beats the stream GEMM on the wide qkv / gate-up shapes, while the stream GEMM
  keeps winning on o / down (tools/bench_gemm_m.py, profiles/bench_gemm_m_*.json)."""
  keep = set(keep_rowmajor)
  from ..ops.weights_layout import can_shuffle, shuffle_for_stream
  from ..ops.linear import to_stream8_layout
  if sw.embed is not None and not sw.embed.is_cuda:
    return sw
  if sw.lm_head is None and not sw.layers:
    return sw

  def conv(t):
    if t is None or not t.is_cuda or getattr(t, "xot_layout", "rowmajor") == "stream":
      return t
    if t.dim() == 3:
      if not all(can_shuffle(t[e]) for e in range(t.shape[0])):
        return t
      out = torch.empty_like(t)
      for e in range(t.shape[0]):
        out[e] = shuffle_for_stream(t[e])
    else:
      if not can_shuffle(t):
        return t
      out = shuffle_for_stream(t)
    out.xot_layout = "stream"
    return out

  def conv8(t):  # fp8=True: the dense projections become weight-only FP8 (experts, latent and LM head stay bf16)
    if t is None or not t.is_cuda or t.dim() != 2 or getattr(t, "xot_layout", "rowmajor") != "rowmajor":
      return conv(t)
    return to_stream8_layout(t) if can_shuffle(t) else t

  def conv_bat(t, transpose: bool):
    """MLA absorbed projections for gemm_batched (N % 128 == 0): W_UV [H, dv, L] per head shuffled ("stream");
    W_UK [H, dn, L] -> per head shuffle(W_UK[h]^T) [H, L, dn] ("stream_t"), so q_lat = q_nope . W_UK is Y = X W^T."""
    if t is None or not t.is_cuda or getattr(t, "xot_layout", "rowmajor") != "rowmajor":
      return t
    ws = [t[h].t() if transpose else t[h] for h in range(t.shape[0])]
    if not all(can_shuffle(w) and w.shape[0] % 128 == 0 for w in ws):
      return t
    out = torch.stack([shuffle_for_stream(w.contiguous()) for w in ws])
    out.xot_layout = "stream_t" if transpose else "stream"
    return out

  if sw.config.is_mixed:  # fused projections of mixed-layer models (bf16 runs; an fp32 run keeps vendor SGEMM layouts)
    def wide(t):  # (the tall-M tiles start at 128 output columns: narrower projections stay row-major)
      return conv(t) if t is not None and t.shape[0] >= 128 else t
    for lw in sw.layers.values():
      if lw.in_w.dtype == torch.bfloat16:
        lw.in_w, lw.out_w, lw.down_w, lw.ff_w = wide(lw.in_w), wide(lw.out_w), wide(lw.down_w), wide(lw.ff_w)
        lw.uq_w, lw.out2_w = wide(lw.uq_w), wide(lw.out2_w)
        lw.ex_up_w, lw.ex_down_w = conv(lw.ex_up_w), conv(lw.ex_down_w)  # experts: shuffled per expert
    if sw.lm_head is not None and sw.lm_head.dtype == torch.bfloat16:
      sw.lm_head = wide(sw.lm_head)
    if sw.loop_in is not None and sw.loop_in.dtype == torch.bfloat16:
      sw.loop_in = wide(sw.loop_in)
    return sw

  proj = conv8 if fp8 else conv

  def keep_logical(new, old):  # a converted weight keeps the padded tensor's logical shape
    if new is not old and getattr(old, "xot_logical", None) is not None:
      new.xot_logical = old.xot_logical
    return new

  for lw in sw.layers.values():
    if ("gu" not in keep and "down" not in keep) or fp8:
      pad_ffn_for_tiles(lw)
    g0, d0 = lw.gu_w, lw.down_w
    lw.qb_w, lw.sh_gu_w, lw.sh_down_w = conv(lw.qb_w), conv(lw.sh_gu_w), conv(lw.sh_down_w)
    lw.wuk, lw.wuv = conv_bat(lw.wuk, True), conv_bat(lw.wuv, False)  # the absorbed MLA projections run on gemm_batched
    if "qkv" not in keep or fp8:
      lw.qkv_w = proj(lw.qkv_w)
    if "o" not in keep or fp8:
      lw.o_w = proj(lw.o_w)
    if "gu" not in keep or fp8:
      lw.gu_w = proj(lw.gu_w)
    if "down" not in keep or fp8:
      lw.down_w = proj(lw.down_w)
    lw.gu_w, lw.down_w = keep_logical(lw.gu_w, g0), keep_logical(lw.down_w, d0)
  if sw.lm_head is not None:
    sw.lm_head = conv(sw.lm_head)  # a tied head becomes a separate shuffled copy; embed stays row-major
  return sw


@torch.no_grad()
def assign_weight(dst: Optional[torch.Tensor], src: torch.Tensor) -> None:
  """Write a row-major `src` into `dst` IN PLACE, honouring dst's storage layout (pre-shuffled or
  not).  In-place matters: captured HIP graphs hold the addresses of the inference weights."""
  if dst is None:
    return
  if getattr(dst, "xot_layout", "rowmajor") == "stream8":  # re-quantize (new row scales, same storage)
    from ..ops.weights_layout import quantize_fp8_rows, shuffle_for_stream8
    if getattr(dst, "xot_logical", None) is not None:
      src = _pad_to(src, dst.shape)
    q, sc = quantize_fp8_rows(src.to(dst.device))
    dst.copy_(shuffle_for_stream8(q))
    dst.xot_scale.copy_(sc)
    return
  src = src.to(device=dst.device, dtype=dst.dtype)
  if getattr(dst, "xot_logical", None) is not None and tuple(src.shape) != tuple(dst.shape):
    src = _pad_to(src, dst.shape)
  if getattr(dst, "xot_layout", "rowmajor") == "stream_t":
    from ..ops.weights_layout import shuffle_for_stream
    for h in range(dst.shape[0]):
      dst[h].copy_(shuffle_for_stream(src[h].t().contiguous()))
  elif getattr(dst, "xot_layout", "rowmajor") == "stream":
    from ..ops.weights_layout import shuffle_for_stream
    if dst.dim() == 3:
      for e in range(dst.shape[0]):
        dst[e].copy_(shuffle_for_stream(src[e]))
    else:
      dst.copy_(shuffle_for_stream(src))
  else:
    dst.copy_(src)


@torch.no_grad()
def copy_weights_into(dst: "ShardWeights", src: "ShardWeights") -> None:
  """Copy every tensor of the row-major `src` shard into the live inference shard `dst` in place."""
  for i, lw in dst.layers.items():
    s = src.layers[i]
    for name in ("qkv_w", "o_w", "gu_w", "down_w", "ln1", "ln2", "qkv_b", "router", "q_ln", "kv_ln", "qb_w", "wuk",
                 "wuv", "router_bias", "sh_gu_w", "sh_down_w"):
      if getattr(lw, name) is not None and getattr(s, name) is not None:
        assign_weight(getattr(lw, name), getattr(s, name))
  if dst.embed is not None and src.embed is not None:
    assign_weight(dst.embed, src.embed)
  if dst.norm is not None and src.norm is not None:
    assign_weight(dst.norm, src.norm)
  if dst.lm_head is not None and dst.lm_head is not dst.embed:
    head = src.lm_head if src.lm_head is not None else src.embed
    if head is not None:
      assign_weight(dst.lm_head, head)


def _needs_embed(c: ModelConfig, s: Shard) -> bool:
  return s.is_first_layer() or (s.is_last_layer() and c.tie_word_embeddings)


# -------------------------------------------------------------------- random init
def _normal(shape, g: torch.Generator, std: float, dev: torch.device, dtype) -> torch.Tensor:
  """N(0, std) of `shape` from generator g; every random weight (and random_head_rows) draws through here, so a
  shard's rows are the same whichever function made them.  (Drawing CPU bf16 weights in fp32 and rounding is ~3x
  faster, but it changes every value, and the exact-equality training tests are pinned to these.)"""
  return torch.empty(shape, device=dev, dtype=dtype).normal_(0.0, std, generator=g)


def random_weights(c: ModelConfig, shard: Shard, device: torch.device | str = "cpu", dtype=torch.bfloat16,
                   seed: int = 0, std: float = 0.02) -> ShardWeights:
  """Deterministic per-layer random weights: layer i is identical whichever shard holds it, so a
  pipeline split reproduces the unsplit model exactly (the split-vs-full equivalence tests)."""
  dev = torch.device(device)
  if c.is_mixed:
    tensors = random_mixed_tensors(c, seed)
    return mixed_weights(c, shard, tensors.__getitem__, dev, dtype)
  D, Fd, E = c.hidden_size, c.intermediate_size, c.num_experts

  def gen(tag: int):
    g = torch.Generator(device=dev)
    g.manual_seed(seed * 1_000_003 + tag)
    return g

  def normal(shape, g, s=std):
    return _normal(shape, g, s, dev, dtype)

  def norm_w(g):
    return (1.0 + torch.empty(D, device=dev, dtype=torch.float32).normal_(0.0, 0.05, generator=g)).to(dtype)

  def vec(n, g):
    return (1.0 + torch.empty(n, device=dev, dtype=torch.float32).normal_(0.0, 0.05, generator=g)).to(dtype)

  sw = ShardWeights(c, shard)
  for i in shard.layers():
    g = gen(1000 + i)
    out_std = std / (2 * c.num_layers) ** 0.5  # GPT-2 style residual-branch scaling keeps deep stacks stable
    moe = c.moe_layer(i)
    Fl = c.expert_dim if moe else Fd
    El = E if moe else 0
    lw = LayerWeights(
      qkv_w=normal((c.qkv_size, D), g),
      o_w=normal((D, c.num_heads * (c.v_head_dim if c.is_mla else c.head_dim)), g, out_std),
      gu_w=normal((El, 2 * Fl, D) if El else (2 * Fl, D), g),
      down_w=normal((El, D, Fl) if El else (D, Fl), g, out_std),
      ln1=norm_w(g),
      ln2=norm_w(g),
      qkv_b=normal((c.qkv_size,), g) if c.attention_bias and not c.is_mla else None,
      router=normal((El, D), g, 0.1) if El else None,
    )
    if c.is_mla:
      H, L = c.num_heads, c.kv_lora_rank
      if c.q_lora_rank:
        lw.q_ln = vec(c.q_lora_rank, g)
        lw.qb_w = normal((H * (c.qk_nope_head_dim + c.qk_rope_head_dim), c.q_lora_rank), g)
      lw.kv_ln = vec(L, g)
      lw.wuk = normal((H, c.qk_nope_head_dim, L), g)
      lw.wuv = normal((H, c.v_head_dim, L), g)
    if moe and c.scoring_func == "sigmoid":
      lw.router_bias = torch.empty(El, device=dev, dtype=torch.float32).normal_(0.0, 0.01, generator=g)
    if moe and c.n_shared_experts:
      Fs = c.n_shared_experts * c.expert_dim
      lw.sh_gu_w = normal((2 * Fs, D), g)
      lw.sh_down_w = normal((D, Fs), g, out_std)
    sw.layers[i] = lw
  if _needs_embed(c, shard):
    sw.embed = normal((c.vocab_size, D), gen(1))
  if shard.is_last_layer():
    sw.norm = norm_w(gen(2))
    sw.lm_head = sw.embed if c.tie_word_embeddings else normal((c.vocab_size, D), gen(3))
  if c.vision and shard.is_first_layer():
    from .vision import random_vision
    sw.vision = random_vision(c, dev, dtype, seed=seed)
  return sw


def random_head_rows(c: ModelConfig, rows_from: int, device: torch.device | str = "cpu", dtype=torch.bfloat16,
                     seed: int = 0, std: float = 0.02) -> torch.Tensor:
  """Rows [rows_from, V) of the LM head random_weights gives the last shard (same generator stream, so
  a stage holding only these rows computes exactly the full head's logits for them)."""
  dev = torch.device(device)
  g = torch.Generator(device=dev)
  g.manual_seed(seed * 1_000_003 + (1 if c.tie_word_embeddings else 3))
  full = _normal((c.vocab_size, c.hidden_size), g, std, dev, dtype)
  return full[rows_from:].clone()


# -------------------------------------------------------------------- HF safetensors
def _weight_map(model_dir: Path) -> Dict[str, str]:
  idx = model_dir / "model.safetensors.index.json"
  if idx.exists():
    return json.loads(idx.read_text())["weight_map"]
  files = sorted(model_dir.glob("*.safetensors"))
  if not files:
    raise FileNotFoundError(f"no safetensors in {model_dir}")
  from safetensors import safe_open
  wm = {}
  for f in files:
    with safe_open(str(f), framework="pt") as sf:
      for k in sf.keys():
        wm[k] = f.name
  return wm


_PREFIXES = (("language_model.model.", "model."), ("language_model.lm_head.", "lm_head."),
             ("model.language_model.", "model."), ("model.vision_tower.", "vision_tower."),
             ("model.multi_modal_projector.", "multi_modal_projector."), ("vision_tower.vision_model.", "vision_tower."))


def canonical_name(k: str) -> str:
  """One name per tensor across checkpoint flavours: LLaVA's `language_model.model.*` (hub) /
  `model.language_model.*` (transformers 5) read as the plain LM's `model.*`, the hub's
  `vision_tower.vision_model.*` as `vision_tower.*`."""
  changed = True
  while changed:
    changed = False
    for a, b in _PREFIXES:
      if k.startswith(a):
        k, changed = b + k[len(a):], True
  return k


def needed_files(model_dir: Path, c: ModelConfig, shard: Shard) -> set:
  """Safetensors files that hold this shard's tensors (for the downloader's allow patterns too)."""
  wm = {canonical_name(k): v for k, v in _weight_map(model_dir).items()}
  want = set()
  for name, fname in wm.items():
    if (name.startswith("vision_tower.") or name.startswith("multi_modal_projector.")) and shard.is_first_layer():
      want.add(fname)
    elif name.startswith("model.layers."):
      if int(name.split(".")[2]) in shard.layers():
        want.add(fname)
    elif name.startswith("model.embed_tokens") and _needs_embed(c, shard):
      want.add(fname)
    elif (name.startswith("model.norm") or name.startswith("lm_head")) and shard.is_last_layer():
      want.add(fname)
  return want


def load_hf_weights(model_dir: str | Path, c: ModelConfig, shard: Shard, device="cpu", dtype=torch.bfloat16) -> ShardWeights:
  """Read only this shard's tensors (mmap'd safetensors, one tensor at a time) into the fused layout."""
  from safetensors import safe_open
  model_dir = Path(model_dir)
  if c.is_mixed:
    return load_mixed_weights(model_dir, c, shard, device, dtype)
  raw = _weight_map(model_dir)
  wm = {canonical_name(k): (k, f) for k, f in raw.items()}
  handles = {}

  def get(name: str, dt: Optional[torch.dtype] = None) -> torch.Tensor:
    key, fname = wm[name]
    if fname not in handles:
      handles[fname] = safe_open(str(model_dir / fname), framework="pt")
    return handles[fname].get_tensor(key).to(device=device, dtype=dt or dtype)

  def has(name: str) -> bool:
    return name in wm

  from ..ops.rope import permute_qk_rows
  H, Hkv, Dh, R = c.num_heads, c.num_kv_heads, c.head_dim, c.rotary_dim
  sw = ShardWeights(c, shard)
  for i in shard.layers():
    p = f"model.layers.{i}."
    if c.is_mla:
      sw.layers[i] = _load_deepseek_layer(c, i, p, get, has)
      continue
    if has(p + "self_attn.qkv_proj.weight"):  # Phi-3: fused [q; k; v]
      qkv = get(p + "self_attn.qkv_proj.weight")
    else:
      qkv = torch.cat([get(p + f"self_attn.{n}_proj.weight") for n in "qkv"], 0)
    qkv = permute_qk_rows(qkv, H, Hkv, Dh, R)  # partial rotary: HF dim order -> the kernels' pair order
    qkv_b = None
    if has(p + "self_attn.q_proj.bias"):
      qkv_b = permute_qk_rows(torch.cat([get(p + f"self_attn.{n}_proj.bias") for n in "qkv"], 0), H, Hkv, Dh, R)
    if c.is_moe:
      pm = p + "block_sparse_moe."
      gu = torch.stack([interleave_gate_up(get(pm + f"experts.{e}.w1.weight"), get(pm + f"experts.{e}.w3.weight"))
                        for e in range(c.num_experts)])
      down = torch.stack([get(pm + f"experts.{e}.w2.weight") for e in range(c.num_experts)])
      router = get(pm + "gate.weight")
    else:
      if has(p + "mlp.gate_up_proj.weight"):  # Phi-3: fused [gate; up]
        gate, up = get(p + "mlp.gate_up_proj.weight").chunk(2, 0)
      else:
        gate, up = get(p + "mlp.gate_proj.weight"), get(p + "mlp.up_proj.weight")
      gu = interleave_gate_up(gate, up)
      down = get(p + "mlp.down_proj.weight")
      router = None
    sw.layers[i] = LayerWeights(qkv.contiguous(), get(p + "self_attn.o_proj.weight"), gu.contiguous(), down,
                                get(p + "input_layernorm.weight"), get(p + "post_attention_layernorm.weight"), qkv_b,
                                router)
  if _needs_embed(c, shard):
    sw.embed = get("model.embed_tokens.weight")
  if shard.is_last_layer():
    sw.norm = get("model.norm.weight")
    if has("lm_head.weight") and not c.tie_word_embeddings:
      sw.lm_head = get("lm_head.weight")
    else:
      sw.lm_head = sw.embed
  if c.vision and shard.is_first_layer():
    from .vision import vision_names
    sw.vision = {n: get(n) for n in vision_names(c.vision)}
  return sw


def _load_deepseek_layer(c: ModelConfig, i: int, p: str, get, has) -> LayerWeights:
  f = _mla_from_hf(c, get, has, p)
  m = p + "mlp."
  lw = LayerWeights(f["qkv_w"], f["o_w"], None, None, get(p + "input_layernorm.weight"),
                    get(p + "post_attention_layernorm.weight"), None, None, f.get("q_ln"), f["kv_ln"], f.get("qb_w"),
                    f["wuk"], f["wuv"])
  if c.moe_layer(i):
    lw.gu_w = torch.stack([interleave_gate_up(get(m + f"experts.{e}.gate_proj.weight"),
                                              get(m + f"experts.{e}.up_proj.weight")) for e in range(c.num_experts)])
    lw.down_w = torch.stack([get(m + f"experts.{e}.down_proj.weight") for e in range(c.num_experts)])
    lw.router = get(m + "gate.weight")
    if has(m + "gate.e_score_correction_bias"):
      lw.router_bias = get(m + "gate.e_score_correction_bias", torch.float32)
    elif c.scoring_func == "sigmoid":
      lw.router_bias = torch.zeros(c.num_experts, dtype=torch.float32, device=lw.router.device)
    if c.n_shared_experts:
      lw.sh_gu_w = interleave_gate_up(get(m + "shared_experts.gate_proj.weight"),
                                      get(m + "shared_experts.up_proj.weight")).contiguous()
      lw.sh_down_w = get(m + "shared_experts.down_proj.weight")
  else:
    lw.gu_w = interleave_gate_up(get(m + "gate_proj.weight"), get(m + "up_proj.weight")).contiguous()
    lw.down_w = get(m + "down_proj.weight")
  return lw


def from_hf_state_dict(sd: Dict[str, torch.Tensor], c: ModelConfig, shard: Shard, device="cpu",
                       dtype=torch.bfloat16) -> ShardWeights:
  """Inverse of ShardWeights.to_hf_state_dict (used by checkpoint resume)."""
  import tempfile
  from safetensors.torch import save_file
  with tempfile.TemporaryDirectory() as d:
    save_file({k: v.contiguous() for k, v in sd.items()}, os.path.join(d, "model.safetensors"))
    return load_hf_weights(d, c, shard, device, dtype)


# -------------------------------------------------------------------- layers of differing mixers (Tarepel)
def _up(n: int, m: int) -> int:
  return -(-n // m) * m


@dataclass
class MixedLayerWeights:
  """One layer of a mixed-layer model (config.MixedLayerSpec) in the device layout.

  Every projection that reads the layer's one normed input is a row block of `in_w` [Np, Dp] (one GEMM per layer):
  `cols[name] = (offset, size)` addresses its slice of the fp32 result.  The mixers' outputs are concatenated along
  K into one row buffer for `out_w` [Dn, Kp] = [attention o | recurrence o]; `down_w` [Dn, Fp] is the feed-forward's
  down projection.  Rows / columns are zero-padded to the GEMM tiles (Np, Dn: 64; Dp, Kp, Fp: 128).  Projection
  weights have the compute dtype (bf16, or fp32 for an all-fp32 run); everything a norm, a score or a recurrence
  reads is fp32."""
  spec: object
  in_w: torch.Tensor
  cols: Dict[str, tuple]
  out_w: torch.Tensor
  mix_cols: Dict[str, tuple]  # "attn" / "rec": (offset, size) in the mixers' output row
  norm_g: Optional[torch.Tensor] = None  # [1] fp32 (parallel blocks)
  ls1: Optional[torch.Tensor] = None  # [D] fp32
  ls2: Optional[torch.Tensor] = None
  down_w: Optional[torch.Tensor] = None
  attn_pb: Optional[torch.Tensor] = None  # [H] fp32
  conv_w: Optional[torch.Tensor] = None  # [2 G d + H dv, taps] fp32 (q | k | v channels)
  A_log: Optional[torch.Tensor] = None
  dt_bias: Optional[torch.Tensor] = None
  rec_norm: Optional[torch.Tensor] = None  # [dv] fp32
  a2_w: Optional[torch.Tensor] = None  # [H d, rank] fp32
  a2_b: Optional[torch.Tensor] = None
  router: Optional[torch.Tensor] = None  # (dense feed-forward only; kept for code that asks)
  # post-norm blocks (config.block "postln"): `in_w` = [the mixer's input projections | the mixer gate], a second
  # fused projection `ff_w` = [feed-forward up (or router | shared up | shared gate) | the feed-forward gate] reads the
  # stream after the first norm (`ff_cols` addresses its result); out_w is the mixer's output projection, down_w the
  # dense (or shared expert's) down projection
  norm1: Optional[torch.Tensor] = None  # [D] fp32 weights of the norms after the mixer / the feed-forward
  norm2: Optional[torch.Tensor] = None
  gate1_b: Optional[torch.Tensor] = None  # [D] fp32 biases of the sublayer gates
  gate2_b: Optional[torch.Tensor] = None
  in_b: Optional[torch.Tensor] = None  # [in_w rows] fp32: q / k / v biases at their columns, zero elsewhere
  sink: Optional[torch.Tensor] = None  # [H] fp32
  conv_b: Optional[torch.Tensor] = None  # [C] fp32
  skip_d: Optional[torch.Tensor] = None  # [H] fp32 (SSD: D)
  ssd_norm: Optional[torch.Tensor] = None  # [inner] fp32
  ff_w: Optional[torch.Tensor] = None
  ff_cols: Optional[Dict[str, tuple]] = None
  act: Optional[torch.Tensor] = None  # [4] fp32 PolyNorm coefficients
  router_b: Optional[torch.Tensor] = None  # [E] fp32
  ex_up_w: Optional[torch.Tensor] = None  # [E, Fp, Dp] experts' up projections ([E, 2 Fp, Dp]: gate / up rows interleaved by 16)
  ex_down_w: Optional[torch.Tensor] = None  # [E, Dq, Fp]
  # sandwich blocks (config.block "sandwich"): norm1 / norm2 weigh the sublayers' inputs, norm1b / norm2b their
  # results; latent attention: `in_w` = [q (or the query latent) | kv latent | rotated key part | output gate]
  norm1b: Optional[torch.Tensor] = None  # [D] fp32
  norm2b: Optional[torch.Tensor] = None
  kv_norm: Optional[torch.Tensor] = None  # [kv_rank] fp32
  q_norm: Optional[torch.Tensor] = None  # [q_rank] fp32
  uq_w: Optional[torch.Tensor] = None  # [H (dim + rot_dim) padded, q_rank padded]
  uk_w: Optional[torch.Tensor] = None  # [H, dim, kv_rank]: q_lat = q_unrotated . W_uk per head
  uv_w: Optional[torch.Tensor] = None  # [H, kv_rank, vdim]: o = o_lat . W_uv^T per head (stored transposed)
  # sandwich blocks with layer norms: the four norms' biases; differential attention: `in_w` = [q (heads regrouped as
  # kv head, map, head of the group; rotary dims in pair order) | k | v | one gate per head], lam = the layer's
  # lambda; mlstm: [q | k | v | output gate | input gate | forget gate] and gate_b = [i bias | f bias]; a parallel layer:
  # [attention q | k | v | gate | lightning q | k | v | gate], two output projections (out_w: attention, out2_w:
  # lightning) and pair_w [2, D] = the weights of the norms over their results; decay [H] = lightning's decays
  norm1_b: Optional[torch.Tensor] = None  # [D] fp32
  norm1b_b: Optional[torch.Tensor] = None
  norm2_b: Optional[torch.Tensor] = None
  norm2b_b: Optional[torch.Tensor] = None
  out2_w: Optional[torch.Tensor] = None
  pair_w: Optional[torch.Tensor] = None
  decay: Optional[torch.Tensor] = None
  gate_b: Optional[torch.Tensor] = None
  lam: float = 0.0

  def tensors(self) -> Dict[str, torch.Tensor]:
    return {k: v for k, v in self.__dict__.items() if isinstance(v, torch.Tensor)}


def mixed_layer_names(spec, p: str) -> Dict[str, list]:
  """Checkpoint tensor names of one layer: {"in": [(column name, tensor)], "out": [(mix name, tensor)], ...}."""
  if spec.kind == "parallel":
    a, r = p + "mix.left.", p + "mix.right."
    return {"in": [("aq", a + "q"), ("ak", a + "k"), ("rq", r + "q"), ("rk", r + "k"), ("rv", r + "v"), ("rg", r + "g"),
                   ("rb", r + "b"), ("ra", r + "a")],
            "out": [("attn", a + "o"), ("rec", r + "o")], "pb": a + "pb", "conv": [r + "q.conv", r + "k.conv", r + "v.conv"],
            "A_log": r + "A_log", "dt_bias": r + "dt_bias", "rec_norm": r + "norm"}
  m = p + "mix."
  return {"in": [("rq", m + "q"), ("rk", m + "k"), ("rv", m + "v"), ("rg", m + "g"), ("ra1", m + "a1")],
          "out": [("rec", m + "o")], "rec_norm": m + "norm", "a2": m + "a2", "a2_b": m + "a2.b"}


def build_mixed_layer(spec, get, p: str, D: int, device, dtype) -> MixedLayerWeights:
  """Assemble one layer from `get(name) -> fp32 CPU tensor` (a checkpoint reader or a random generator)."""
  names = mixed_layer_names(spec, p)
  blocks = [(n, get(t)) for n, t in names["in"]]
  if spec.ff:
    blocks += [("gate", get(p + "mlp.gate")), ("up", get(p + "mlp.up"))]
  cols, off = {}, 0
  for n, w in blocks:
    cols[n] = (off, w.shape[0])
    off += w.shape[0]
  Dp = _up(D, 128)
  in_w = torch.zeros(_up(off, 64), Dp)
  in_w[:off, :D] = torch.cat([w for _, w in blocks], 0)
  outs = [(n, get(t)) for n, t in names["out"]]
  mix_cols, k = {}, 0
  for n, w in outs:
    mix_cols[n] = (k, w.shape[1])
    k += w.shape[1]
  out_w = torch.zeros(_up(D, 64), _up(k, 128))
  out_w[:D, :k] = torch.cat([w for _, w in outs], 1)

  def dev(t, dt=torch.float32):
    return t.to(device=device, dtype=dt).contiguous()
  lw = MixedLayerWeights(spec, dev(in_w, dtype), cols, dev(out_w, dtype), mix_cols, dev(get(p + "norm1").reshape(1)),
                         dev(get(p + "ls1")))
  if spec.ff:
    down = get(p + "mlp.down")
    dw = torch.zeros(_up(D, 64), _up(spec.ff, 128))
    dw[:D, :spec.ff] = down
    lw.down_w, lw.ls2 = dev(dw, dtype), dev(get(p + "ls2"))
  if "pb" in names:
    lw.attn_pb = dev(get(names["pb"]))
  if "conv" in names:
    lw.conv_w = dev(torch.cat([get(n) for n in names["conv"]], 0))
    lw.A_log, lw.dt_bias = dev(get(names["A_log"])), dev(get(names["dt_bias"]))
  if "a2" in names:
    lw.a2_w, lw.a2_b = dev(get(names["a2"])), dev(get(names["a2_b"]))
  lw.rec_norm = dev(get(names["rec_norm"]))
  return lw


def _fused_rows(blocks, D: int, row_mult: int = 64):
  """[(name, [n_i, D] tensor)] -> (zero-padded [Np, Dp] matrix, {name: (row offset, rows)})."""
  cols, off = {}, 0
  for n, w in blocks:
    cols[n] = (off, w.shape[0])
    off += w.shape[0]
  m = torch.zeros(_up(max(off, 1), row_mult), _up(D, 128))
  if off:
    m[:off, :D] = torch.cat([w for _, w in blocks], 0)
  return m, cols


def _pad2(w: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
  out = torch.zeros(rows, cols)
  out[:w.shape[0], :w.shape[1]] = w
  return out


def build_postln_layer(spec, get, p: str, D: int, device, dtype) -> MixedLayerWeights:
  """One post-norm layer (window attention or SSD mixer, PolyNorm or relu^2-MoE feed-forward) from `get(name)`."""
  def dev(t, dt=torch.float32):
    return t.to(device=device, dtype=dt).contiguous()
  m = p + "mix."
  a, sd, f = spec.wattn, spec.ssd, spec.ffn
  blocks, bias = [], {}
  if a is not None:
    names = ["q"] if a.kv_from >= 0 else ["q", "k", "v"]
    blocks = [(n, get(m + n)) for n in names]
    if a.bias:
      bias = {n: get(m + n + ".b") for n in names}
    out = get(m + "o")
  else:
    blocks = [("in", get(m + "in"))]
    out = get(m + "o")
  blocks.append(("gate", get(p + "rg1")))
  in_w, cols = _fused_rows(blocks, D)
  lw = MixedLayerWeights(spec, dev(in_w, dtype), cols, dev(_pad2(out, _up(D, 64), _up(out.shape[1], 128)), dtype),
                         {"mix": (0, out.shape[1])})
  lw.norm1, lw.gate1_b = dev(get(p + "norm1")), dev(get(p + "rg1.b"))
  if bias:
    b = torch.zeros(in_w.shape[0])
    for n, t in bias.items():
      b[cols[n][0]:cols[n][0] + cols[n][1]] = t
    lw.in_b = dev(b)
  if a is not None and a.sink:
    lw.sink = dev(get(m + "sink"))
  if sd is not None:
    lw.conv_w, lw.conv_b = dev(get(m + "conv")), dev(get(m + "conv.b"))
    lw.A_log, lw.dt_bias, lw.skip_d = dev(get(m + "A_log")), dev(get(m + "dt_bias")), dev(get(m + "D"))
    lw.ssd_norm = dev(get(m + "norm"))
  if f is None:
    return lw
  q = p + "mlp."
  if f.kind == "polynorm":
    fb = [("up", get(q + "up"))]
    down = get(q + "down")
    lw.act = dev(get(q + "act"))
  else:
    lw.router_b = dev(get(q + "router.b"))
    _relu2_moe_weights(lw, f, get, q, D, dev, dtype, gate_rows=get(p + "rg2"))
    lw.norm2, lw.gate2_b = dev(get(p + "norm2")), dev(get(p + "rg2.b"))
    return lw
  fb.append(("gate", get(p + "rg2")))
  ff_w, lw.ff_cols = _fused_rows(fb, D)
  lw.ff_w = dev(ff_w, dtype)
  if down is not None:
    lw.down_w = dev(_pad2(down, _up(D, 64), _up(down.shape[1], 128)), dtype)
  lw.norm2, lw.gate2_b = dev(get(p + "norm2")), dev(get(p + "rg2.b"))
  return lw


def build_sandwich_layer(spec, get, p: str, D: int, device, dtype) -> MixedLayerWeights:
  """One sandwich layer (latent attention; clamped gated or SiLU-expert feed-forward) from `get(name)`."""
  def dev(t, dt=torch.float32):
    return t.to(device=device, dtype=dt).contiguous()
  m = p + "mix."
  a, f = spec.lattn, spec.ffn
  blocks = [("q", get(m + "dq" if a.q_rank else m + "q")), ("ckv", get(m + "dkv"))]
  if a.gate != "none":
    blocks.append(("gate", get(m + "g")))
  in_w, cols = _fused_rows(blocks, D)
  out = get(m + "o")
  lw = MixedLayerWeights(spec, dev(in_w, dtype), cols, dev(_pad2(out, _up(D, 64), _up(out.shape[1], 128)), dtype),
                         {"mix": (0, out.shape[1])})
  lw.norm1, lw.norm1b, lw.kv_norm = dev(get(p + "norm1")), dev(get(p + "norm1b")), dev(get(m + "dkv.norm"))
  if a.q_rank:
    lw.q_norm = dev(get(m + "dq.norm"))
    uq = get(m + "uq")
    lw.uq_w = dev(_pad2(uq, _up(uq.shape[0], 64), _up(a.q_rank, 128)), dtype)
  lw.uk_w = dev(get(m + "uk").reshape(a.heads, a.dim, a.kv_rank), dtype)
  lw.uv_w = dev(get(m + "uv").reshape(a.heads, a.vdim, a.kv_rank).transpose(1, 2), dtype)
  if a.sink:
    lw.sink = dev(get(m + "sink"))
  if f is None:
    return lw
  q = p + "mlp."
  if f.kind == "clamped_glu":
    fb = [("gate", get(q + "gate")), ("up", get(q + "up"))]
    down = get(q + "down")
  else:
    fb = [("router", get(q + "router"))]
    down = None
    if f.shared_ff:
      fb += [("sh_gate", get(q + "shared.gate")), ("sh_up", get(q + "shared.up"))]
      down = get(q + "shared.down")
    Fp, Dp = _up(f.ff, 128), _up(D, 128)
    # gate and up rows interleaved in tiles of 16 (the grouped GEMM's SiLU epilogue pairs them)
    lw.ex_up_w = dev(torch.stack([interleave_gate_up(_pad2(get(q + f"e{e}.gate"), Fp, Dp), _pad2(get(q + f"e{e}.up"), Fp, Dp))
                                  for e in range(f.experts)]), dtype)
    lw.ex_down_w = dev(torch.stack([_pad2(get(q + f"e{e}.down"), Dp, Fp) for e in range(f.experts)]), dtype)
  ff_w, lw.ff_cols = _fused_rows(fb, D)
  lw.ff_w = dev(ff_w, dtype)
  if down is not None:
    lw.down_w = dev(_pad2(down, _up(D, 64), _up(down.shape[1], 128)), dtype)
  lw.norm2, lw.norm2b = dev(get(p + "norm2")), dev(get(p + "norm2b"))
  return lw


def _pair_order(d: int, R: int) -> torch.Tensor:
  """Row order of one head whose rotation pairs (2i, 2i + 1) become (i, i + R / 2), the kernels' layout: a
  permutation of the head's dims, applied to queries and keys alike, leaves every score as it was."""
  return torch.tensor(list(range(0, R, 2)) + list(range(1, R, 2)) + list(range(R, d)), dtype=torch.long)


def _relu2_moe_weights(lw: MixedLayerWeights, f, get, q: str, D: int, dev, dtype, gate_rows=None):
  """Router | shared up | shared gate (| the sublayer's gate) fused into ff_w, experts stacked and padded."""
  fb = [("router", get(q + "router"))]
  down = None
  if f.shared_ff:
    fb += [("sh_up", get(q + "shared.up")), ("sh_gate", get(q + "shared.sg").reshape(1, D))]
    down = get(q + "shared.down")
  Fp, Dp = _up(f.ff, 128), _up(D, 128)
  lw.ex_up_w = dev(torch.stack([_pad2(get(q + f"e{e}.up"), Fp, Dp) for e in range(f.experts)]), dtype)
  lw.ex_down_w = dev(torch.stack([_pad2(get(q + f"e{e}.down"), Dp, Fp) for e in range(f.experts)]), dtype)
  if gate_rows is not None:
    fb.append(("gate", gate_rows))
  ff_w, lw.ff_cols = _fused_rows(fb, D)
  lw.ff_w = dev(ff_w, dtype)
  if down is not None:
    lw.down_w = dev(_pad2(down, _up(D, 64), _up(down.shape[1], 128)), dtype)


def build_ln_sandwich_layer(spec, get, p: str, D: int, device, dtype) -> MixedLayerWeights:
  """One layer-norm sandwich layer (differential attention, mlstm, or gated attention beside lightning attention;
  relu^2 experts with grouped sigmoid routing) from `get(name)`."""
  def dev(t, dt=torch.float32):
    return t.to(device=device, dtype=dt).contiguous()
  m = p + "mix."
  a, w, r, f = spec.dattn, spec.wattn, spec.rec, spec.ffn
  bias, out2 = {}, None
  if a is not None:
    rep, d = a.heads // a.kv_heads, a.dim
    order = _pair_order(d, a.rot_dims)
    q = get(m + "q").reshape(a.kv_heads, rep, 2, d, D).permute(0, 2, 1, 3, 4)[:, :, :, order]  # [kv head, map, head, d]
    k = get(m + "k").reshape(a.kv_heads, 2, d, D)[:, :, order]
    blocks = [("q", q.reshape(-1, D)), ("k", k.reshape(-1, D)), ("v", get(m + "v")), ("gate", get(m + "g"))]
    out = get(m + "o")
  elif w is not None:
    l, rr = m + "left.", m + "right."
    blocks = [(n, get(l + n)) for n in ("q", "k", "v")] + [("gate", get(l + "g"))]
    bias = {n: get(l + n + ".b") for n in ("q", "k", "v")}
    blocks += [("rq", get(rr + "q")), ("rk", get(rr + "k")), ("rv", get(rr + "v")), ("rg", get(rr + "g"))]
    out, out2 = get(l + "o"), get(rr + "o")
  else:
    blocks = [("rq", get(m + "q")), ("rk", get(m + "k")), ("rv", get(m + "v")), ("rg", get(m + "g")), ("ri", get(m + "i")),
              ("rf", get(m + "f"))]
    out = get(m + "o")
  in_w, cols = _fused_rows(blocks, D)
  lw = MixedLayerWeights(spec, dev(in_w, dtype), cols, dev(_pad2(out, _up(D, 64), _up(out.shape[1], 128)), dtype),
                         {"mix": (0, out.shape[1])})
  for n in ("norm1", "norm1b") + (("norm2", "norm2b") if f is not None else ()):
    setattr(lw, n, dev(get(p + n)))
    setattr(lw, n + "_b", dev(get(p + n + ".b")))
  if a is not None:
    lam = torch.exp((get(m + "lq1") * get(m + "lk1")).sum()) - torch.exp((get(m + "lq2") * get(m + "lk2")).sum()) + a.lam_init
    lw.lam = float(lam)
  if bias:
    b = torch.zeros(in_w.shape[0])
    for n, t in bias.items():
      b[cols[n][0]:cols[n][0] + cols[n][1]] = t
    lw.in_b = dev(b)
  if out2 is not None:
    lw.out2_w = dev(_pad2(out2, _up(D, 64), _up(out2.shape[1], 128)), dtype)
    lw.mix_cols["mix2"] = (0, out2.shape[1])
    lw.pair_w = dev(torch.stack([get(m + "left.out"), get(m + "right.out")]))
    lw.rec_norm = dev(get(m + "right.norm"))
    lw.decay = dev(torch.tensor(r.decays))
  elif r is not None:
    lw.rec_norm = dev(get(m + "norm"))
    lw.gate_b = dev(torch.cat([get(m + "i.b"), get(m + "f.b")]))
  if f is not None:
    _relu2_moe_weights(lw, f, get, p + "mlp.", D, dev, dtype)
    lw.router_b = dev(get(p + "mlp.correction"))
  return lw


def ln_sandwich_tensor_shapes(c: ModelConfig) -> Dict[str, tuple]:
  """Name -> shape of every tensor of a layer-norm sandwich checkpoint (Kopalorn)."""
  D, out = c.hidden_size, {}
  out["embed"] = (c.vocab_size, D)
  if c.loop:
    out["loop.step"] = (c.loop[2], D)
  for i, s in enumerate(c.layer_specs):
    p, m = f"l{i}.", f"l{i}.mix."
    a, w, r, f = s.dattn, s.wattn, s.rec, s.ffn
    for n in ("norm1", "norm1b") + (("norm2", "norm2b") if f is not None else ()):
      out[p + n], out[p + n + ".b"] = (D,), (D,)
    if a is not None:
      out[m + "q"], out[m + "k"], out[m + "v"] = (2 * a.heads * a.dim, D), (2 * a.kv_heads * a.dim, D), (a.kv_heads * a.vdim, D)
      for n in ("lq1", "lk1", "lq2", "lk2"):
        out[m + n] = (a.dim,)
      out[m + "g"], out[m + "o"] = (a.heads, D), (D, a.heads * a.vdim)
    elif w is not None:
      l, rr = m + "left.", m + "right."
      for n, rows in (("q", w.heads * w.dim), ("k", w.kv_heads * w.dim), ("v", w.kv_heads * w.vdim)):
        out[l + n], out[l + n + ".b"] = (rows, D), (rows,)
      out[l + "g"], out[l + "o"] = (w.heads * w.vdim, D), (D, w.heads * w.vdim)
      out[rr + "q"], out[rr + "k"], out[rr + "v"] = (r.heads * r.dim, D), (r.heads * r.dim, D), (r.heads * r.vdim, D)
      out[rr + "g"], out[rr + "o"], out[rr + "norm"] = (r.heads * r.vdim, D), (D, r.heads * r.vdim), (r.heads * r.vdim,)
      out[l + "out"], out[rr + "out"] = (D,), (D,)
    else:
      out[m + "q"], out[m + "k"], out[m + "v"] = (r.heads * r.dim, D), (r.heads * r.dim, D), (r.heads * r.vdim, D)
      out[m + "g"], out[m + "o"], out[m + "norm"] = (r.heads * r.vdim, D), (D, r.heads * r.vdim), (r.heads * r.vdim,)
      out[m + "i"], out[m + "i.b"], out[m + "f"], out[m + "f.b"] = (r.heads, D), (r.heads,), (r.heads, D), (r.heads,)
    if f is None:
      continue
    q = p + "mlp."
    for e in range(f.experts):
      out[q + f"e{e}.up"], out[q + f"e{e}.down"] = (f.ff, D), (D, f.ff)
    out[q + "router"], out[q + "correction"] = (f.experts, D), (f.experts,)
    if f.shared_ff:
      out[q + "shared.up"], out[q + "shared.down"], out[q + "shared.sg"] = (f.shared_ff, D), (D, f.shared_ff), (1, D)
  out["final.norm"], out["final.norm.b"], out["head"] = (D,), (D,), (c.vocab_size, D)
  return out


def sandwich_tensor_shapes(c: ModelConfig) -> Dict[str, tuple]:
  """Name -> shape of every tensor of a sandwich-block checkpoint (Nenizen); the LM head is the embedding table."""
  D, out = c.hidden_size, {}
  out["embed"] = (c.vocab_size, D)
  if c.loop:
    out["loop.in"], out["loop.step"] = (D, 2 * D), (c.loop[2], D)
  for i, s in enumerate(c.layer_specs):
    p, m, a, f = f"l{i}.", f"l{i}.mix.", s.lattn, s.ffn
    out[p + "norm1"], out[p + "norm1b"] = (D,), (D,)
    qd = a.heads * (a.dim + a.rot_dim)
    if a.q_rank:
      out[m + "dq"], out[m + "dq.norm"], out[m + "uq"] = (a.q_rank, D), (a.q_rank,), (qd, a.q_rank)
    else:
      out[m + "q"] = (qd, D)
    out[m + "dkv"], out[m + "dkv.norm"] = (a.kv_rank + a.rot_dim, D), (a.kv_rank,)
    out[m + "uk"], out[m + "uv"] = (a.heads * a.dim, a.kv_rank), (a.heads * a.vdim, a.kv_rank)
    if a.gate != "none":
      out[m + "g"] = (a.gate_rows, D)
    if a.sink:
      out[m + "sink"] = (a.heads,)
    out[m + "o"] = (D, a.heads * a.vdim)
    if f is None:
      continue
    q = p + "mlp."
    out[p + "norm2"], out[p + "norm2b"] = (D,), (D,)
    if f.kind == "clamped_glu":
      out[q + "gate"], out[q + "up"], out[q + "down"] = (f.ff, D), (f.ff, D), (D, f.ff)
    else:
      for e in range(f.experts):
        out[q + f"e{e}.gate"], out[q + f"e{e}.up"], out[q + f"e{e}.down"] = (f.ff, D), (f.ff, D), (D, f.ff)
      out[q + "router"] = (f.experts, D)
      if f.shared_ff:
        out[q + "shared.gate"], out[q + "shared.up"], out[q + "shared.down"] = (f.shared_ff, D), (f.shared_ff, D), \
          (D, f.shared_ff)
  out["final.norm"] = (D,)
  return out


def postln_tensor_shapes(c: ModelConfig) -> Dict[str, tuple]:
  """Name -> shape of every tensor of a post-norm mixed-layer checkpoint (Mogelix)."""
  D, out = c.hidden_size, {}
  out["embed"] = (c.vocab_size, D)
  for i, s in enumerate(c.layer_specs):
    p, m = f"l{i}.", f"l{i}.mix."
    out[p + "norm1"], out[p + "rg1"], out[p + "rg1.b"] = (D,), (D, D), (D,)
    a, sd, f = s.wattn, s.ssd, s.ffn
    if a is not None:
      proj = [("q", a.heads * a.dim)] + ([("k", a.kv_heads * a.dim), ("v", a.kv_heads * a.vdim)] if a.kv_from < 0 else [])
      for n, rows in proj:
        out[m + n] = (rows, D)
        if a.bias:
          out[m + n + ".b"] = (rows,)
      if a.sink:
        out[m + "sink"] = (a.heads,)
      out[m + "o"] = (D, a.heads * a.vdim)
    if sd is not None:
      out[m + "in"] = (2 * sd.inner + 2 * sd.groups * sd.state + sd.heads, D)
      out[m + "conv"], out[m + "conv.b"] = (sd.conv_channels, sd.conv), (sd.conv_channels,)
      out[m + "dt_bias"], out[m + "A_log"], out[m + "D"] = (sd.heads,), (sd.heads,), (sd.heads,)
      out[m + "norm"], out[m + "o"] = (sd.inner,), (D, sd.inner)
    if f is None:
      continue
    q = p + "mlp."
    out[p + "norm2"], out[p + "rg2"], out[p + "rg2.b"] = (D,), (D, D), (D,)
    if f.kind == "polynorm":
      out[q + "up"], out[q + "down"], out[q + "act"] = (f.ff, D), (D, f.ff), (4,)
    else:
      for e in range(f.experts):
        out[q + f"e{e}.up"], out[q + f"e{e}.down"] = (f.ff, D), (D, f.ff)
      out[q + "router"], out[q + "router.b"] = (f.experts, D), (f.experts,)
      if f.shared_ff:
        out[q + "shared.up"], out[q + "shared.down"], out[q + "shared.sg"] = (f.shared_ff, D), (D, f.shared_ff), (1, D)
  out["final.norm"], out["head"] = (D,), (c.vocab_size, D)
  return out


def mixed_tensor_shapes(c: ModelConfig) -> Dict[str, tuple]:
  """Name -> shape of every tensor of a mixed-layer checkpoint (random init, checkpoint validation)."""
  if c.block == "postln":
    return postln_tensor_shapes(c)
  if c.block == "sandwich":
    return ln_sandwich_tensor_shapes(c) if c.norm_kind == "layer" else sandwich_tensor_shapes(c)
  D, out = c.hidden_size, {}
  out["embed"] = (c.vocab_size, D)
  for i, s in enumerate(c.layer_specs):
    p = f"l{i}."
    out[p + "norm1"], out[p + "ls1"] = (), (D,)
    if s.attn is not None:
      a, m = s.attn, p + "mix.left."
      out[m + "q"], out[m + "k"], out[m + "pb"], out[m + "o"] = (a.heads * a.dim, D), (a.kv_heads * a.dim, D), (a.heads,), \
        (D, a.heads * a.vdim)
    r = s.rec
    if r is not None and r.rule == "delta":
      m = p + "mix.right."
      for n, rows in (("q", r.kv_heads * r.dim), ("k", r.kv_heads * r.dim), ("v", r.heads * r.vdim)):
        out[m + n], out[m + n + ".conv"] = (rows, D), (rows, r.conv)
      out[m + "b"], out[m + "a"], out[m + "A_log"], out[m + "dt_bias"] = (r.heads, D), (r.heads, D), (r.heads,), (r.heads,)
      out[m + "norm"], out[m + "g"], out[m + "o"] = (r.vdim,), (r.heads * r.vdim, D), (D, r.heads * r.vdim)
    elif r is not None:
      m, rank = p + "mix.", r.rank or 8
      out[m + "q"], out[m + "k"], out[m + "v"] = (r.heads * r.dim, D), (r.heads * r.dim, D), (r.heads * r.vdim, D)
      out[m + "g"], out[m + "o"], out[m + "norm"] = (r.heads * r.vdim, D), (D, r.heads * r.vdim), (r.vdim,)
      out[m + "a1"], out[m + "a2"], out[m + "a2.b"] = (rank, D), (r.heads * r.dim, rank), (r.heads * r.dim,)
    if s.ff:
      out[p + "mlp.gate"], out[p + "mlp.up"], out[p + "mlp.down"], out[p + "ls2"] = (s.ff, D), (s.ff, D), (D, s.ff), (D,)
  out["final.norm"], out["head"] = (), (c.vocab_size, D)
  return out


def random_mixed_tensors(c: ModelConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
  """Deterministic random checkpoint of a mixed-layer architecture, values rounded to bf16 (as a stored checkpoint's
  are): projections ~ N(0, 1/sqrt(fan_in)), gains / layer scales / biases of order one so every mechanism shows."""
  out = {}
  for j, (name, shape) in enumerate(mixed_tensor_shapes(c).items()):
    g = torch.Generator().manual_seed(seed * 1_000_003 + 7919 * j + 17)
    leaf = name.split(".")[-1]
    if name.endswith(".conv"):
      t = torch.randn(shape, generator=g) * 0.5
    elif c.norm_kind == "layer" and leaf in ("b", "correction", "out", "lq1", "lk1", "lq2", "lk2"):
      # norm biases, projection biases, gate biases (forget gates mostly open), the router's correction (large enough to
      # change the choice), the lambda vectors
      kind = name.split(".")[-2]
      t = {"b": torch.randn(shape, generator=g) * (0.1 if kind.startswith("norm") else 0.5) + (2.0 if kind == "f" else 0.0),
           "correction": torch.randn(shape, generator=g) * 0.3,
           "out": 1.0 + 0.1 * torch.randn(shape, generator=g)}.get(leaf)
      if t is None:
        t = torch.randn(shape, generator=g) * 0.4
    elif leaf in ("sink", "D", "act") or (leaf == "b" and c.block == "postln"):
      t = torch.randn(shape, generator=g) * (0.5 if leaf == "b" else 1.0)
    elif leaf in ("norm1", "norm2", "norm1b", "norm2b") or name == "final.norm":
      t = 1.0 + 0.1 * torch.randn(shape, generator=g)
    elif leaf in ("ls1", "ls2"):
      t = 0.5 + 0.1 * torch.randn(shape, generator=g)
    elif leaf == "norm":
      t = 1.0 + 0.1 * torch.randn(shape, generator=g)
    elif leaf in ("pb", "dt_bias"):
      t = torch.randn(shape, generator=g) - (2.0 if leaf == "pb" else 0.0)
    elif leaf == "A_log":
      t = torch.rand(shape, generator=g) * 1.5 - 2.0
    elif leaf == "b" and len(shape) == 1:  # a2.b: decays close to one
      t = 3.0 + torch.randn(shape, generator=g)
    elif name == "loop.step":
      t = torch.randn(shape, generator=g) * 0.3
    elif name == "embed":
      t = torch.randn(shape, generator=g) * (0.25 if c.block == "sandwich" else 1.0)
    else:
      t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
    out[name] = t.to(torch.bfloat16).float()
  return out


def mixed_weights(c: ModelConfig, shard: Shard, get, device, dtype) -> ShardWeights:
  """ShardWeights of a mixed-layer model from `get(name) -> fp32 CPU tensor`."""
  sw = ShardWeights(c, shard)
  D = c.hidden_size
  build = {"postln": build_postln_layer, "sandwich": build_sandwich_layer}.get(c.block, build_mixed_layer)
  if c.block == "sandwich" and c.norm_kind == "layer":
    build = build_ln_sandwich_layer
  for i in shard.layers():
    sw.layers[i] = build(c.layer_specs[i], get, f"l{i}.", D, device, dtype)
  if shard.is_first_layer():
    # gathered into the fp32 residual; a model that scales its embedding output gathers from the scaled table
    sw.embed = (get("embed") * c.embed_scale).to(device=device, dtype=torch.float32).contiguous()
  if c.loop and c.loop_input == "add" and any(c.loop[0] <= i < c.loop[1] for i in shard.layers()):
    sw.loop_step = get("loop.step").to(device=device, dtype=torch.float32).contiguous()
  elif c.loop and any(c.loop[0] <= i < c.loop[1] for i in shard.layers()):
    w_in = get("loop.in")  # [D, 2 D] over [x | embedding output]: each half padded to the GEMM's K tile
    Dp = _up(D, 128)
    li = torch.zeros(_up(D, 64), 2 * Dp)
    li[:D, :D], li[:D, Dp:Dp + D] = w_in[:, :D], w_in[:, D:]
    sw.loop_in = li.to(device=device, dtype=dtype).contiguous()
    sw.loop_step = get("loop.step").to(device=device, dtype=torch.float32).contiguous()
  if shard.is_last_layer():
    sw.norm = get("final.norm").reshape(-1).to(device=device, dtype=torch.float32)
    if c.norm_kind == "layer":
      sw.norm_b = get("final.norm.b").reshape(-1).to(device=device, dtype=torch.float32)
    head = torch.zeros(_up(c.vocab_size, 64), _up(D, 128))
    head[:c.vocab_size, :D] = get("embed" if c.tie_word_embeddings and c.is_mixed else "head")
    sw.lm_head = head.to(device=device, dtype=dtype).contiguous()
  return sw


def load_mixed_weights(model_dir: Path, c: ModelConfig, shard: Shard, device, dtype) -> ShardWeights:
  """Tarepel / Mogelix / Nenizen checkpoint (flat names: embed, l<i>.norm1, l<i>.mix.*, l<i>.mlp.*, l<i>.ls1 / ls2 or l<i>.rg1 /
  rg2, final.norm, head).  The decay rank of a gated-linear-attention layer is the a1 tensor's row count."""
  from safetensors import safe_open
  wm = _weight_map(Path(model_dir))
  handles = {}

  def get(name: str) -> torch.Tensor:
    if name not in wm:
      raise KeyError(f"checkpoint has no tensor {name!r}")
    f = wm[name]
    if f not in handles:
      handles[f] = safe_open(str(Path(model_dir) / f), framework="pt")
    return handles[f].get_tensor(name).float()
  want = mixed_tensor_shapes(c)
  for name, shape in want.items():
    if name.split(".")[0] in ("embed", "final", "head", "loop") or int(name.split(".")[0][1:]) in shard.layers():
      got = tuple(get(name).shape) if not name.endswith((".a1", ".a2")) else None
      if name == "loop.step" and got is not None and got[1:] == tuple(shape)[1:] and got[0] >= shape[0]:
        continue
      if got is not None and got != tuple(shape):
        raise ValueError(f"{name}: checkpoint shape {got}, config says {tuple(shape)}")
  return mixed_weights(c, shard, get, device, dtype)
