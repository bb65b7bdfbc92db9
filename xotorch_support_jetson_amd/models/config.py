"""Model configuration: HF `config.json` -> typed ModelConfig, plus built-in presets.

Presets carry the public HF architecture numbers for the BASELINE.json configs so the framework can
build random-init models of the exact shape offline (there is no network on the GPU box).
Reference: load_model_config (xotorch/inference/torch/models/llm_utils.py:30-77); unlike it, the
layer count comes from config.json and is validated against the model card.
"""
from __future__ import annotations

import json
from dataclasses import asdict, dataclass, field, replace
from pathlib import Path
from typing import Optional


@dataclass(frozen=True)
class GatedAttnSpec:
  """Chunk-local gated attention: GQA, rotate-half RoPE on the first rot_dims dims of each head, a key is
  visible to a query of the same chunk-sized block at or before it, and weighs sigmoid(score * scale + bias[head])
  (no normalisation over keys).  values_are_keys: the value of a token is its key before rotation (no v
  projection; vdim == dim)."""
  heads: int
  kv_heads: int
  dim: int
  vdim: int
  chunk: int
  rot_dims: int
  rot_base: float
  scale: float
  values_are_keys: bool = True


@dataclass(frozen=True)
class LinearRecurrenceSpec:
  """A linear-attention state S [dim, vdim] per head carried in fp32: S <- decay * S (+ delta-rule or plain
  outer-product write), o = S^T q.
  rule "delta": scalar decay per head g = exp(-exp(A_log) softplus(a + dt_bias)), write k (beta (v - S^T k))^T,
    q / k shared by heads / kv_heads value heads, short causal convolutions (conv taps) + SiLU on q, k, v,
    unit-norm q and k, q scaled by dim^-1/2.
  rule "gla": decay per key channel sigmoid(z)^(1/tau) with a low-rank z, write k v^T, q scaled by dim^-1/2.
  rule "lightning": one fixed decay per head (`decays`), SiLU on q, k, v, write k v^T, no scale; the heads' outputs are
    RMS-normed together, weighted and gated by a sigmoid.
  rule "mlstm": the matrix memory of xLSTM.  Log input gate i = cap tanh(z_i / cap), log forget gate f = logsigmoid(cap
    tanh(z_f / cap)) per head (gate_cap), a running maximum m_t = max(f + m_(t-1), i) that starts at 0, S <- e^(f + m_(t-1) -
    m_t) S + e^(i - m_t) k v^T and a normaliser n likewise from k alone, o = S^T q / (max(|n . q|, e^(-m_t)) + 1e-6), q
    scaled by dim^-1/2.  The normaliser travels as one more value channel of the state (value = 1), the maximum beside it."""
  rule: str  # delta | gla | lightning | mlstm
  heads: int
  kv_heads: int
  dim: int
  vdim: int
  conv: int = 0  # taps of the short convolutions (delta)
  tau: float = 1.0  # decay temperature (gla)
  rank: int = 0  # rank of the decay projection (gla; from the tensor's shape)
  decays: tuple = ()  # lightning: one per head
  gate_cap: float = 0.0  # mlstm

  @property
  def state_vdim(self) -> int:
    """Value channels of the state: mlstm keeps its normaliser as one channel more."""
    return self.vdim + 1 if self.rule == "mlstm" else self.vdim


@dataclass(frozen=True)
class WindowAttnSpec:
  """Softmax attention (GQA) over a sliding window plus pooled blocks: a query at position i sees the tokens j with
  0 <= i - j < window (window 0: every earlier token) and, with pool > 0, one mean key / mean value per block of
  `pool` tokens that ends at or before i - window; tokens, blocks and an optional per-head sink logit (no value) share
  one softmax.  q / k / v may carry biases; rotate-half RoPE on the first rot_dims dims with optional wavelength-banded
  frequency scaling rot_scaling = (factor, low, high, original); qk_norm divides q and k by their RMS per head after
  the rotation.  kv_from >= 0: no key / value projections, the layer reads that layer's caches with its own queries
  and its own window / pool.  gate "elem": the heads' outputs times sigmoid of a projection of the mixer's input, element
  by element."""
  heads: int
  kv_heads: int
  dim: int
  vdim: int
  window: int
  pool: int
  rot_dims: int
  rot_base: float
  rot_scaling: Optional[tuple]
  scale: float
  qk_norm: bool = True
  bias: bool = True
  sink: bool = True
  kv_from: int = -1
  gate: str = "none"  # none | elem


@dataclass(frozen=True)
class DiffAttnSpec:
  """Differential softmax attention (GQA): every head holds two query / key maps of size dim that attend to the same
  values; o = a_1 - lam a_2 with lam = exp(lq1 . lk1) - exp(lq2 . lk2) + lam_init (learned vectors, one number per
  layer), then o / rms(o) per head (no weight) times (1 - lam_init), times sigmoid of one gate per head.  RoPE on the
  first rot_dims dims of each map, pairs (2i, 2i + 1); window > 0: a query at position i sees 0 <= i - j < window, else
  every j <= i.  The cache holds 2 kv_heads key heads (a kv head's two maps side by side) and kv_heads value heads."""
  heads: int
  kv_heads: int
  dim: int
  vdim: int
  window: int
  rot_dims: int
  rot_base: float
  scale: float
  lam_init: float


@dataclass(frozen=True)
class SSDSpec:
  """State-space-duality recurrence (Mamba-2): per head a state S [state, vdim] in fp32,
  S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x, with B / C shared by heads / groups heads, a causal
  convolution of `conv` taps + SiLU over the x | B | C channels, dt = softplus(dt + bias); y is gated by silu(z) and
  RMS-normed in norm_groups equal parts."""
  heads: int
  vdim: int
  state: int
  groups: int
  conv: int
  norm_groups: int = 1

  @property
  def inner(self) -> int:
    return self.heads * self.vdim

  @property
  def conv_channels(self) -> int:
    return self.inner + 2 * self.groups * self.state


@dataclass(frozen=True)
class FeedForwardSpec:
  """A non-gated feed-forward W_down act(W_up h).  kind "polynorm": act(z) = a N(z) + b N(z^2) + c N(z^3) + e with N the
  division of the token's ff vector by its RMS; kind "relu2_moe": `experts` experts with act = relu^2, the `top` largest
  router logits chosen per token and weighted by the softmax over the chosen logits (or the `route` rule below), plus
  (shared_ff > 0) one shared expert of the same form scaled by a per-token sigmoid gate.
  Gated kinds, W_down (a(W_gate h) * b(W_up h)): "clamped_glu": g = min(gate, limit), u = clamp(up, -limit, limit),
  g sigmoid(1.702 g) (u + 1); "silu_moe": `experts` SiLU-gated experts, scores = softmax of the router logits over
  all experts, the `top` largest chosen and weighted by their scores as they are (no renormalisation), plus
  (shared_ff > 0) one ungated shared expert of the same form."""
  kind: str  # polynorm | relu2_moe | clamped_glu | silu_moe
  ff: int
  experts: int = 0
  top: int = 0
  shared_ff: int = 0
  limit: float = 0.0  # clamped_glu
  # relu2_moe routing.  "softmax_top": the rule above.  "sigmoid_groups": scores = sigmoid(logits); the choice is made on
  # scores + a learned correction, among the experts of the `keep` best of `groups` equal groups of neighbours (a
  # group's value: the sum of its two largest corrected scores); weights = the chosen experts' uncorrected scores over
  # their sum, times route_scale
  route: str = "softmax_top"
  groups: int = 1
  keep: int = 1
  route_scale: float = 1.0


@dataclass(frozen=True)
class LatentAttnSpec:
  """Softmax attention through a low-rank key / value latent: per token the cache holds one RMS-normed latent c
  [kv_rank] and one rotated key part [rot_dim] shared by every head.  Head h scores q_h = [dim unrotated | rot_dim
  rotated] against [W_uk,h c | rotated part] (times scale) and sums the values W_uv,h c.  q_rank > 0: the queries go
  through their own RMS-normed latent.  RoPE on the first rot_dims of the rot_dim part, pairs (2i, 2i + 1)
  (rot_interleaved) or (i, i + rot_dims / 2).  window > 0: a query at position i sees 0 <= i - j < window, else every
  j <= i.  sink: one learned logit per head joins the softmax's denominator (no key, no value, unscaled).  gate: the
  heads' outputs times sigmoid of a projection of the mixer's input, per element ("elem") or per head ("head")."""
  heads: int
  dim: int
  rot_dim: int
  vdim: int
  kv_rank: int
  q_rank: int
  rot_dims: int
  rot_base: float
  rot_interleaved: bool
  scale: float
  window: int = 0
  sink: bool = False
  gate: str = "none"  # none | elem | head

  @property
  def gate_rows(self) -> int:
    return {"none": 0, "elem": self.heads * self.vdim, "head": self.heads}[self.gate]


@dataclass(frozen=True)
class MixedLayerSpec:
  """One layer of a model whose layers differ (ModelConfig.layer_specs).  Parallel blocks (ModelConfig.block
  "parallel"): the token mixers attn / rec read the layer's one normed input side by side, with their output scales and
  the gated feed-forward size ff (0: none).  Post-norm blocks ("postln"): one mixer, wattn or ssd, then the
  feed-forward ffn (None: none)."""
  kind: str  # config.json's layer type
  attn: Optional[GatedAttnSpec] = None
  rec: Optional[LinearRecurrenceSpec] = None
  attn_scale: float = 1.0
  rec_scale: float = 1.0
  ff: int = 0
  wattn: Optional[WindowAttnSpec] = None
  ssd: Optional[SSDSpec] = None
  ffn: Optional[FeedForwardSpec] = None
  lattn: Optional[LatentAttnSpec] = None  # sandwich blocks
  dattn: Optional[DiffAttnSpec] = None  # sandwich blocks; a "parallel" layer there is wattn beside rec

  @property
  def kv_dims(self) -> Optional[tuple]:
    """(key heads, key dim, value dim[, value heads]) of the paged K / V pool this layer owns (None: it has none of its
    own).  A latent-attention layer keeps one row [kv_rank | rot_dim] per token and no value pool (value dim 0); a
    differential-attention layer two key heads per value head."""
    if self.lattn is not None:
      return 1, self.lattn.kv_rank + self.lattn.rot_dim, 0
    if self.dattn is not None:
      return 2 * self.dattn.kv_heads, self.dattn.dim, self.dattn.vdim, self.dattn.kv_heads
    if self.attn is not None:
      return self.attn.kv_heads, self.attn.dim, self.attn.dim
    if self.wattn is not None and self.wattn.kv_from < 0:
      return self.wattn.kv_heads, self.wattn.dim, self.wattn.vdim
    return None

  @property
  def state_dims(self) -> Optional[tuple]:
    """(heads, value channels, key dim, convolution taps, convolution channels, scalars per head) of the layer's
    recurrent state."""
    if self.rec is not None:
      r = self.rec
      return r.heads, r.state_vdim, r.dim, r.conv, (2 * r.kv_heads * r.dim + r.heads * r.vdim) if r.conv > 0 else 0, \
        1 if r.rule == "mlstm" else 0
    if self.ssd is not None:
      m = self.ssd
      return m.heads, m.vdim, m.state, m.conv, m.conv_channels if m.conv > 0 else 0, 0
    return None


@dataclass(frozen=True)
class ModelConfig:
  model_type: str  # llama | qwen2 | mistral | mixtral | ... | tarepel | mogelix | nenizen
  vocab_size: int
  hidden_size: int
  intermediate_size: int
  num_layers: int
  num_heads: int
  num_kv_heads: int
  head_dim: int
  rms_norm_eps: float = 1e-5
  rope_theta: float = 500000.0
  rope_scaling: Optional[dict] = None
  max_position_embeddings: int = 8192
  tie_word_embeddings: bool = False
  attention_bias: bool = False
  num_experts: int = 0  # >0: MoE (Mixtral) MLP
  num_experts_per_tok: int = 0
  bos_token_id: int = 128000
  eos_token_ids: tuple = (128001, 128009)
  partial_rotary_factor: float = 1.0  # Phi-3: RoPE on the first 75 % of each head's dims
  # DeepSeek-V2/V3 multi-head latent attention (kv_lora_rank > 0): per token the cache holds one
  # normalised latent [kv_lora_rank] + one shared rotated key [qk_rope_head_dim]
  q_lora_rank: int = 0  # 0: plain q_proj
  kv_lora_rank: int = 0
  qk_nope_head_dim: int = 0
  qk_rope_head_dim: int = 0
  v_head_dim: int = 0
  # MoE routing (Mixtral: softmax top-k renormalised; DeepSeek: shared experts, dense first layers,
  # group-limited selection, sigmoid scores with a selection bias (V3), scaled weights)
  moe_intermediate_size: int = 0  # 0: intermediate_size
  n_shared_experts: int = 0
  first_k_dense_replace: int = 0
  moe_layer_freq: int = 1
  routed_scaling_factor: float = 1.0
  topk_method: str = "greedy"  # greedy | group_limited_greedy (V2) | noaux_tc (V3)
  n_group: int = 1
  topk_group: int = 1
  norm_topk_prob: bool = True
  scoring_func: str = "softmax"  # softmax | sigmoid
  # LLaVA: CLIP vision tower + projector on the first shard (HF vision_config keys), image token id
  vision: Optional[dict] = None
  image_token_id: int = -1
  vision_feature_layer: int = -2
  vision_select: str = "default"  # default: drop the CLS feature | full
  projector_act: str = "gelu"
  # models with per-layer mixers (Tarepel): one MixedLayerSpec per layer; parallel mixer + feed-forward blocks on
  # an fp32 residual stream, scalar-gain RMS norms, per-channel layer scales, scaled logits
  layer_specs: Optional[tuple] = None
  logit_scale: float = 1.0
  # block form of a mixed-layer model: "parallel" (Tarepel: pre-norm, mixers and feed-forward side by side) or "postln"
  # (Mogelix: x <- norm(alpha x + gate * sublayer(x)) for the mixer, then for the feed-forward; per-channel norm weights)
  block: str = "parallel"
  postln_alpha: float = 1.0
  # "sandwich" blocks (Nenizen): x += norm_b(mixer(norm(x))), then x += norm_b(ff(norm(x))), per-channel weights.
  # loop = (start, stop, times): layers start .. stop - 1 run `times` times in a row with the same weights and a cache
  # of their own per pass; each pass starts with x <- W_in [x; embedding output] + step[pass]
  embed_scale: float = 1.0
  logit_softcap: float = 0.0  # > 0: logits <- cap * tanh(logits / cap)
  loop: Optional[tuple] = None
  # sandwich blocks with layer norms (Kopalorn): every norm is (x - mean) / sqrt(var + eps) * w + b, the sublayers'
  # normed results enter the stream times residual_mult, and a pass of the loop starts with x <- x + embedding output
  # (passes after the first) + step[pass] instead of the linear mix
  norm_kind: str = "rms"  # rms | layer
  residual_mult: float = 1.0
  loop_input: str = "linear"  # linear | add

  def layer_runs(self, layers=None) -> list:
    """[(layer, pass or -1)] in execution order for the given layers (default: all): a looped layer appears once per
    pass; pass >= 0 marks the first layer of a pass (where the pass's input mix happens)."""
    ids = list(range(self.num_layers)) if layers is None else list(layers)
    if not self.loop:
      return [(i, -1) for i in ids]
    a, b, times = self.loop
    inside = [i for i in ids if a <= i < b]
    if inside and (inside != list(range(a, b)) or ids[0] != 0):
      raise ValueError(f"layers {a}..{b - 1} run as a loop that mixes in the embedding output: a shard must hold all of "
                       "them together with the first layer")
    out = [(i, -1) for i in ids if i < a]
    for t in range(times if inside else 0):
      out += [(i, t if i == a else -1) for i in inside]
    return out + [(i, -1) for i in ids if i >= b]

  @property
  def is_mixed(self) -> bool:
    return self.layer_specs is not None

  @property
  def has_state(self) -> bool:
    """Some layer carries recurrent state per request (a state slot beside the KV pages)."""
    return bool(self.layer_specs) and any(s.state_dims is not None for s in self.layer_specs)

  @property
  def qkv_size(self) -> int:
    if self.is_mla:  # fused A projection: [q_a (or the full q) | kv_a latent | shared rope key]
      q = self.q_lora_rank or self.num_heads * (self.qk_nope_head_dim + self.qk_rope_head_dim)
      return q + self.kv_lora_rank + self.qk_rope_head_dim
    return (self.num_heads + 2 * self.num_kv_heads) * self.head_dim

  @property
  def is_mla(self) -> bool:
    return self.kv_lora_rank > 0

  @property
  def mla_dim(self) -> int:
    """Latent cache row: normalised kv latent + rotated shared key."""
    return self.kv_lora_rank + self.qk_rope_head_dim

  @property
  def rope_dim(self) -> int:
    return self.qk_rope_head_dim if self.is_mla else self.head_dim

  @property
  def rotary_dim(self) -> int:
    r = int(self.rope_dim * self.partial_rotary_factor)
    return r - (r % 2)

  @property
  def is_moe(self) -> bool:
    return self.num_experts > 0

  @property
  def expert_dim(self) -> int:
    return self.moe_intermediate_size or self.intermediate_size

  def moe_layer(self, i: int) -> bool:
    """Layer i has a routed-expert MLP (HF DeepseekV3DecoderLayer's rule; every layer for Mixtral)."""
    return self.is_moe and i >= self.first_k_dense_replace and i % max(1, self.moe_layer_freq) == 0

  def attn_scale(self) -> float:
    """Softmax scale: 1/sqrt(q.k dim); DeepSeek YaRN multiplies by mscale(factor, mscale_all_dim)^2."""
    import math
    dq = self.qk_nope_head_dim + self.qk_rope_head_dim if self.is_mla else self.head_dim
    s = dq ** -0.5
    sc = self.rope_scaling or {}
    if sc.get("rope_type") == "yarn" and sc.get("mscale_all_dim"):
      f = float(sc.get("factor", 1.0))
      m = 1.0 if f <= 1 else 0.1 * float(sc["mscale_all_dim"]) * math.log(f) + 1.0
      s *= m * m
    return s

  def params_per_layer(self, i: int = -1) -> int:
    D, F = self.hidden_size, self.intermediate_size
    if self.layer_specs:
      return sum(mixed_layer_params(D, s) for s in self.layer_specs) // len(self.layer_specs) if i < 0 else \
        mixed_layer_params(D, self.layer_specs[i])
    if self.is_mla:
      H, dn, dr, dv = self.num_heads, self.qk_nope_head_dim, self.qk_rope_head_dim, self.v_head_dim
      attn = D * self.qkv_size + (self.q_lora_rank * H * (dn + dr) if self.q_lora_rank else 0)
      attn += self.kv_lora_rank * H * (dn + dv) + H * dv * D
    else:
      attn = D * self.qkv_size + self.num_heads * self.head_dim * D
    moe = self.moe_layer(i) if i >= 0 else self.is_moe
    if moe:
      Fe = self.expert_dim
      mlp = 3 * D * Fe * (self.num_experts + self.n_shared_experts) + D * self.num_experts
    else:
      mlp = 3 * D * F
    return attn + mlp + 2 * D

  def num_params(self) -> int:
    emb = self.vocab_size * self.hidden_size
    layers = sum(self.params_per_layer(i) for i in range(self.num_layers))
    return layers + emb * (1 if self.tie_word_embeddings else 2) + self.hidden_size

  def to_dict(self) -> dict:
    d = asdict(self)
    d["eos_token_ids"] = list(self.eos_token_ids)
    return d

  def with_layers(self, n: int) -> "ModelConfig":
    if self.layer_specs is not None and n != len(self.layer_specs):
      specs = tuple(self.layer_specs[i % len(self.layer_specs)] for i in range(n))
      loop = self.loop if self.loop and self.loop[1] <= n else None  # (a loop that no longer fits is dropped)
      return replace(self, num_layers=n, layer_specs=specs, loop=loop)
    return replace(self, num_layers=n)


def _ln_sandwich_params(D: int, s: MixedLayerSpec) -> int:
  """Layers of layer-norm sandwich blocks: differential attention, mlstm, or gated attention beside lightning attention."""
  n = 4 * D  # the mixer's two norms with their biases
  a, w, r, f = s.dattn, s.wattn, s.rec, s.ffn
  if a is not None:
    n += D * (2 * a.heads * a.dim + 2 * a.kv_heads * a.dim + a.kv_heads * a.vdim + a.heads) + 4 * a.dim + a.heads * a.vdim * D
  if w is not None:
    n += (D + 1) * (w.heads * w.dim + w.kv_heads * (w.dim + w.vdim)) + 2 * w.heads * w.vdim * D + 2 * D
  if r is not None:
    n += D * r.heads * (2 * r.dim + 2 * r.vdim) + r.heads * r.vdim * (D + 1)
    if r.rule == "mlstm":
      n += 2 * r.heads * (D + 1)
  if f is not None:
    n += 4 * D + f.experts * (2 * D * f.ff + D + 1) + (2 * D * f.shared_ff + D if f.shared_ff else 0)
  return n


def mixed_layer_params(D: int, s: MixedLayerSpec) -> int:
  if s.dattn is not None or (s.rec is not None and s.rec.rule in ("lightning", "mlstm")):
    return _ln_sandwich_params(D, s)
  if s.lattn is not None:
    a, f = s.lattn, s.ffn
    qd = a.heads * (a.dim + a.rot_dim)
    n = 4 * D + (D * a.q_rank + a.q_rank + a.q_rank * qd if a.q_rank else D * qd)
    n += D * (a.kv_rank + a.rot_dim) + a.kv_rank + a.kv_rank * a.heads * (a.dim + a.vdim) + a.heads * a.vdim * D
    n += a.gate_rows * D + (a.heads if a.sink else 0)
    if f is not None and f.kind == "clamped_glu":
      n += 3 * D * f.ff
    elif f is not None:
      n += f.experts * (3 * D * f.ff + D) + 3 * D * f.shared_ff
    return n
  if s.wattn is not None or s.ssd is not None:
    n = 2 * D * (D + 1) + 2 * D  # the two sublayer gates and norms
    if s.wattn is not None:
      a = s.wattn
      n += (D + 1) * a.heads * a.dim + a.heads * a.vdim * D + a.heads
      if a.kv_from < 0:
        n += (D + 1) * a.kv_heads * (a.dim + a.vdim)
    if s.ssd is not None:
      m = s.ssd
      n += D * (2 * m.inner + 2 * m.groups * m.state + m.heads) + m.conv_channels * (m.conv + 1) + 3 * m.heads + \
        m.inner + m.inner * D
    f = s.ffn
    if f is not None and f.kind == "polynorm":
      n += 2 * D * f.ff + 4
    elif f is not None:
      n += f.experts * 2 * D * f.ff + f.experts * (D + 1) + (2 * D * f.shared_ff + D if f.shared_ff else 0)
    return n
  n = 1 + 2 * D + 3 * D * s.ff
  if s.attn is not None:
    a = s.attn
    n += D * a.dim * (a.heads + a.kv_heads * (1 if a.values_are_keys else 2)) + a.heads * a.vdim * D + a.heads
  if s.rec is not None:
    r = s.rec
    n += D * (2 * r.kv_heads * r.dim + 2 * r.heads * r.vdim) + r.heads * r.vdim * D + r.vdim
    if r.rule == "delta":
      n += r.conv * (2 * r.kv_heads * r.dim + r.heads * r.vdim) + 2 * r.heads * D + 2 * r.heads
    else:
      n += r.rank * (D + r.heads * r.dim) + r.heads * r.dim
  return n


def _rope_fields(cfg: dict) -> tuple:
  """(theta, scaling dict or None, partial_rotary_factor) from either config.json flavour: the hub's
  top-level `rope_theta` + `rope_scaling`, or transformers-5's `rope_parameters` (theta inside)."""
  rp = cfg.get("rope_parameters") or {}
  theta = float(cfg.get("rope_theta", rp.get("rope_theta", 10000.0)))
  partial = float(cfg.get("partial_rotary_factor", rp.get("partial_rotary_factor", 1.0)) or 1.0)
  scaling = cfg.get("rope_scaling")
  if not scaling and rp:
    scaling = {k: v for k, v in rp.items() if k not in ("rope_theta", "partial_rotary_factor")}
  if scaling:
    kind = scaling.get("rope_type", scaling.get("type", "default"))
    if kind in ("su", "longrope"):  # Phi-3 LongRoPE: needs the pretraining window and the extended one
      scaling = dict(scaling, rope_type="longrope",
                     original_max_position_embeddings=int(scaling.get("original_max_position_embeddings")
                                                          or cfg.get("original_max_position_embeddings", 4096)),
                     max_position_embeddings=int(cfg.get("max_position_embeddings", 131072)))
    elif kind == "yarn":
      scaling = dict(scaling, rope_type="yarn",
                     original_max_position_embeddings=int(scaling.get("original_max_position_embeddings")
                                                          or cfg.get("original_max_position_embeddings", 4096)))
    elif kind in ("default", None):
      scaling = None
  return theta, (scaling or None), partial


def _tarepel_config(cfg: dict) -> ModelConfig:
  """Tarepel config.json: {"architecture", "vocab", "width", "norm": {"eps"}, "logit_scale", "layers": [{"type":
  "parallel" | "gla", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}]}.  A "parallel" mixer holds a
  chunked gated attention ("left") beside a gated delta rule ("right") with their output scales; a "gla" mixer
  is one gated linear attention (its decay rank comes from the checkpoint, see models.weights)."""
  specs = []
  for i, L in enumerate(cfg["layers"]):
    m, mlp = L["mixer"], L.get("mlp")
    if mlp is not None and mlp.get("kind", "dense") != "dense":
      raise ValueError(f"layer {i}: unsupported feed-forward kind {mlp.get('kind')!r}")
    ff = int(mlp["ff"]) if mlp is not None else 0
    if L["type"] == "parallel":
      a, r = m["left"], m["right"]
      if int(a["vdim"]) != int(a["dim"]):
        raise ValueError(f"layer {i}: values are the keys, so vdim must equal dim")
      attn = GatedAttnSpec(int(a["heads"]), int(a["kv_heads"]), int(a["dim"]), int(a["vdim"]), int(a["mask"]["size"]),
                           int(a["rot"]["dims"]), float(a["rot"]["base"]), float(a["scale"]))
      rec = LinearRecurrenceSpec("delta", int(r["heads"]), int(r["kv_heads"]), int(r["dim"]), int(r["vdim"]),
                                 conv=int(r["conv"]))
      specs.append(MixedLayerSpec("parallel", attn, rec, float(m["left_scale"]), float(m["right_scale"]), ff))
    elif L["type"] == "gla":
      rec = LinearRecurrenceSpec("gla", int(m["heads"]), int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                                 tau=float(m["tau"]), rank=int(m.get("rank", 0)))
      specs.append(MixedLayerSpec("gla", None, rec, 1.0, 1.0, ff))
    else:
      raise ValueError(f"layer {i}: unknown layer type {L['type']!r}")
  first = next((s.attn for s in specs if s.attn is not None), None)
  return ModelConfig(
    model_type="tarepel", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]),
    intermediate_size=max([s.ff for s in specs] + [0]), num_layers=len(specs),
    num_heads=first.heads if first else 1, num_kv_heads=first.kv_heads if first else 1,
    head_dim=first.dim if first else 64, rms_norm_eps=float(cfg["norm"]["eps"]),
    rope_theta=first.rot_base if first else 10000.0, max_position_embeddings=int(cfg.get("max_positions", 1 << 20)),
    bos_token_id=int(cfg.get("bos_token_id", 0)), eos_token_ids=tuple(cfg.get("eos_token_ids", ())),
    layer_specs=tuple(specs), logit_scale=float(cfg.get("logit_scale", 1.0)))


def _mogelix_config(cfg: dict) -> ModelConfig:
  """Mogelix config.json: {"architecture", "vocab", "width", "norm": {"eps"}, "postln_alpha", "layers": [{"type":
  "attention" | "mamba2", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"}, "router":
  {"experts", "top"}, "shared": {"ff"}} | null}]}.  An attention mixer without "mask" sees every earlier token, without
  "pool" no pooled blocks, without "rot" nothing is rotated; "kv_from": j borrows layer j's keys and values."""
  specs = []
  for i, L in enumerate(cfg["layers"]):
    m, mlp = L["mixer"], L.get("mlp")
    ffn = None
    if mlp is not None:
      kind = mlp.get("kind", "dense")
      if kind == "dense":
        ffn = FeedForwardSpec("polynorm", int(mlp["ff"]))
      elif kind == "moe":
        sh = mlp.get("shared")
        ffn = FeedForwardSpec("relu2_moe", int(mlp["expert"]["ff"]), int(mlp["router"]["experts"]),
                              int(mlp["router"]["top"]), int(sh["ff"]) if sh else 0)
        if not 1 <= ffn.top <= ffn.experts:
          raise ValueError(f"layer {i}: top {ffn.top} of {ffn.experts} experts")
      else:
        raise ValueError(f"layer {i}: unsupported feed-forward kind {kind!r}")
    if L["type"] == "attention":
      rot, mask = m.get("rot") or {}, m.get("mask") or {}
      sc = rot.get("scaling")
      scaling = (float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])) if sc else None
      src = m.get("kv_from")
      a = WindowAttnSpec(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), int(mask.get("size", 0)),
                         int(mask.get("pool", 0)) if mask.get("size") else 0, int(rot.get("dims", 0)),
                         float(rot.get("base", 10000.0)), scaling, float(m["scale"]), kv_from=-1 if src is None else int(src))
      if a.heads % a.kv_heads or a.rot_dims % 2 or a.rot_dims > a.dim:
        raise ValueError(f"layer {i}: heads {a.heads} / kv_heads {a.kv_heads} / rotary dims {a.rot_dims} do not fit")
      if a.kv_from >= 0:
        b = specs[a.kv_from].wattn if 0 <= a.kv_from < i else None
        if b is None or b.kv_from >= 0 or (b.kv_heads, b.dim, b.vdim) != (a.kv_heads, a.dim, a.vdim):
          raise ValueError(f"layer {i}: kv_from {a.kv_from} must name an earlier attention layer with projections of "
                           "its own and the same key / value heads")
      specs.append(MixedLayerSpec("attention", wattn=a, ffn=ffn))
    elif L["type"] == "mamba2":
      s = SSDSpec(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups", 1)), int(m.get("conv", 1)),
                  int(m.get("norm_groups", 1)))
      if s.heads % s.groups or s.inner % s.norm_groups or s.conv < 1:
        raise ValueError(f"layer {i}: heads {s.heads} / groups {s.groups} / norm_groups {s.norm_groups} do not fit")
      specs.append(MixedLayerSpec("mamba2", ssd=s, ffn=ffn))
    else:
      raise ValueError(f"layer {i}: unknown layer type {L['type']!r}")
  first = next((s.wattn for s in specs if s.wattn is not None), None)
  return ModelConfig(
    model_type="mogelix", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]),
    intermediate_size=max([s.ffn.ff for s in specs if s.ffn is not None] + [0]), num_layers=len(specs),
    num_heads=first.heads if first else 1, num_kv_heads=first.kv_heads if first else 1,
    head_dim=first.dim if first else 64, rms_norm_eps=float(cfg["norm"]["eps"]),
    rope_theta=first.rot_base if first else 10000.0, max_position_embeddings=int(cfg.get("max_positions", 1 << 20)),
    bos_token_id=int(cfg.get("bos_token_id", 0)), eos_token_ids=tuple(cfg.get("eos_token_ids", ())),
    layer_specs=tuple(specs), block="postln", postln_alpha=float(cfg.get("postln_alpha", 1.0)))


_LATENT_KINDS = {
  # layer type: (queries through a latent, interleaved rotation pairs, sliding window, sink, output gate)
  "latent_attention": (False, True, False, False, "elem"),
  "latent_attention_2": (True, False, True, False, "head"),
  "latent_attention_3": (True, False, False, True, "none"),
}


def _nenizen_config(cfg: dict) -> ModelConfig:
  """Nenizen config.json: {"architecture", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"}, "logit_softcap",
  "loop": {"start", "stop", "times"} | null, "layers": [{"type": "latent_attention" | "latent_attention_2" |
  "latent_attention_3", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "rot": {"base", "dims"},
  "scale", "mask": {"size"}}, "mlp": {"kind": "dense", "ff", "limit"} | {"kind": "moe", "expert": {"ff"}, "router":
  {"experts", "top"}, "shared": {"ff"}} | null}]}."""
  specs = []
  for i, L in enumerate(cfg["layers"]):
    m, mlp = L["mixer"], L.get("mlp")
    if L["type"] not in _LATENT_KINDS:
      raise ValueError(f"layer {i}: unknown layer type {L['type']!r}")
    qlat, inter, windowed, sink, gate = _LATENT_KINDS[L["type"]]
    rot = m.get("rot") or {}
    a = LatentAttnSpec(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]),
                       int(m["q_rank"]) if qlat else 0, int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), inter,
                       float(m["scale"]), int(m["mask"]["size"]) if windowed else 0, sink, gate)
    if a.rot_dims % 2 or a.rot_dims > a.rot_dim or min(a.heads, a.dim + a.rot_dim, a.vdim, a.kv_rank) < 1 or \
       (windowed and a.window < 1):
      raise ValueError(f"layer {i}: sizes of the latent attention do not fit")
    ffn = None
    if mlp is not None:
      kind = mlp.get("kind", "dense")
      if kind == "dense":
        ffn = FeedForwardSpec("clamped_glu", int(mlp["ff"]), limit=float(mlp["limit"]))
      elif kind == "moe":
        sh = mlp.get("shared")
        ffn = FeedForwardSpec("silu_moe", int(mlp["expert"]["ff"]), int(mlp["router"]["experts"]),
                              int(mlp["router"]["top"]), int(sh["ff"]) if sh else 0)
        if not 1 <= ffn.top <= ffn.experts:
          raise ValueError(f"layer {i}: top {ffn.top} of {ffn.experts} experts")
      else:
        raise ValueError(f"layer {i}: unsupported feed-forward kind {kind!r}")
    specs.append(MixedLayerSpec(L["type"], lattn=a, ffn=ffn))
  lp = cfg.get("loop")
  loop = None
  if lp and int(lp.get("times", 1)) >= 1 and int(lp["stop"]) > int(lp["start"]):
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
    if not 0 <= loop[0] < loop[1] <= len(specs):
      raise ValueError(f"loop {loop} outside the {len(specs)} layers")
  first = specs[0].lattn
  return ModelConfig(
    model_type="nenizen", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]),
    intermediate_size=max([s.ffn.ff for s in specs if s.ffn is not None] + [0]), num_layers=len(specs),
    num_heads=first.heads, num_kv_heads=1, head_dim=first.dim + first.rot_dim, rms_norm_eps=float(cfg["norm"]["eps"]),
    rope_theta=first.rot_base, max_position_embeddings=int(cfg.get("max_positions", 1 << 20)),
    tie_word_embeddings=True, bos_token_id=int(cfg.get("bos_token_id", 0)), eos_token_ids=tuple(cfg.get("eos_token_ids", ())),
    layer_specs=tuple(specs), block="sandwich", embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
    logit_softcap=float(cfg.get("logit_softcap") or 0.0), loop=loop)


def _kopalorn_config(cfg: dict) -> ModelConfig:
  """Kopalorn config.json: {"architecture", "vocab", "width", "norm": {"eps"}, "residual_mult", "loop": {"start", "stop",
  "times"} | null, "layers": [{"type": "attention" | "mlstm" | "parallel", "mixer": {...}, "mlp": {"kind": "moe", "expert":
  {"ff"}, "router": {"experts", "top", "scale", "groups": {"count", "keep"}}, "shared": {"ff"}} | null}]}.  "attention":
  {"heads", "kv_heads", "dim", "vdim", "diff", "scale", "mask": {"size"}, "rot": {"base", "dims"}}; "mlstm": {"heads", "dim",
  "vdim", "gate_cap"}; "parallel": {"left": {"heads", "kv_heads", "dim", "vdim", "scale"}, "right": {"heads", "dim", "vdim",
  "decay": [one per head]}}.  Without "mask" every earlier token is seen, without "rot" nothing is rotated."""
  specs = []
  for i, L in enumerate(cfg["layers"]):
    m, mlp = L["mixer"], L.get("mlp")
    ffn = None
    if mlp is not None:
      if mlp.get("kind", "moe") != "moe":
        raise ValueError(f"layer {i}: unsupported feed-forward kind {mlp.get('kind')!r}")
      r, sh = mlp["router"], mlp.get("shared")
      gr = r.get("groups") or {}
      ffn = FeedForwardSpec("relu2_moe", int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), int(sh["ff"]) if sh else 0,
                            route="sigmoid_groups", groups=int(gr.get("count", 1)), keep=int(gr.get("keep", gr.get("count", 1))),
                            route_scale=float(r.get("scale", 1.0)))
      if not 1 <= ffn.top <= ffn.experts or ffn.experts % ffn.groups or not 1 <= ffn.keep <= ffn.groups or \
         ffn.keep * (ffn.experts // ffn.groups) < ffn.top:
        raise ValueError(f"layer {i}: top {ffn.top} of {ffn.experts} experts in {ffn.groups} groups, {ffn.keep} kept")
    if L["type"] == "attention":
      rot, mask = m.get("rot") or {}, m.get("mask") or {}
      a = DiffAttnSpec(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), int(mask.get("size", 0)),
                       int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), float(m["scale"]), float(m["diff"]))
      if a.heads % a.kv_heads or a.rot_dims % 2 or a.rot_dims > a.dim:
        raise ValueError(f"layer {i}: heads {a.heads} / kv_heads {a.kv_heads} / rotary dims {a.rot_dims} do not fit")
      specs.append(MixedLayerSpec("attention", dattn=a, ffn=ffn))
    elif L["type"] == "mlstm":
      r = LinearRecurrenceSpec("mlstm", int(m["heads"]), int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                               gate_cap=float(m["gate_cap"]))
      specs.append(MixedLayerSpec("mlstm", rec=r, ffn=ffn))
    elif L["type"] == "parallel":
      a, r = m["left"], m["right"]
      w = WindowAttnSpec(int(a["heads"]), int(a["kv_heads"]), int(a["dim"]), int(a["vdim"]), 0, 0, 0, 10000.0, None,
                         float(a["scale"]), qk_norm=False, bias=True, sink=False, gate="elem")
      if w.heads % w.kv_heads:
        raise ValueError(f"layer {i}: heads {w.heads} / kv_heads {w.kv_heads} do not fit")
      decays = tuple(float(x) for x in r["decay"])
      if len(decays) != int(r["heads"]):
        raise ValueError(f"layer {i}: {len(decays)} decays for {r['heads']} heads")
      rec = LinearRecurrenceSpec("lightning", int(r["heads"]), int(r["heads"]), int(r["dim"]), int(r["vdim"]), decays=decays)
      specs.append(MixedLayerSpec("parallel", rec=rec, wattn=w, ffn=ffn))
    else:
      raise ValueError(f"layer {i}: unknown layer type {L['type']!r}")
  lp = cfg.get("loop")
  loop = None
  if lp and int(lp.get("times", 1)) >= 1 and int(lp["stop"]) > int(lp["start"]):
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
    if not 0 <= loop[0] < loop[1] <= len(specs):
      raise ValueError(f"loop {loop} outside the {len(specs)} layers")
  first = next((s.dattn or s.wattn for s in specs if s.dattn or s.wattn), None)
  return ModelConfig(
    model_type="kopalorn", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]),
    intermediate_size=max([s.ffn.ff for s in specs if s.ffn is not None] + [0]), num_layers=len(specs),
    num_heads=first.heads if first else 1, num_kv_heads=first.kv_heads if first else 1, head_dim=first.dim if first else 64,
    rms_norm_eps=float(cfg["norm"]["eps"]), rope_theta=getattr(first, "rot_base", 10000.0),
    max_position_embeddings=int(cfg.get("max_positions", 1 << 20)), bos_token_id=int(cfg.get("bos_token_id", 0)),
    eos_token_ids=tuple(cfg.get("eos_token_ids", ())), layer_specs=tuple(specs), block="sandwich", loop=loop,
    norm_kind="layer", residual_mult=float(cfg.get("residual_mult", 1.0)), loop_input="add")


def from_hf_config(cfg: dict) -> ModelConfig:
  if cfg.get("architecture") == "Kopalorn":
    return _kopalorn_config(cfg)
  if cfg.get("architecture") == "Nenizen":
    return _nenizen_config(cfg)
  if cfg.get("architecture") == "Tarepel":
    return _tarepel_config(cfg)
  if cfg.get("architecture") == "Mogelix":
    return _mogelix_config(cfg)
  mt = cfg.get("model_type", "llama")
  if mt == "llava":
    return _llava_config(cfg)
  H = int(cfg["num_attention_heads"])
  D = int(cfg["hidden_size"])
  eos = cfg.get("eos_token_id")
  eos_ids = tuple(eos) if isinstance(eos, (list, tuple)) else ((int(eos),) if eos is not None else (2,))
  theta, scaling, partial = _rope_fields(cfg)
  if cfg.get("sliding_window") and mt == "phi3":
    import warnings
    warnings.warn(f"phi3 sliding_window={cfg['sliding_window']} is not applied (full causal attention)")
  if mt in ("deepseek_v2", "deepseek_v3"):
    return _deepseek_config(cfg, mt, theta, scaling, eos_ids)
  return ModelConfig(
    model_type=mt,
    vocab_size=int(cfg["vocab_size"]),
    hidden_size=D,
    intermediate_size=int(cfg["intermediate_size"]),
    num_layers=int(cfg["num_hidden_layers"]),
    num_heads=H,
    num_kv_heads=int(cfg.get("num_key_value_heads", H)),
    head_dim=int(cfg.get("head_dim") or D // H),
    rms_norm_eps=float(cfg.get("rms_norm_eps", 1e-5)),
    rope_theta=theta,
    rope_scaling=scaling,
    max_position_embeddings=int(cfg.get("max_position_embeddings", 8192)),
    tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
    attention_bias=bool(cfg.get("attention_bias", mt == "qwen2")),
    num_experts=int(cfg.get("num_local_experts", 0)),
    num_experts_per_tok=int(cfg.get("num_experts_per_tok", 0)),
    bos_token_id=int(cfg.get("bos_token_id", 1) or 1),
    eos_token_ids=eos_ids,
    partial_rotary_factor=partial,
  )


def _deepseek_config(cfg: dict, mt: str, theta: float, scaling, eos_ids) -> ModelConfig:
  """DeepSeek-V2 / V3 (and R1): MLA attention, DeepSeekMoE with shared experts."""
  H = int(cfg["num_attention_heads"])
  v3 = mt == "deepseek_v3"
  return ModelConfig(
    model_type=mt,
    vocab_size=int(cfg["vocab_size"]),
    hidden_size=int(cfg["hidden_size"]),
    intermediate_size=int(cfg["intermediate_size"]),
    num_layers=int(cfg["num_hidden_layers"]),
    num_heads=H,
    num_kv_heads=1,  # one shared latent per token
    head_dim=int(cfg["qk_nope_head_dim"]) + int(cfg["qk_rope_head_dim"]),
    rms_norm_eps=float(cfg.get("rms_norm_eps", 1e-6)),
    rope_theta=theta,
    rope_scaling=scaling,
    max_position_embeddings=int(cfg.get("max_position_embeddings", 4096)),
    tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
    attention_bias=bool(cfg.get("attention_bias", False)),
    num_experts=int(cfg.get("n_routed_experts") or 0),
    num_experts_per_tok=int(cfg.get("num_experts_per_tok") or 0),
    bos_token_id=int(cfg.get("bos_token_id", 0) or 0),
    eos_token_ids=eos_ids,
    q_lora_rank=int(cfg.get("q_lora_rank") or 0),
    kv_lora_rank=int(cfg["kv_lora_rank"]),
    qk_nope_head_dim=int(cfg["qk_nope_head_dim"]),
    qk_rope_head_dim=int(cfg["qk_rope_head_dim"]),
    v_head_dim=int(cfg["v_head_dim"]),
    moe_intermediate_size=int(cfg.get("moe_intermediate_size") or 0),
    n_shared_experts=int(cfg.get("n_shared_experts") or 0),
    first_k_dense_replace=int(cfg.get("first_k_dense_replace") or 0),
    moe_layer_freq=int(cfg.get("moe_layer_freq") or 1),
    routed_scaling_factor=float(cfg.get("routed_scaling_factor") or 1.0),
    topk_method="noaux_tc" if v3 else str(cfg.get("topk_method") or "greedy"),
    n_group=int(cfg.get("n_group") or 1),
    topk_group=int(cfg.get("topk_group") or 1),
    # HF's V2 router never renormalises (norm_topk_prob is ignored there); V3 follows the flag
    norm_topk_prob=bool(cfg.get("norm_topk_prob", True)) if v3 else False,
    scoring_func="sigmoid" if v3 else "softmax",
  )


_VISION_KEYS = ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads", "patch_size",
                "image_size", "layer_norm_eps", "hidden_act", "num_channels")


def _llava_config(cfg: dict) -> ModelConfig:
  """HF LlavaConfig: a Llama text model + CLIP vision tower (vision_config) + projector."""
  text = dict(cfg.get("text_config") or {})
  text.setdefault("model_type", "llama")
  for k in ("bos_token_id", "eos_token_id", "pad_token_id"):
    if k not in text and k in cfg:
      text[k] = cfg[k]
  lm = from_hf_config(text)
  vc = cfg.get("vision_config") or {}
  vision = {k: vc[k] for k in _VISION_KEYS if k in vc}
  vision.setdefault("num_channels", 3)
  vision.setdefault("hidden_act", "quick_gelu")
  vision.setdefault("layer_norm_eps", 1e-5)
  fl = cfg.get("vision_feature_layer", -2)
  if isinstance(fl, (list, tuple)):
    raise ValueError("multi-layer vision features are not supported")
  return replace(lm, model_type="llava", vision=vision,
                 image_token_id=int(cfg.get("image_token_index", cfg.get("image_token_id", 32000))),
                 vision_feature_layer=int(fl), vision_select=str(cfg.get("vision_feature_select_strategy", "default")),
                 projector_act=str(cfg.get("projector_hidden_act", "gelu")))


def load_config(model_dir: str | Path) -> ModelConfig:
  with open(Path(model_dir) / "config.json") as f:
    return from_hf_config(json.load(f))


_L3 = dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
           original_max_position_embeddings=8192)
_L31 = dict(_L3, factor=8.0)
_DS_YARN = dict(rope_type="yarn", factor=40.0, original_max_position_embeddings=4096, beta_fast=32, beta_slow=1,
                mscale=1.0, mscale_all_dim=1.0)  # DeepSeek-V3 / R1
_DS2_YARN = dict(_DS_YARN, mscale=0.707, mscale_all_dim=0.707)  # DeepSeek-V2(-Lite)

PRESETS: dict[str, ModelConfig] = {
  "llama-3.2-1b": ModelConfig("llama", 128256, 2048, 8192, 16, 32, 8, 64, 1e-5, 500000.0, _L3, 131072, True),
  "llama-3.2-3b": ModelConfig("llama", 128256, 3072, 8192, 28, 24, 8, 128, 1e-5, 500000.0, _L3, 131072, True),
  "llama-3-8b": ModelConfig("llama", 128256, 4096, 14336, 32, 32, 8, 128, 1e-5, 500000.0, None, 8192, False),
  "llama-3.1-8b": ModelConfig("llama", 128256, 4096, 14336, 32, 32, 8, 128, 1e-5, 500000.0, _L31, 131072, False),
  "llama-3-70b": ModelConfig("llama", 128256, 8192, 28672, 80, 64, 8, 128, 1e-5, 500000.0, None, 8192, False),
  "llama-3.1-70b": ModelConfig("llama", 128256, 8192, 28672, 80, 64, 8, 128, 1e-5, 500000.0, _L31, 131072, False),
  "llama-3.3-70b": ModelConfig("llama", 128256, 8192, 28672, 80, 64, 8, 128, 1e-5, 500000.0, _L31, 131072, False),
  "qwen-2.5-0.5b": ModelConfig("qwen2", 151936, 896, 4864, 24, 14, 2, 64, 1e-6, 1000000.0, None, 32768, True, True,
                               bos_token_id=151643, eos_token_ids=(151645, 151643)),
  "qwen-2.5-1.5b": ModelConfig("qwen2", 151936, 1536, 8960, 28, 12, 2, 128, 1e-6, 1000000.0, None, 32768, True, True,
                               bos_token_id=151643, eos_token_ids=(151645, 151643)),
  "qwen-2.5-7b": ModelConfig("qwen2", 152064, 3584, 18944, 28, 28, 4, 128, 1e-6, 1000000.0, None, 32768, False, True,
                             bos_token_id=151643, eos_token_ids=(151645, 151643)),
  "qwen-2.5-3b": ModelConfig("qwen2", 151936, 2048, 11008, 36, 16, 2, 128, 1e-6, 1000000.0, None, 32768, True, True,
                             bos_token_id=151643, eos_token_ids=(151645, 151643)),
  "qwen-2.5-14b": ModelConfig("qwen2", 152064, 5120, 13824, 48, 40, 8, 128, 1e-5, 1000000.0, None, 32768, False, True,
                              bos_token_id=151643, eos_token_ids=(151645, 151643)),
  "qwen-2.5-32b": ModelConfig("qwen2", 152064, 5120, 27648, 64, 40, 8, 128, 1e-5, 1000000.0, None, 32768, False, True,
                              bos_token_id=151643, eos_token_ids=(151645, 151643)),
  "qwen-2.5-72b": ModelConfig("qwen2", 152064, 8192, 29568, 80, 64, 8, 128, 1e-5, 1000000.0, None, 32768, False, True,
                              bos_token_id=151643, eos_token_ids=(151645, 151643)),
  "llama-3.1-405b": ModelConfig("llama", 128256, 16384, 53248, 126, 128, 8, 128, 1e-5, 500000.0, _L31, 131072, False),
  "mistral-large": ModelConfig("mistral", 32768, 12288, 28672, 88, 96, 8, 128, 1e-5, 1000000.0, None, 131072, False,
                               bos_token_id=1, eos_token_ids=(2,)),
  "mistral-7b": ModelConfig("mistral", 32768, 4096, 14336, 32, 32, 8, 128, 1e-5, 1000000.0, None, 32768, False,
                            bos_token_id=1, eos_token_ids=(2,)),
  "mixtral-8x7b": ModelConfig("mixtral", 32000, 4096, 14336, 32, 32, 8, 128, 1e-5, 1000000.0, None, 32768, False,
                              num_experts=8, num_experts_per_tok=2, bos_token_id=1, eos_token_ids=(2,)),
  "mistral-nemo": ModelConfig("mistral", 131072, 5120, 14336, 40, 32, 8, 128, 1e-5, 1000000.0, None, 131072, False,
                              bos_token_id=1, eos_token_ids=(2,)),
  # Phi-4-mini (HF Phi3ForCausalLM): fused qkv / gate_up checkpoints, RoPE on 96 of 128 head dims, LongRoPE.
  # The hub config's 48 short / long LongRoPE factors are not available offline: the preset uses unit
  # factors (plain RoPE inside the 4k pretraining window, same attention factor); a downloaded config.json
  # carries the real ones.
  "phi-4-mini-instruct": ModelConfig("phi3", 200064, 3072, 8192, 32, 24, 8, 128, 1e-5, 10000.0,
                                     dict(rope_type="longrope", short_factor=[1.0] * 48, long_factor=[1.0] * 48,
                                          original_max_position_embeddings=4096, max_position_embeddings=131072),
                                     131072, True, bos_token_id=199999, eos_token_ids=(199999, 200020),
                                     partial_rotary_factor=0.75),
  # DeepSeek (HF DeepseekV2/V3ForCausalLM): MLA (latent 512 + rope 64), DeepSeekMoE with shared experts
  "deepseek-coder-v2-lite": ModelConfig("deepseek_v2", 102400, 2048, 10944, 27, 16, 1, 192, 1e-6, 10000.0,
                                        _DS2_YARN, 163840, False, num_experts=64, num_experts_per_tok=6,
                                        bos_token_id=100000, eos_token_ids=(100001,), kv_lora_rank=512,
                                        qk_nope_head_dim=128, qk_rope_head_dim=64, v_head_dim=128,
                                        moe_intermediate_size=1408, n_shared_experts=2, first_k_dense_replace=1,
                                        norm_topk_prob=False),
  "deepseek-v3": ModelConfig("deepseek_v3", 129280, 7168, 18432, 61, 128, 1, 192, 1e-6, 10000.0, _DS_YARN, 163840,
                             False, num_experts=256, num_experts_per_tok=8, bos_token_id=0, eos_token_ids=(1,),
                             q_lora_rank=1536, kv_lora_rank=512, qk_nope_head_dim=128, qk_rope_head_dim=64,
                             v_head_dim=128, moe_intermediate_size=2048, n_shared_experts=1, first_k_dense_replace=3,
                             routed_scaling_factor=2.5, topk_method="noaux_tc", n_group=8, topk_group=4,
                             norm_topk_prob=True, scoring_func="sigmoid"),
  # LLaVA-1.5-7B (HF LlavaForConditionalGeneration): Vicuna-7B text model + CLIP ViT-L/14-336 + MLP projector
  "llava-1.5-7b-hf": ModelConfig("llava", 32064, 4096, 11008, 32, 32, 32, 128, 1e-5, 10000.0, None, 4096, False,
                                 bos_token_id=1, eos_token_ids=(2,), image_token_id=32000,
                                 vision=dict(hidden_size=1024, intermediate_size=4096, num_hidden_layers=24,
                                             num_attention_heads=16, patch_size=14, image_size=336,
                                             layer_norm_eps=1e-5, hidden_act="quick_gelu", num_channels=3)),
  # small shapes for tests / CPU plumbing
  "tiny-llama": ModelConfig("llama", 512, 256, 512, 4, 4, 2, 64, 1e-5, 10000.0, None, 2048, False,
                            bos_token_id=1, eos_token_ids=(2,)),
  # 8 layers: multi-rank rehearsals of the 8-GPU ring (one layer per rank)
  "tiny-llama-8l": ModelConfig("llama", 512, 256, 512, 8, 4, 2, 64, 1e-5, 10000.0, None, 2048, False,
                               bos_token_id=1, eos_token_ids=(2,)),
  "tiny-llama-d64": ModelConfig("llama", 1024, 256, 512, 6, 4, 2, 64, 1e-5, 10000.0, _L3, 4096, True,
                                bos_token_id=1, eos_token_ids=(2,)),
  "tiny-qwen": ModelConfig("qwen2", 512, 256, 512, 4, 4, 2, 64, 1e-6, 1000000.0, None, 2048, True, True,
                           bos_token_id=1, eos_token_ids=(2,)),
  "tiny-mixtral": ModelConfig("mixtral", 512, 256, 512, 4, 4, 2, 64, 1e-5, 10000.0, None, 2048, False,
                              num_experts=4, num_experts_per_tok=2, bos_token_id=1, eos_token_ids=(2,)),
  "tiny-phi3": ModelConfig("phi3", 512, 256, 512, 4, 2, 1, 128, 1e-5, 10000.0,
                           dict(rope_type="longrope", short_factor=[1.0 + 0.05 * i for i in range(48)],
                                long_factor=[2.0 + 0.1 * i for i in range(48)], original_max_position_embeddings=64,
                                max_position_embeddings=2048), 2048, True, bos_token_id=1, eos_token_ids=(2,),
                           partial_rotary_factor=0.75),
  "tiny-llava": ModelConfig("llava", 512, 256, 512, 4, 4, 2, 64, 1e-5, 10000.0, None, 2048, False, bos_token_id=1,
                            eos_token_ids=(2,), image_token_id=500,
                            vision=dict(hidden_size=128, intermediate_size=256, num_hidden_layers=3, num_attention_heads=4,
                                        patch_size=14, image_size=56, layer_norm_eps=1e-5, hidden_act="quick_gelu",
                                        num_channels=3)),
  "tiny-deepseek-v2": ModelConfig("deepseek_v2", 512, 256, 512, 3, 4, 1, 192, 1e-6, 10000.0, None, 2048, False,
                                  num_experts=8, num_experts_per_tok=2, bos_token_id=1, eos_token_ids=(2,),
                                  kv_lora_rank=256, qk_nope_head_dim=128, qk_rope_head_dim=64, v_head_dim=128,
                                  moe_intermediate_size=256, n_shared_experts=2, first_k_dense_replace=1,
                                  topk_method="group_limited_greedy", n_group=4, topk_group=2, norm_topk_prob=False,
                                  routed_scaling_factor=1.5),
  "tiny-deepseek-v3": ModelConfig("deepseek_v3", 512, 256, 512, 3, 16, 1, 192, 1e-6, 10000.0,
                                  dict(_DS_YARN, original_max_position_embeddings=64), 2048, False, num_experts=16,
                                  num_experts_per_tok=4, bos_token_id=1, eos_token_ids=(2,), q_lora_rank=256,
                                  kv_lora_rank=256, qk_nope_head_dim=128, qk_rope_head_dim=64, v_head_dim=128,
                                  moe_intermediate_size=256, n_shared_experts=1, first_k_dense_replace=1,
                                  routed_scaling_factor=2.5, topk_method="noaux_tc", n_group=4, topk_group=2,
                                  norm_topk_prob=True, scoring_func="sigmoid"),
}
TINY_TAREPEL = {
  "architecture": "Tarepel", "vocab": 320, "width": 128, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
  "layers": [
    {"type": "parallel", "mlp": {"kind": "dense", "ff": 192},
     "mixer": {"left": {"heads": 4, "kv_heads": 1, "dim": 32, "vdim": 32, "mask": {"size": 48},
                        "rot": {"base": 10000.0, "dims": 16}, "scale": 0.2},
               "right": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "conv": 3},
               "left_scale": 0.7, "right_scale": 0.9}},
    {"type": "gla", "mlp": None, "mixer": {"heads": 2, "dim": 32, "vdim": 64, "tau": 8.0}},
    {"type": "gla", "mlp": {"kind": "dense", "ff": 128}, "mixer": {"heads": 4, "dim": 16, "vdim": 32, "tau": 12.0}},
    {"type": "parallel", "mlp": {"kind": "dense", "ff": 192},
     "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 64, "mask": {"size": 32},
                        "rot": {"base": 50000.0, "dims": 64}, "scale": 0.125},
               "right": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 32, "conv": 4},
               "left_scale": 1.0, "right_scale": 0.5}},
  ]}
PRESETS["tiny-tarepel"] = _tarepel_config(TINY_TAREPEL)
_TINY_ROT = {"base": 10000.0, "dims": 16, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}
_TINY_MOE = {"kind": "moe", "expert": {"ff": 48}, "router": {"experts": 6, "top": 2}, "shared": {"ff": 64}}
TINY_MOGELIX = {
  "architecture": "Mogelix", "vocab": 288, "width": 96, "norm": {"eps": 1e-5}, "postln_alpha": 1.5,
  "layers": [
    {"type": "mamba2", "mlp": {"kind": "dense", "ff": 160},
     "mixer": {"heads": 4, "vdim": 16, "state": 24, "groups": 2, "conv": 3, "norm_groups": 2}},
    {"type": "attention", "mlp": _TINY_MOE,
     "mixer": {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 32, "mask": {"size": 20, "pool": 5}, "rot": _TINY_ROT,
               "scale": 0.3}},
    {"type": "attention", "mlp": None,
     "mixer": {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 32, "kv_from": 1, "mask": {"size": 9, "pool": 3},
               "rot": _TINY_ROT, "scale": 0.25}},
    {"type": "mamba2", "mlp": _TINY_MOE,
     "mixer": {"heads": 2, "vdim": 32, "state": 16, "groups": 1, "conv": 4, "norm_groups": 1}},
  ]}
PRESETS["tiny-mogelix"] = _mogelix_config(TINY_MOGELIX)
_TINY_LMOE = {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 5, "top": 3}, "shared": {"ff": 24}}
TINY_NENIZEN = {
  "architecture": "Nenizen", "vocab": 272, "width": 80, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
  "logit_softcap": 20.0, "loop": {"start": 1, "stop": 4, "times": 2},
  "layers": [
    {"type": "latent_attention_2", "mlp": {"kind": "dense", "ff": 112, "limit": 1.5},
     "mixer": {"heads": 3, "dim": 24, "rot_dim": 8, "vdim": 20, "kv_rank": 48, "q_rank": 40, "mask": {"size": 11},
               "rot": {"base": 10000.0, "dims": 8}, "scale": 0.2}},
    {"type": "latent_attention", "mlp": _TINY_LMOE,
     "mixer": {"heads": 5, "dim": 8, "rot_dim": 16, "vdim": 16, "kv_rank": 32,
               "rot": {"base": 50000.0, "dims": 16}, "scale": 0.25}},
    {"type": "latent_attention_3", "mlp": None,
     "mixer": {"heads": 2, "dim": 16, "rot_dim": 16, "vdim": 40, "kv_rank": 24, "q_rank": 16,
               "rot": {"base": 1000.0, "dims": 12}, "scale": 0.3}},
    {"type": "latent_attention_2", "mlp": _TINY_LMOE,
     "mixer": {"heads": 4, "dim": 16, "rot_dim": 4, "vdim": 8, "kv_rank": 64, "q_rank": 24, "mask": {"size": 70},
               "rot": {"base": 10000.0, "dims": 4}, "scale": 0.2}},
    {"type": "latent_attention_3", "mlp": {"kind": "dense", "ff": 96, "limit": 3.0},
     "mixer": {"heads": 4, "dim": 16, "rot_dim": 16, "vdim": 16, "kv_rank": 32, "q_rank": 48,
               "rot": {"base": 10000.0, "dims": 16}, "scale": 0.2}},
  ]}
PRESETS["tiny-nenizen"] = _nenizen_config(TINY_NENIZEN)
_TINY_GMOE = {"kind": "moe", "expert": {"ff": 40}, "shared": {"ff": 56},
              "router": {"experts": 6, "top": 3, "scale": 1.5, "groups": {"count": 3, "keep": 2}}}
TINY_KOPALORN = {
  "architecture": "Kopalorn", "vocab": 304, "width": 112, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
  "loop": {"start": 1, "stop": 3, "times": 3},
  "layers": [
    {"type": "mlstm", "mlp": _TINY_GMOE, "mixer": {"heads": 2, "dim": 24, "vdim": 40, "gate_cap": 10.0}},
    {"type": "attention", "mlp": _TINY_GMOE,
     "mixer": {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "diff": 0.3, "scale": 0.3, "mask": {"size": 21},
               "rot": {"base": 10000.0, "dims": 8}}},
    {"type": "parallel", "mlp": None,
     "mixer": {"left": {"heads": 4, "kv_heads": 1, "dim": 24, "vdim": 16, "scale": 0.2},
               "right": {"heads": 3, "dim": 16, "vdim": 24, "decay": [0.5, 0.9, 0.99]}}},
    {"type": "attention", "mlp": {"kind": "moe", "expert": {"ff": 48}, "shared": None,
                                  "router": {"experts": 4, "top": 1, "scale": 1.0, "groups": {"count": 1, "keep": 1}}},
     "mixer": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 32, "diff": 0.6, "scale": 0.18, "mask": {"size": 70},
               "rot": {"base": 1000.0, "dims": 32}}},
  ]}
PRESETS["tiny-kopalorn"] = _kopalorn_config(TINY_KOPALORN)
# aliases of the reference's model cards that share an architecture
for _alias, _base in {"llama-3.1-70b-bf16": "llama-3.1-70b", "nemotron-70b": "llama-3.1-70b",
                      "deepseek-r1-distill-llama-70b": "llama-3.1-70b", "deepseek-r1-distill-llama-8b": "llama-3.1-8b",
                      "qwen-2.5-coder-1.5b": "qwen-2.5-1.5b", "qwen-2.5-coder-7b": "qwen-2.5-7b",
                      "qwen-2.5-math-7b": "qwen-2.5-7b", "deepseek-r1-distill-qwen-1.5b": "qwen-2.5-1.5b",
                      "deepseek-r1-distill-qwen-7b": "qwen-2.5-7b", "qwen-2.5-coder-3b": "qwen-2.5-3b",
                      "qwen-2.5-coder-14b": "qwen-2.5-14b", "deepseek-r1-distill-qwen-14b": "qwen-2.5-14b",
                      "qwen-2.5-coder-32b": "qwen-2.5-32b", "deepseek-r1-distill-qwen-32b": "qwen-2.5-32b",
                      "qwen-2.5-math-72b": "qwen-2.5-72b", "llama-3.1-405b-8bit": "llama-3.1-405b",
                      "deepseek-r1": "deepseek-v3"}.items():
  PRESETS.setdefault(_alias, PRESETS[_base])


def preset(model_id: str) -> ModelConfig:
  if model_id not in PRESETS:
    raise KeyError(f"no built-in architecture preset for {model_id!r}; provide a config.json")
  return PRESETS[model_id]
