"""Nenizen in the framework against the plain implementation in tests/nenizen_oracle.py.

Every test makes its own small configuration and random checkpoint tensors, runs them through the serving runner
(paged latent cache with one pool per layer run, batched steps; HIP kernels and HIP-graph decode on a GPU, the torch
twins on the CPU) and compares logits at every position with the oracle's float64 run over the whole sequence.
Each body runs on the CPU and, marked gpu, on cuda:0 in float32 and bfloat16.
"""
import asyncio
import json

import numpy as np
import pytest
import torch

import nenizen_oracle as oracle
from xotorch_support_jetson_amd.inference.shard import Shard
from xotorch_support_jetson_amd.models.config import TINY_NENIZEN, from_hf_config
from xotorch_support_jetson_amd.models.weights import mixed_weights, random_mixed_tensors
from xotorch_support_jetson_amd.runtime.runner import ShardRunner

RUNS = [pytest.param("cpu", torch.float32, id="cpu-f32"),
        pytest.param("cuda:0", torch.float32, id="gpu-f32", marks=pytest.mark.gpu),
        pytest.param("cuda:0", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]
TOL = {torch.float32: 2e-4, torch.bfloat16: 6e-2}


def mixer(heads=4, dim=16, rot_dim=16, vdim=16, kv_rank=32, q_rank=24, window=0, base=10000.0, dims=None, scale=0.25):
  m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
       "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
  if q_rank:
    m["q_rank"] = q_rank
  if window:
    m["mask"] = {"size": window}
  return m


def dense(ff=80, limit=2.0):
  return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff=32, experts=5, top=2, shared=48):
  m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
  if shared:
    m["shared"] = {"ff": shared}
  return m


def plain(m, mlp):  # causal, interleaved rotation, gate per element, queries projected directly
  m = dict(m)
  m.pop("q_rank", None)
  return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def windowed(m, mlp):  # sliding window, rotate-half, gate per head, query latent
  return {"type": "latent_attention_2", "mixer": m, "mlp": mlp}


def sinked(m, mlp):  # causal with a sink, rotate-half, no gate, query latent
  return {"type": "latent_attention_3", "mixer": m, "mlp": mlp}


def config(layers, width=64, vocab=96, eps=1e-5, scale=2.0, cap=12.0, loop=None):
  c = {"architecture": "Nenizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
       "logit_softcap": cap, "layers": layers}
  if loop:
    c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
  return c


SMALL = config([plain(mixer(3, 16, 16, 16, 32), dense()), windowed(mixer(4, 24, 8, 12, 48, 40, window=20), moe()),
                sinked(mixer(2, 16, 16, 24, 32, 16), None), windowed(mixer(2, 16, 16, 16, 16, 16, window=70), moe(top=1, shared=0))],
               loop=(1, 3, 2))
_ORACLE = {}


class Rig:
  """A configuration + random tensors in the runner and in the oracle."""

  def __init__(self, cfg, dev, dtype, seed=1, pages=24, slots=4, tweak=None, graphs=None):
    self.cfg, self.dev, self.dtype = cfg, torch.device(dev), dtype
    self.c = from_hf_config(cfg)
    self.tensors = random_mixed_tensors(self.c, seed)
    if tweak:
      tweak(self.tensors)
    self.key = (json.dumps(cfg, sort_keys=True), seed, getattr(tweak, "__name__", None))
    shard = Shard("t", 0, self.c.num_layers - 1, self.c.num_layers)
    w = mixed_weights(self.c, shard, self.tensors.__getitem__, self.dev, dtype)
    self.runner = ShardRunner(self.c, shard, self.dev, weights=w, num_pages=pages, max_batch=slots, max_ctx=pages * 64,
                              dtype=dtype, use_graphs=graphs)
    self.V = self.c.vocab_size

  def tokens(self, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, self.V, (n,), generator=g).tolist()

  def want(self, toks):
    k = self.key + (tuple(toks),)
    if k[2] is None or k not in _ORACLE:  # (an anonymous tweak is not a cache key)
      _ORACLE[k] = oracle.forward(self.cfg, self.tensors, toks)[0]
    return _ORACLE[k]

  def step(self, entries):
    """entries [(rid, tokens)] -> logits of every token of the step, split per entry."""
    rids = [r for r, _ in entries]
    qlens = [len(t) for _, t in entries]
    flat = [t for _, ts in entries for t in ts]
    out = self.runner.forward(rids, qlens, torch.tensor(flat, dtype=torch.int32), logit_rows=list(range(len(flat))))
    return list(out.double().cpu().split(qlens))

  def run_alone(self, rid, toks, cuts):
    """One request in portions of the given sizes (the last size repeats); logits at every position."""
    outs, lo, i = [], 0, 0
    while lo < len(toks):
      n = min(cuts[min(i, len(cuts) - 1)], len(toks) - lo)
      outs.append(self.step([(rid, toks[lo:lo + n])])[0])
      lo, i = lo + n, i + 1
    self.runner.free(rid)
    return torch.cat(outs)

  def check(self, got, toks, what=""):
    want = self.want(toks)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
    worst = int(err.argmax())
    if self.dtype == torch.bfloat16 and any(L.get("mlp") and L["mlp"]["kind"] == "moe" for L in self.cfg["layers"]):
      # two router scores closer than bf16 rounding send a token to another expert: a rare position differs by a whole
      # expert's output; all others stay inside the tolerance (the float32 runs are exact about every position)
      over = int((err >= TOL[self.dtype]).sum())
      if max(L["mlp"]["router"]["experts"] for L in self.cfg["layers"] if L.get("mlp") and L["mlp"]["kind"] == "moe") > 16:
        # dozens of experts with near-uniform scores: the chosen sets differ at many positions in bf16 (the torch twins
        # in bf16 show the same); only the typical position is checked, the float32 runs pin the mechanism
        assert err.median() < TOL[self.dtype], f"{what}: median error {float(err.median()):.3g}"
        return
      assert over <= max(2, len(toks) // 12) and err.median() < TOL[self.dtype] / 3, \
        f"{what}: {over} of {len(toks)} positions off, the worst ({worst}) by {float(err.max()):.3g}"
      return
    assert err.max() < TOL[self.dtype], f"{what}: position {worst} of {len(toks)} is off by {float(err.max()):.3g}"


def small_rig(dev, dtype, **kw):
  def small(t):
    pass
  return Rig(SMALL, dev, dtype, tweak=small, **kw)


# ------------------------------------------------------------------ whole prompts, portions, decoding
@pytest.mark.parametrize("dev,dtype", RUNS)
def test_whole_prompt(dev, dtype):
  rig = small_rig(dev, dtype)
  toks = rig.tokens(110, 3)
  rig.check(rig.run_alone("a", toks, [len(toks)]), toks, "whole prompt")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_residual_stream_after_every_layer_run(dev, dtype):
  """The stream after each layer run (looped layers once per pass), read off by running the first runs only."""
  rig = small_rig(dev, dtype)
  toks = rig.tokens(40, 4)
  trail = oracle.forward(SMALL, rig.tensors, toks)[1]
  model = rig.runner.model
  all_runs = model.runs
  assert [i for i, _ in all_runs] == [0, 1, 2, 1, 2, 3] and len(trail) == len(all_runs)
  model.shard = Shard("t", 0, 2, rig.c.num_layers)  # (not the last layer: forward returns the stream)
  try:
    for n in range(1, len(all_runs) + 1):
      model.runs = all_runs[:n]
      x = rig.runner.forward(["a"], [len(toks)], torch.tensor(toks, dtype=torch.int32)).double().cpu()
      rig.runner.free("a")
      err = (x - trail[n - 1]).abs().max(-1).values / trail[n - 1].abs().max()
      if dtype == torch.float32:
        assert err.max() < 1e-4, f"after run {n - 1}: {float(err.max()):.3g}"
      else:  # (bf16: a token now and then goes to another expert, see Rig.check)
        assert err.median() < 1e-2 and (err >= 4e-2).sum() <= 3, f"after run {n - 1}: {float(err.max()):.3g}"
  finally:
    model.runs = all_runs


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_first_tokens(dev, dtype):
  """Sequences of one, two and three tokens: empty cache, the sink beside a single key."""
  rig = small_rig(dev, dtype)
  for n in (1, 2, 3):
    toks = rig.tokens(n, 10 + n)
    rig.check(rig.run_alone("a", toks, [n]), toks, f"{n}-token prompt")
    rig.check(rig.run_alone("a", toks, [1]), toks, f"{n} tokens one by one")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_prefill_against_decoding(dev, dtype):
  rig = small_rig(dev, dtype)
  toks = rig.tokens(110, 3)
  whole = rig.run_alone("a", toks, [len(toks)])
  single = rig.run_alone("b", toks, [1])
  rig.check(single, toks, "token by token")
  diff = (whole - single).abs().max(-1).values / whole.abs().max()
  assert diff.median() < TOL[dtype] / 4 and (diff >= TOL[dtype]).sum() <= (0 if dtype == torch.float32 else 9)


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("cuts", [[2], [3, 2, 5, 1, 1, 7], [47, 1, 1, 17, 2], [64, 1], [63, 2, 1], [100, 1]])
def test_portions(dev, dtype, cuts):
  """A prompt cut anywhere (inside pages and windows, down to two tokens)."""
  rig = small_rig(dev, dtype)
  toks = rig.tokens(110, 3)
  rig.check(rig.run_alone("a", toks, cuts), toks, f"portions {cuts}")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_long_decoding(dev, dtype):
  """A short prompt, then 150 single tokens: pages and windows are crossed while decoding."""
  rig = small_rig(dev, dtype)
  toks = rig.tokens(165, 6)
  rig.check(rig.run_alone("a", toks, [15, 1]), toks, "long decoding")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16])
def test_graph_decoding_matches_eager(dtype):
  """Single-token steps replayed from a captured HIP graph (no logit rows asked: the runner's decode path) give the
  logits of the eager steps, replay after replay, with eager prompt steps of another request in between."""
  rig = Rig(config([plain(mixer(3, 16, 16, 16, 32), dense()), sinked(mixer(2, 16, 16, 24, 32, 16), moe())], loop=(0, 2, 2)),
            "cuda:0", dtype, graphs=True)
  toks = rig.tokens(60, 8)
  want = rig.run_alone("e", toks, [20, 1])
  rig.runner.forward(["g"], [20], torch.tensor(toks[:20], dtype=torch.int32))
  for i in range(20, 60):
    out = rig.runner.forward(["g"], [1], torch.tensor(toks[i:i + 1], dtype=torch.int32)).double().cpu()[0]
    assert (out - want[i]).abs().max() < 2e-2 * want[i].abs().max(), f"graph step {i}"
    if i % 7 == 0:
      rig.run_alone("other", rig.tokens(30, i), [30])
  rig.runner.free("g")


# ------------------------------------------------------------------ batches and pages
@pytest.mark.parametrize("dev,dtype", RUNS)
def test_mixed_batches_match_alone(dev, dtype):
  """Unequal requests in one step (portions beside single tokens, a request that sits a step out) give each the
  logits it gets alone."""
  rig = small_rig(dev, dtype, pages=12)
  seqs = {"a": rig.tokens(110, 3), "b": rig.tokens(70, 22), "c": rig.tokens(9, 23), "d": rig.tokens(40, 24)}
  plan = [[("a", 50), ("b", 2)], [("a", 1), ("b", 30), ("c", 9)], [("a", 1), ("d", 17)], [("a", 40), ("b", 1), ("d", 1)],
          [("b", 37), ("d", 22)], [("a", 18)]]
  at = {k: 0 for k in seqs}
  got = {k: [] for k in seqs}
  for stepplan in plan:
    entries = [(r, seqs[r][at[r]:at[r] + n]) for r, n in stepplan]
    for (r, n), o in zip(stepplan, rig.step(entries)):
      got[r].append(o)
      at[r] += n
      if at[r] == len(seqs[r]):
        rig.runner.free(r)
  for r, toks in seqs.items():
    assert at[r] == len(toks)
    rig.check(torch.cat(got[r]), toks, f"request {r} in mixed batches")


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_pages_are_reused(dev, dtype):
  """A pool of four pages serves six requests in turn, two at a time: every page is handed out again with another
  request's latents in it (in every pass's cache)."""
  rig = small_rig(dev, dtype, pages=4, slots=2)
  for rnd in range(3):
    seqs = {f"r{rnd}x": rig.tokens(100 + rnd, 30 + rnd), f"r{rnd}y": rig.tokens(90 - rnd, 40 + rnd)}
    got = {k: [] for k in seqs}
    for lo in range(0, 128, 16):
      entries = [(r, t[lo:lo + 16]) for r, t in seqs.items() if t[lo:lo + 16]]
      if not entries:
        break
      for (r, _), o in zip(entries, rig.step(entries)):
        got[r].append(o)
    for r, toks in seqs.items():
      rig.runner.free(r)
      rig.check(torch.cat(got[r]), toks, f"round {rnd} request {r}")
  assert rig.runner.bm.num_free == 4


# ------------------------------------------------------------------ other sizes
SIZES = [
  # one head everywhere, one expert of one, a window of one token, no loop, no cap, embedding scale one
  config([windowed(mixer(1, 16, 8, 8, 16, 8, window=1), moe(16, 1, 1, 0)), plain(mixer(1, 8, 8, 16, 8), dense(48, 0.5)),
          sinked(mixer(1, 8, 2, 8, 8, 8), None)], width=48, vocab=50, scale=1.0, cap=0),
  # sizes that are no multiples of 8 or 16, rotation on part of the rotated dims, a window longer than a page, every
  # expert chosen, the whole model inside the loop, latent above 128
  config([plain(mixer(5, 12, 10, 20, 136, dims=6, base=1e6), moe(24, 3, 3, 16)),
          windowed(mixer(6, 36, 6, 20, 40, 12, window=70, dims=4), dense(40, 9.0))], width=72, vocab=130, loop=(0, 2, 3)),
  # no unrotated query dims, no rotation at all, the loop at the end and of one layer, one pass
  config([sinked(mixer(2, 0, 16, 48, 24, 8), None), windowed(mixer(2, 16, 16, 16, 32, 16, window=5, dims=0), dense(32)),
          plain(mixer(4, 16, 8, 16, 16, dims=8), None)], width=32, vocab=40, loop=(2, 3, 1)),
  # more experts and more chosen than the small routing kernel takes, latent of 256 on the matrix-core path
  config([sinked(mixer(2, 8, 8, 8, 256, 8), moe(8, 70, 9, 0)), plain(mixer(8, 16, 16, 16, 64), moe(8, 3, 2, 8))],
         width=32, vocab=40, loop=(1, 2, 2)),
]


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("n", range(len(SIZES)))
def test_other_sizes(dev, dtype, n):
  rig = Rig(SIZES[n], dev, dtype, seed=50 + n)
  toks = rig.tokens(150 if n == 1 else 90, 60 + n)
  rig.check(rig.run_alone("a", toks, [33, 2, 1, 1, 29, 1]), toks, f"sizes {n}")


# ------------------------------------------------------------------ faults that random weights would hide
def _marked(kind, window):
  """One layer without rotation whose rotated key part measures how much a token's normed input points along token B's,
  whose rotated query part is minus four times that, and a token C whose embedding is minus B's: C's query scores far
  above all others with a B's key and far below with its own, and B's latent is minus C's, so whether an earlier B is
  inside C's window, or how much the sink weighs, moves C's logits."""
  dn, dr, R, qr = 16, 4, 24, 16
  m = mixer(2, dn, dr, 16, R, 0 if kind is plain else qr, window=window, dims=0, scale=1.0)
  cfg = config([kind(m, None)], width=32, vocab=24, cap=0)

  def marked(t):
    t["embed"][1] = t["embed"][1] * 2.0
    t["embed"][2] = -t["embed"][1]
    t["l0.mix.o"] = t["l0.mix.o"] * 4.0
    hb = t["embed"][1] / t["embed"][1].pow(2).mean().sqrt() * t["l0.norm1"]
    wr = (2.0 * torch.ones(dr, 1) * hb[None, :] / hb.pow(2).sum()).bfloat16().float()
    t["l0.mix.dkv"][R:] = wr
    for h in range(2):
      lo = h * (dn + dr) + dn
      if kind is plain:
        t["l0.mix.q"][lo:lo + dr] = -4.0 * wr
      else:
        t["l0.mix.uq"][lo:lo + dr] = 0.0
        t["l0.mix.uq"][lo:lo + dr, :dr] = -4.0 * torch.eye(dr)
    if kind is not plain:
      t["l0.mix.dq"][:dr] = wr
      t["l0.mix.dq.norm"] = torch.ones(qr)
    if "l0.mix.sink" in t:
      t["l0.mix.sink"] = torch.full((2,), 3.0)
  return cfg, marked


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("window", [16, 64, 65, 9])
def test_window_edges(dev, dtype, window):
  """A token B, then a token C at distance window - 2, window - 1, window, window + 1: for C the B is inside the
  window, its last token, the first outside.  In a prompt, in portions that end on and straddle the edges, and decoded
  one by one."""
  cfg, tweak = _marked(windowed, window)
  rig = Rig(cfg, dev, dtype, tweak=tweak, pages=16)
  toks, marks = [0, 0, 0], []
  for g in (window - 2, window - 1, window, window + 1, 2 * window):
    marks.append(len(toks))
    toks += [1] + [3 + (i % 5) for i in range(max(g - 1, 0))] + [2, 0, 0]
  rig.check(rig.run_alone("a", toks, [len(toks)]), toks, "prompt")
  rig.check(rig.run_alone("a", toks, [marks[1] + 1, 2, 1, window, 3, 1]), toks, "portions over the edges")
  rig.check(rig.run_alone("a", toks, [marks[0] + 2, 1]), toks, "decoding over the edges")
  # the test bites: a window one token wider or narrower changes some C's logits
  for w2 in (window + 1, window - 1):
    c2 = json.loads(json.dumps(cfg))
    c2["layers"][0]["mixer"]["mask"]["size"] = w2
    a, b = oracle.forward(c2, rig.tensors, toks)[0], rig.want(toks)
    assert (a - b).abs().max() > 0.02 * b.abs().max()


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_far_key_and_sink(dev, dtype):
  """Causal layers see a key 700 tokens back, over many pages; the sink's weight in the denominator shows in the logits
  (the oracle without it differs)."""
  cfg, tweak = _marked(sinked, 0)
  rig = Rig(cfg, dev, dtype, tweak=tweak, pages=16)
  toks = [0, 1] + [3 + (i % 7) for i in range(700)] + [2, 0]
  rig.check(rig.run_alone("a", toks, [300, 250, 1]), toks, "far key")
  for name, val in (("l0.mix.sink", torch.full((2,), -30.0)),):
    t2 = dict(rig.tensors, **{name: val})
    a = oracle.forward(cfg, t2, toks)[0]
    assert (a - rig.want(toks)).abs().max() > 0.02 * a.abs().max(), "the sink must matter for this test to bite"
  far = dict(rig.tensors)
  a = oracle.forward(cfg, far, [0, 4] + toks[2:])[0][-2]  # the same run without the far token B
  assert (a - rig.want(toks)[-2]).abs().max() > 0.02 * a.abs().max(), "the far key must matter for this test to bite"


def test_loop_needs_the_first_layer_on_its_shard():
  c = from_hf_config(SMALL)
  with pytest.raises(ValueError, match="loop"):
    ShardRunner(c, Shard("t", 1, 3, 4), "cpu", num_pages=4, max_batch=2, max_ctx=256, dtype=torch.float32)
  assert [i for i, _ in c.layer_runs([3])] == [3]


# ------------------------------------------------------------------ the engine's own entry point
@pytest.mark.parametrize("dev", ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_engine(dev):
  """Three prompts of unequal length at once through ShardedInferenceEngine (queue, batched steps, sampler at
  temperature 0): every token drawn is the oracle's greedy token for the text so far (ties within rounding
  aside), and pages are all free at the end."""
  from xotorch_support_jetson_amd.download.shard_download import NoopShardDownloader
  from xotorch_support_jetson_amd.inference.sharded_engine import ShardedInferenceEngine
  from xotorch_support_jetson_amd.models.config import preset
  c = preset("tiny-nenizen")
  tensors = random_mixed_tensors(c, 0)
  shard = Shard("tiny-nenizen", 0, c.num_layers - 1, c.num_layers)
  prompts = {"p0": [7, 3, 99, 42, 5, 17], "p1": [11] * 53, "p2": [200, 1]}
  steps = 24

  async def one(e, rid, ids):
    out, st = await e.infer_tensor(rid, shard, np.array([ids]), {"temperature": 0.0})
    seq = list(ids)
    for _ in range(steps):
      tok = int(np.asarray(await e.sample(out, temp=0.0)).reshape(-1)[0])
      seq.append(tok)
      out, st = await e.infer_tensor(rid, shard, np.array([[tok]]), dict(st, temperature=0.0))
    await e.finish_request(rid)
    return seq

  async def main():
    e = ShardedInferenceEngine(NoopShardDownloader(), device=torch.device(dev))
    seqs = await asyncio.gather(*[one(e, r, p) for r, p in prompts.items()])
    return e, seqs
  e, seqs = asyncio.run(main())
  assert e.runner.bm.num_free == e.runner.bm.num_blocks
  for (rid, p), seq in zip(prompts.items(), seqs):
    lg = oracle.forward(TINY_NENIZEN, tensors, seq[:-1])[0]
    for t in range(len(p) - 1, len(seq) - 1):
      best = float(lg[t].max())
      assert float(lg[t][seq[t + 1]]) >= best - 0.05 * float(lg[t].std()), f"{rid}: token {t + 1} is not the greedy one"


def test_checkpoint_directory_through_registry_and_engine(tmp_path):
  """config.json + model.safetensors (bf16) in a folder: registered as a local model, loaded by the engine's own
  build path, and the prompt's last-token logits match the oracle run on the same tensors."""
  from safetensors.torch import save_file
  from xotorch_support_jetson_amd.download.shard_download import NoopShardDownloader
  from xotorch_support_jetson_amd.inference.sharded_engine import ShardedInferenceEngine
  from xotorch_support_jetson_amd.models import registry
  cfg = SIZES[1]
  c = from_hf_config(cfg)
  tensors = random_mixed_tensors(c, 5)
  (tmp_path / "config.json").write_text(json.dumps(cfg))
  save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()}, str(tmp_path / "model.safetensors"))
  mid = registry.register_local_model(str(tmp_path))
  assert mid is not None and registry.model_cards[mid]["layers"] == len(cfg["layers"])
  shard = registry.build_full_shard(mid, "ShardedInferenceEngine")
  toks = [3, 99, 7, 7, 120, 64, 1, 0, 55]

  async def main():
    e = ShardedInferenceEngine(NoopShardDownloader(), device=torch.device("cpu"))
    out, _ = await e.infer_tensor("r", shard, np.array([toks]), {})
    return e, out
  e, out = asyncio.run(main())
  assert e.config.model_type == "nenizen" and e.config.layer_specs[1].lattn.window == 70 and e.config.loop == (0, 2, 3)
  want = oracle.forward(cfg, tensors, toks)[0][-1]
  got = out.double().reshape(-1)
  assert (got - want).abs().max() < 0.03 * want.abs().max()  # bf16 activations on the serving path
