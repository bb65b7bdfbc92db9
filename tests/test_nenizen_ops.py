"""Each mechanism of the sandwich-block / latent-attention ops against its function in tests/nenizen_oracle.py.

The ops run as the framework calls them (HIP kernels on a GPU, torch twins on the CPU), on their own inputs: scrambled
pages, several sequences per step, steps that continue earlier ones.  Bodies run on the CPU and, marked gpu, on cuda:0
in float32 and bfloat16.
"""
import pytest
import torch

import nenizen_oracle as oracle
from xotorch_support_jetson_amd.ops import kernels as K
from xotorch_support_jetson_amd.ops.rope import build_cos_sin

RUNS = [pytest.param("cpu", torch.float32, id="cpu-f32"),
        pytest.param("cuda:0", torch.float32, id="gpu-f32", marks=pytest.mark.gpu),
        pytest.param("cuda:0", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]
PAGE = 64


def tol(dtype):
  return 2e-5 if dtype == torch.float32 else 2e-2


def close(got, want, dtype, what=""):
  if want.numel() == 0:
    assert got.numel() == 0
    return
  err = (got.double().cpu() - want.double()).abs().max() / max(float(want.abs().max()), 1e-9)
  assert err < tol(dtype), f"{what}: off by {float(err):.3g}"


def rnd(*shape, seed=0, scale=1.0):
  return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def r16(t, dtype):
  """Values as the op's storage dtype holds them, so the oracle sees the same numbers."""
  return t.to(dtype).float()


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_sandwich_add_norm(dev, dtype):
  T, D, eps = 9, 72, 1e-5
  x, y, wb, wn = rnd(T, D, seed=1), rnd(T, D + 24, seed=2, scale=3.0), rnd(D, seed=3), rnd(D, seed=4)
  xs = x.clone().to(dev)
  out = torch.zeros(T, 128, dtype=dtype, device=dev)
  K.sandwich_add_norm(xs, y.to(dev), wb.to(dev), wn.to(dev), eps, out)
  want_x = x.double() + oracle.rms_norm(y[:, :D].double(), wb.double(), eps)
  close(xs, want_x, torch.float32, "stream")
  close(out[:, :D], oracle.rms_norm(want_x, wn.double(), eps), dtype, "next input")
  assert float(out[:, D:].abs().max()) == 0.0  # the operand's padding columns stay zero
  # only the norm (no sublayer result), only the add (no next norm)
  out2 = torch.zeros(T, D, dtype=dtype, device=dev)
  K.sandwich_add_norm(xs, None, None, wn.to(dev), eps, out2)
  close(out2, oracle.rms_norm(want_x, wn.double(), eps), dtype, "norm alone")
  K.sandwich_add_norm(xs, y.to(dev), wb.to(dev), None, eps, None)
  close(xs, want_x + oracle.rms_norm(y[:, :D].double(), wb.double(), eps), torch.float32, "add alone")


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("inter", [True, False])
@pytest.mark.parametrize("H,dn,dr,rot", [(3, 10, 16, 12), (1, 0, 8, 8), (4, 16, 6, 0), (2, 24, 32, 32)])
def test_query_rotation(dev, dtype, inter, H, dn, dr, rot):
  T, base, off = 11, 5000.0, 5
  Q = rnd(T, off + H * (dn + dr) + 3, seed=5)
  pos = torch.tensor([0, 1, 2, 63, 64, 65, 300, 7, 7, 511, 128], dtype=torch.int32)
  tab = build_cos_sin(rot, 512, base, None, dev) if rot else torch.zeros(1, 0, device=dev)
  qn = torch.zeros(H, T, dn, dtype=dtype, device=dev)
  qpe = torch.zeros(T, H, dr, dtype=dtype, device=dev)
  K.latent_q_rope(Q.to(dev), off, H, dn, dr, rot, inter, pos.to(dev), tab, qn, qpe)
  q = Q[:, off:off + H * (dn + dr)].double().reshape(T, H, dn + dr)
  close(qn, q[..., :dn].transpose(0, 1), dtype, "unrotated parts")
  close(qpe, oracle.rotate(q[..., dn:], pos, rot, base, inter), dtype, "rotated parts")


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("inter", [True, False])
def test_latent_store(dev, dtype, inter):
  """Latent norm, rotation of the shared key part and the paged write at scattered slots (one token without a slot);
  the query latent's norm."""
  T, R, dr, qr, rot, eps, base = 13, 40, 12, 20, 8, 1e-5, 10000.0
  P = rnd(T, 100, seed=6)
  kvn, qn = rnd(R, seed=7), rnd(qr, seed=8)
  pos = torch.arange(T, dtype=torch.int32) * 37 % 400
  slots = torch.randperm(4 * PAGE, generator=torch.Generator().manual_seed(9))[:T].long()
  slots[4] = -1
  cache = torch.full((4, 1, PAGE, R + dr), 7.0, dtype=dtype, device=dev)
  qa = torch.zeros(T, 64, dtype=dtype, device=dev)
  tab = build_cos_sin(rot, 512, base, None, dev)
  K.latent_kv_store(P.to(dev), 30, R, dr, kvn.to(dev), 3, qr, qn.to(dev), eps, rot, inter, pos.to(dev), tab,
                    slots.to(dev), cache, qa)
  c = oracle.rms_norm(P[:, 30:30 + R].double(), kvn.double(), eps)
  kr = oracle.rotate(P[:, 30 + R:30 + R + dr].double().reshape(T, 1, dr), pos, rot, base, inter).reshape(T, dr)
  flat = cache.reshape(4 * PAGE, R + dr)
  keep = slots >= 0
  close(flat[slots[keep].to(dev)], torch.cat([c, kr], 1)[keep], dtype, "cache rows")
  untouched = torch.ones(4 * PAGE, dtype=torch.bool)
  untouched[slots[keep]] = False
  assert bool((flat.cpu()[untouched] == 7.0).all())
  close(qa[:, :qr], oracle.rms_norm(P[:, 3:3 + qr].double(), qn.double(), eps), dtype, "query latent")
  # no query latent: nothing but the cache is written
  K.latent_kv_store(P.to(dev), 30, R, dr, kvn.to(dev), 0, 0, None, eps, rot, inter, pos.to(dev), tab, slots.to(dev),
                    cache, None)


def _attention_case(dev, dtype, H, R, dr, window, sink, seqs, steps, scale=0.3, seed=0):
  """seqs: lengths; steps: per step [(sequence, new tokens)].  Keys are written to scrambled pages step by step as the
  runner would; every step's outputs are compared with the oracle's softmax over the visible keys."""
  n_pages = sum(-(-n // PAGE) for n in seqs) + 2
  order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
  tables, at = [], 0
  for n in seqs:
    tables.append(order[at:at + -(-n // PAGE)])
    at += -(-n // PAGE)
  width = max(len(t) for t in tables)
  rows = [r16(rnd(n, R + dr, seed=seed + 10 + i, scale=0.7), dtype) for i, n in enumerate(seqs)]
  cache = torch.full((n_pages, 1, PAGE, R + dr), 3.0, dtype=dtype)  # (stale values where nothing was written yet)
  sk = rnd(H, seed=seed + 5) if sink else None
  done = [0] * len(seqs)
  for step in steps:
    bt = torch.zeros(len(step), width, dtype=torch.int32)
    cu, ctx, ql, qp = [0], [], [], []
    for b, (i, n) in enumerate(step):
      for p in range(done[i], done[i] + n):
        cache[tables[i][p // PAGE], 0, p % PAGE] = rows[i][p].to(dtype)
      bt[b, :len(tables[i])] = torch.tensor(tables[i], dtype=torch.int32)
      cu.append(cu[-1] + n)
      ctx.append(done[i] + n)
      ql.append(r16(rnd(H, n, R, seed=seed + 100 * i + done[i], scale=0.5), dtype))
      qp.append(r16(rnd(n, H, dr, seed=seed + 100 * i + done[i] + 50, scale=0.5), dtype))
    q_lat, q_pe = torch.cat(ql, 1), torch.cat(qp, 0)
    out = torch.zeros(H, cu[-1], R, dtype=dtype, device=dev)
    K.latent_attn(q_lat.to(dtype).to(dev), q_pe.to(dtype).to(dev), cache.to(dev), bt.to(dev),
                  torch.tensor(cu, dtype=torch.int32, device=dev), torch.tensor(ctx, dtype=torch.int32, device=dev),
                  None if sk is None else sk.to(dev), scale, window, out, max_qlen=max(n for _, n in step))
    for b, (i, n) in enumerate(step):
      N = done[i] + n
      keys = rows[i][:N].double()
      s = (torch.einsum("hqr,jr->hqj", ql[b].double(), keys[:, :R]) +
           torch.einsum("qhr,jr->hqj", qp[b].double(), keys[:, R:])) * scale
      full = torch.full((H, N, N), float("-inf"), dtype=torch.float64)
      full[:, done[i]:] = s
      w = oracle.softmax_with_sink(full, oracle.visible(N, window), sk)[:, done[i]:]
      close(out[:, cu[b]:cu[b + 1]], torch.einsum("hqj,jr->hqr", w, keys[:, :R]), dtype,
            f"step {step} sequence {i}")
      done[i] += n


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("H,R,dr,window,sink", [(6, 32, 16, 0, False), (4, 48, 8, 20, True), (1, 40, 6, 64, True),
                                                (5, 136, 10, 65, False), (2, 64, 32, 1, True), (9, 16, 0, 7, False)])
def test_latent_attention_small_steps(dev, dtype, H, R, dr, window, sink):
  """Single tokens and short portions of three sequences, together and in turn (the vector-unit kernel)."""
  _attention_case(dev, dtype, H, R, dr, window, sink, [70, 131, 9],
                  [[(0, 3), (1, 1)], [(0, 1), (1, 2), (2, 9)], [(1, 1)], [(0, 9), (1, 12)], [(0, 1), (1, 1)], [(1, 15), (0, 1)],
                   [(0, 15), (1, 15)], [(0, 15), (1, 15)], [(0, 15), (1, 15)], [(0, 10), (1, 15)], [(1, 15)], [(1, 15)],
                   [(1, 8)], [(1, 1)]])


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("H,R,dr,window,sink", [(4, 128, 32, 0, True), (3, 48, 8, 72, False), (2, 256, 64, 100, True),
                                                (5, 64, 16, 64, False), (2, 32, 24, 17, True)])
def test_latent_attention_prompt_portions(dev, dtype, H, R, dr, window, sink):
  """Portions of 16 tokens and more beside single tokens (bf16 on a GPU: the matrix-core kernel), cut inside pages and
  windows; a sequence that starts in a later step."""
  _attention_case(dev, dtype, H, R, dr, window, sink, [300, 150, 40],
                  [[(0, 100)], [(0, 64), (1, 17)], [(0, 1), (1, 100), (2, 40)], [(0, 120), (1, 33)], [(0, 15)]], seed=3)


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("window", [0, 5, 64, 200])
def test_one_key_stands_out(dev, dtype, window):
  """A key far back whose latent is the query's direction: the output is that key's latent while it is visible, and
  something else one token later (every head, prompt portion and single token)."""
  H, R, dr, N = 2, 32, 8, 260
  for qlen in (1, 20):
    for dist in ([window - 1, window] if window else [N - 1]):
      rows = r16(rnd(N, R + dr, seed=4, scale=0.1), dtype)
      star = N - 1 - dist
      if star < 0:
        continue
      rows[star, :R] = r16(rnd(R, seed=5), dtype)
      cache = torch.zeros(5, 1, PAGE, R + dr, dtype=dtype)
      cache.view(5 * PAGE, R + dr)[:N] = rows.to(dtype)
      q_lat = (rows[star, :R] * 3.0).expand(H, qlen, R).contiguous()
      out = torch.zeros(H, qlen, R, dtype=dtype, device=dev)
      K.latent_attn(q_lat.to(dtype).to(dev), torch.zeros(qlen, H, dr, dtype=dtype, device=dev), cache.to(dev),
                    torch.arange(5, dtype=torch.int32, device=dev)[None], torch.tensor([0, qlen], dtype=torch.int32, device=dev),
                    torch.tensor([N], dtype=torch.int32, device=dev), None, 1.0, window, out, max_qlen=qlen)
      last = out[:, -1].double().cpu()
      seen = (last - rows[star, :R].double()).abs().max() < 0.05 * rows[star, :R].abs().max()
      assert bool(seen) == (window == 0 or dist < window), f"window {window}, key {dist} back, {qlen} queries"


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("gate", [0, 1, 2])
def test_output_gate(dev, dtype, gate):
  H, T, dv = 3, 7, 20
  o = r16(rnd(H, T, dv, seed=6), dtype)
  P = rnd(T, 90, seed=7)
  out = torch.zeros(T, 128, dtype=dtype, device=dev)
  K.latent_out_gate(o.to(dtype).to(dev), P.to(dev) if gate else None, 11, gate, out)
  want = o.double().transpose(0, 1)
  if gate == 1:
    want = want * torch.sigmoid(P[:, 11:11 + H * dv].double()).reshape(T, H, dv)
  if gate == 2:
    want = want * torch.sigmoid(P[:, 11:11 + H].double()).reshape(T, H, 1)
  close(out[:, :H * dv], want.reshape(T, H * dv), dtype)


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_gated_activations(dev, dtype):
  """The clamped form and the SiLU form against the oracle's feed-forwards with an identity down projection."""
  T, Fd = 6, 24
  P = rnd(T, 70, seed=8, scale=3.0)
  eye = torch.eye(Fd)
  sel = lambda off: torch.eye(70)[off:off + Fd]  # picks Fd columns of P as a "projection"
  tensors = {"m.gate": sel(5), "m.up": sel(40), "m.down": eye}
  for clamped, want in ((True, oracle.dense_ff(P.double(), {"limit": 1.25}, tensors, "m.")),
                        (False, oracle.silu_expert(P.double(), tensors, "m."))):
    out = torch.zeros(T, 32, dtype=dtype, device=dev)
    K.glu_act(P.to(dev), 5, 40, Fd, clamped, 1.25, out)
    close(out[:, :Fd], want, dtype, f"clamped {clamped}")


@pytest.mark.parametrize("dev", ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)])
def test_weighted_sum_with_ungated_shared_expert(dev):
  T, k, D = 5, 3, 40
  y, sh = rnd(T * k, D + 8, seed=9), rnd(T, D, seed=10)
  topw = torch.rand(T * k, generator=torch.Generator().manual_seed(11))
  slot_of = torch.randperm(T * k, generator=torch.Generator().manual_seed(12)).int()
  out = torch.zeros(T, D, device=dev)
  K.moe_weighted_sum(y.to(dev), slot_of.to(dev), topw.to(dev), k, sh.to(dev), None, 0, out)
  want = (y[slot_of.long(), :D].reshape(T, k, D).double() * topw.reshape(T, k, 1).double()).sum(1) + sh.double()
  close(out, want, torch.float32)
