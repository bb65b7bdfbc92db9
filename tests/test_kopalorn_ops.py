"""The ops behind Kopalorn's layers, one mechanism at a time, against the functions of tests/kopalorn_oracle.py: the torch
twins on the CPU and, marked gpu, the HIP kernels in float32 and bfloat16 (the activations' dtype; states, norms, gates
and scores are float32 in both)."""
import math

import pytest
import torch

import kopalorn_oracle as oracle
from xotorch_support_jetson_amd.ops import kernels as K

RUNS = [pytest.param("cpu", torch.float32, id="cpu-f32"),
        pytest.param("cuda:0", torch.float32, id="gpu-f32", marks=pytest.mark.gpu),
        pytest.param("cuda:0", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
  return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(got, want, tol, what=""):
  err = (got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-9)
  assert err < tol, f"{what}: off by {float(err):.3g}"


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("D", [48, 200, 1100, 3000, 4200])
def test_layer_norm_add_and_next_norm(dev, dtype, D):
  """x += mult * layer_norm(y) and the next sublayer's input layer_norm(x), biases and all; y rows wider than D."""
  T, eps, mult = 5, 1e-5, 0.3
  x, y = rnd(T, D, seed=1) + 0.7, rnd(T, D + 24, seed=2) * 3 - 1.0
  wb, bb, wn, bn = rnd(D, seed=3), rnd(D, seed=4), rnd(D, seed=5), rnd(D, seed=6)
  x2 = x.double() + mult * oracle.layer_norm(y[:, :D].double(), wb.double(), bb.double(), eps)
  want = oracle.layer_norm(x2, wn.double(), bn.double(), eps)
  x0 = x.clone()
  xd, out = x.clone().to(dev), torch.zeros(T, D + 8, dtype=dtype, device=dev)
  K.sandwich_add_norm(xd, y.to(dev), wb.to(dev), wn.to(dev), eps, out, bb=bb.to(dev), bn=bn.to(dev), mult=mult)
  close(xd, x2, 1e-5, "stream")
  close(out[:, :D], want, 1e-5 if dtype == torch.float32 else 1e-2, "normed")
  assert float(out[:, D:].abs().max()) == 0.0
  # without biases the same op is the RMS norm with a weight
  xd = x0.clone().to(dev)
  K.sandwich_add_norm(xd, y.to(dev), wb.to(dev), None, eps, None)
  close(xd, x0.double() + oracle.rms(y[:, :D].double(), eps) * wb.double(), 1e-5, "rms")


@pytest.mark.parametrize("dev", ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("E,top,groups,keep", [(10, 2, 2, 1), (6, 3, 3, 2), (4, 2, 4, 3), (48, 9, 8, 3), (5, 5, 1, 1), (1, 1, 1, 1)])
def test_grouped_sigmoid_routing(dev, E, top, groups, keep):
  """Choice on the corrected scores inside the best groups (corrections push choice scores below zero: a masked expert
  must count as minus infinity, not zero), weights from the uncorrected scores, groups of one expert."""
  T, scale = 40, 1.75
  z, corr = rnd(T, E, seed=E), rnd(E, seed=top) * 0.5 - 1.0
  r = {"experts": E, "top": top, "scale": scale, "groups": {"count": groups, "keep": keep}}
  out = K.moe_route_ds(z.to(dev), corr.to(dev), top, groups, keep, 2, True, True, scale)
  topw, topi = out[0].reshape(T, top).cpu(), out[1].reshape(T, top).cpu()
  for t in range(T):
    idx, w = oracle.route(z[t].double(), corr.double(), r)
    got = dict(zip(topi[t].tolist(), topw[t].tolist()))
    assert sorted(got) == sorted(idx), f"token {t}: experts {sorted(got)} for {sorted(idx)}"
    for e, we in zip(idx, w):
      assert abs(got[e] - we) < 1e-5 * scale


def _paged(seqs, slots_of, k_rows, v_rows, G, Gv, d, dv, dev, dtype, pages):
  """Caches [pages, G, 64, d] / [pages, Gv, dv, 64] filled with the given rows at the given pages."""
  kc = torch.zeros(pages, G, 64, d, dtype=dtype, device=dev)
  vc = torch.zeros(pages, Gv, dv, 64, dtype=dtype, device=dev)
  for b, table in enumerate(slots_of):
    for p in range(k_rows[b].shape[0]):
      kc[table[p // 64], :, p % 64] = k_rows[b][p].to(dtype)
      vc[table[p // 64], :, :, p % 64] = v_rows[b][p].to(dtype)
  return kc, vc


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("H,G,Gv,d,dv,window", [(8, 4, 2, 16, 24, 11), (4, 2, 1, 32, 64, 70), (2, 2, 2, 48, 48, 0), (16, 2, 1, 8, 8, 64),
                                                  (4, 2, 1, 64, 128, 100), (4, 4, 2, 128, 128, 0), (6, 2, 2, 64, 64, 33)])
def test_window_attention_with_shared_values(dev, dtype, H, G, Gv, d, dv, window):
  """Key head g reads value head g / (G / Gv); fp32 output beside caches of the activations' dtype; two sequences on
  scrambled pages, a portion of 19 tokens and a single token."""
  n = [150, 131]
  new = [19, 1]
  tables = [[5, 2, 7], [0, 6, 3]]
  ks = [rnd(n[b], G, d, seed=10 + b).to(dtype).float() for b in range(2)]
  vs = [rnd(n[b], Gv, dv, seed=20 + b).to(dtype).float() for b in range(2)]
  kc, vc = _paged(n, tables, ks, vs, G, Gv, d, dv, dev, dtype, 8)
  q = torch.cat([rnd(new[b], H, d, seed=30 + b) for b in range(2)]).to(dtype)
  out = torch.empty(sum(new), H * dv, dtype=torch.float32, device=dev)
  bt = torch.tensor(tables, dtype=torch.int32, device=dev)
  cu = torch.tensor([0, new[0], sum(new)], dtype=torch.int32, device=dev)
  ctx = torch.tensor(n, dtype=torch.int32, device=dev)
  scale = 0.3
  K.attn_window_pool(q.to(dev), kc, vc, None, None, bt, cu, ctx, None, scale, window, 0, out, max_qlen=max(new))
  row = 0
  for b in range(2):
    qf = torch.zeros(n[b], H, d, dtype=F64)
    qf[n[b] - new[b]:] = q[row:row + new[b]].double()
    vfull = vs[b].double().repeat_interleave(G // Gv, 1)
    want = oracle.softmax_attention(qf, ks[b].double(), vfull, scale, window)[n[b] - new[b]:].reshape(new[b], H * dv)
    close(out[row:row + new[b]], want, 1e-5 if dtype == torch.float32 else 2e-2, f"sequence {b}")
    row += new[b]


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_differential_combination(dev, dtype):
  """a_1 - lam a_2 per head, the per-head RMS division, the post factor and the per-head gate, with the maps' heads ordered
  (kv head, map, head of the group)."""
  T, H, G, dv, lam, post, eps = 7, 6, 2, 20, 0.37, 0.6, 1e-5
  rep = H // G
  a = rnd(T, G, 2, rep, dv, seed=1)
  P = rnd(T, 40, seed=2)
  o = a[:, :, 0].double() - lam * a[:, :, 1].double()  # [T, G, rep, dv] -> head g rep + r
  want = oracle.rms(o.reshape(T, H, dv), eps) * post * torch.sigmoid(P[:, 5:5 + H].double())[:, :, None]
  out = torch.zeros(T, H * dv + 8, dtype=dtype, device=dev)
  K.diff_attn_out(a.reshape(T, -1).to(dev), P.to(dev), 5, H, G, lam, post, eps, out)
  close(out[:, :H * dv], want.reshape(T, -1), 1e-5 if dtype == torch.float32 else 1e-2)


def _state_case(H, dv_state, d, dev):
  """Two sequences in two steps (7 + 1 tokens, then 70 + 3), slots 2 and 0 of three; the unused slot holds another
  request's leftovers."""
  S = torch.zeros(3, H, dv_state, d, device=dev)
  S[1] = 7.0
  steps = [([0, 7, 8], [7, 1]), ([0, 70, 73], [70, 3])]
  return S, torch.tensor([2, 0], dtype=torch.int32, device=dev), steps


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("H,d,dv,cap", [(2, 16, 16, 15.0), (3, 24, 40, 2.0), (1, 72, 9, 50.0), (2, 16, 200, 15.0)])
def test_mlstm_gates_recurrence_and_norm(dev, dtype, H, d, dv, cap):
  """Gates with their cap, the running maximum from zero, decay and input scale, the recurrence with the normaliser as the
  state's last value channel, the stabilised division, the per-head norm, weight and sigmoid gate; states carried over
  two steps."""
  D, eps = 32, 1e-5
  lens = [77, 4]
  hs = [rnd(n, D, seed=40 + b) for b, n in enumerate(lens)]
  t = {"q": rnd(H * d, D, seed=1, scale=0.3), "k": rnd(H * d, D, seed=2, scale=0.3), "v": rnd(H * dv, D, seed=3, scale=0.3),
       "g": rnd(H * dv, D, seed=4, scale=0.3), "i": rnd(H, D, seed=5), "i.b": rnd(H, seed=6), "f": rnd(H, D, seed=7),
       "f.b": rnd(H, seed=8) + 2.0, "norm": 1.0 + 0.1 * rnd(H * dv, seed=9), "o": torch.eye(H * dv)}
  m = {"heads": H, "dim": d, "vdim": dv, "gate_cap": cap}
  want = [oracle.mlstm(h.double(), m, {k: v.double() for k, v in t.items()}, "", eps) for h in hs]
  W = torch.cat([t["q"], t["k"], t["v"], t["g"], t["i"], t["f"]]).t()
  qo, ko, vo, go, io, fo = 0, H * d, 2 * H * d, 2 * H * d + H * dv, 2 * H * d + 2 * H * dv, 2 * H * d + 2 * H * dv + H
  S, slots, steps = _state_case(H, dv + 1, d, dev)
  mstate = torch.full((3, H), 3.0, device=dev)
  mstate[slots.long()] = 0.0
  gate_b = torch.cat([t["i.b"], t["f.b"]]).to(dev)
  at, got = [0, 0], [[], []]
  for cu, ns in steps:
    P = torch.cat([hs[b][at[b]:at[b] + ns[b]] for b in range(2)]) @ W
    P = P.to(dev)
    T = P.shape[0]
    decay, inscale, mo = (torch.empty(T, H, device=dev) for _ in range(3))
    cuq = torch.tensor(cu, dtype=torch.int32, device=dev)
    K.mlstm_gates(P, io, fo, gate_b, cap, mstate, slots, cuq, decay, inscale, mo)
    o = torch.empty(T, H * (dv + 1), device=dev)
    K.linear_recurrence(P[:, qo:qo + H * d], P[:, ko:ko + H * d], P[:, vo:vo + H * dv], decay, inscale, d ** -0.5, S, slots, cuq, o)
    out = torch.zeros(T, H * dv, dtype=dtype, device=dev)
    K.gated_group_norm(o, mo, t["norm"].to(dev), P, go, H, eps, out)
    for b in range(2):
      got[b].append(out[cu[b]:cu[b + 1]])
      at[b] += ns[b]
  for b in range(2):
    close(torch.cat(got[b]), want[b], 2e-4 if dtype == torch.float32 else 2e-2, f"sequence {b}")
  assert float(S[1].min()) == 7.0 and float(mstate[1].min()) == 3.0  # the slot of no request stays as it was


@pytest.mark.parametrize("dev,dtype", RUNS)
@pytest.mark.parametrize("H,d,dv", [(2, 16, 16), (3, 40, 24)])
def test_lightning_recurrence_and_norm(dev, dtype, H, d, dv):
  """SiLU on q, k, v, one fixed decay per head, the norm over all heads together, weight and sigmoid gate."""
  D, eps = 32, 1e-5
  lens = [77, 4]
  decays = [0.5, 0.97, 0.999][:H]
  hs = [rnd(n, D, seed=50 + b) for b, n in enumerate(lens)]
  t = {"q": rnd(H * d, D, seed=1, scale=0.3), "k": rnd(H * d, D, seed=2, scale=0.3), "v": rnd(H * dv, D, seed=3, scale=0.3),
       "g": rnd(H * dv, D, seed=4, scale=0.3), "norm": 1.0 + 0.1 * rnd(H * dv, seed=9), "o": torch.eye(H * dv)}
  m = {"heads": H, "dim": d, "vdim": dv, "decay": decays}
  want = [oracle.lightning(h.double(), m, {k: v.double() for k, v in t.items()}, "", eps) for h in hs]
  W = torch.cat([t["q"], t["k"], t["v"], t["g"]]).t()
  nq, nv = H * d, H * dv
  S, slots, steps = _state_case(H, dv, d, dev)
  dec = torch.tensor(decays, device=dev)
  at, got = [0, 0], [[], []]
  for cu, ns in steps:
    P = (torch.cat([hs[b][at[b]:at[b] + ns[b]] for b in range(2)]) @ W).to(dev)
    T = P.shape[0]
    cuq = torch.tensor(cu, dtype=torch.int32, device=dev)
    qkv = torch.empty(T, 2 * nq + nv, device=dev)
    K.silu_cols(P, 0, 2 * nq + nv, qkv)
    o = torch.empty(T, nv, device=dev)
    K.linear_recurrence(qkv[:, :nq], qkv[:, nq:2 * nq], qkv[:, 2 * nq:], dec, None, 1.0, S, slots, cuq, o)
    out = torch.zeros(T, nv, dtype=dtype, device=dev)
    K.gated_group_norm(o, None, t["norm"].to(dev), P, 2 * nq + nv, 1, eps, out)
    for b in range(2):
      got[b].append(out[cu[b]:cu[b + 1]])
      at[b] += ns[b]
  for b in range(2):
    close(torch.cat(got[b]), want[b], 2e-4 if dtype == torch.float32 else 2e-2, f"sequence {b}")
  assert float(S[1].min()) == 7.0


@pytest.mark.parametrize("dev,dtype", RUNS)
def test_gate_and_pair_mean(dev, dtype):
  T, n, D, eps = 6, 40, 72, 1e-5
  a, P = rnd(T, n, seed=1), rnd(T, 64, seed=2)
  out = torch.zeros(T, n + 8, dtype=dtype, device=dev)
  K.sigmoid_gate_mul(a.to(dev), P.to(dev), 3, out)
  close(out[:, :n], a.double() * torch.sigmoid(P[:, 3:3 + n].double()), 1e-5 if dtype == torch.float32 else 1e-2, "gate")
  y1, y2, w = rnd(T, D + 56, seed=3) * 4, rnd(T, D, seed=4) * 0.1, rnd(2, D, seed=5)
  mean = torch.empty(T, D, device=dev)
  K.pair_norm_mean(y1.to(dev), y2.to(dev), w.to(dev), eps, mean)
  want = 0.5 * (oracle.rms(y1[:, :D].double(), eps) * w[0].double() + oracle.rms(y2.double(), eps) * w[1].double())
  close(mean, want, 1e-5, "pair mean")


def test_rotation_pairs_become_halves():
  """The loader's row order turns pairs (2i, 2i + 1) into (i, i + R / 2): rotating the reordered head with the kernels'
  layout equals reordering the head rotated with the design's."""
  from xotorch_support_jetson_amd.models.weights import _pair_order
  d, R, n, base = 12, 8, 9, 100.0
  x = rnd(n, 1, d, seed=1).double()
  want = oracle.rope_interleaved(x, base, R)
  order = _pair_order(d, R)
  y = x[..., order]
  half = R // 2
  ang = torch.arange(n, dtype=F64)[:, None] * base ** (-2.0 * torch.arange(half, dtype=F64) / R)[None, :]
  c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
  rot = torch.cat([y[..., :half] * c - y[..., half:R] * s, y[..., half:R] * c + y[..., :half] * s, y[..., R:]], -1)
  assert (rot - want[..., order]).abs().max() < 1e-12 and math.isclose(float(rot.pow(2).sum()), float(x.pow(2).sum()))
