// Post-norm hybrid blocks on an fp32 residual stream (gfx950): window attention with pooled blocks and a sink, the
// Mamba-2 (SSD) mixer's element-wise stages, non-gated feed-forward activations and the routed experts' sum.
//
//   gated_postnorm      x <- rms_norm(alpha x + y * sigmoid(gate + b)) * w, and its copy in the GEMM operand dtype
//   qk_norm_rope_store  q / k / v biases, partial rotate-half RoPE, per-head RMS division, paged write of k and v
//   kv_pool_update      mean key / value of every block of `pool` tokens that the step completed -> pooled caches
//   attn_window_pool    softmax attention over [window tokens | pooled blocks before the window | sink]: a workgroup per
//                       (token, head) for any sizes and fp32; an MFMA kernel for bf16 prompt portions
//   ssd_prep            causal convolution + bias + SiLU over x | B | C, dt = softplus(dt + bias), decay, v = dt x
//   ssd_gate_norm       (o + D x) * silu(z), RMS norm in equal groups, weight
//   polynorm_act        a N(z) + b N(z^2) + c N(z^3) + e with N = division by the row's RMS
//   relu2               relu(z)^2
//   moe_weighted_sum    sum_j w_j y[slot_j] + sigmoid(gate) * shared (or + shared, ungated)
//
// P is a fused projection's fp32 output [T, ldp]; "column offset" arguments address its slices.  Activations that
// feed the next GEMM (AT) are bf16 or fp32; norms, scores, softmax weights, gates and everything a recurrence reads
// are fp32.
#include "mixer_util.h"

namespace xot {
namespace {
using namespace mix;

// ------------------------------------------------------------------ gated residual + RMS norm with a weight
template <typename AT>
__global__ void gated_postnorm_k(float* __restrict__ x, const float* __restrict__ y, int ldy, const float* __restrict__ P,
                                 int ldp, int g_off, const float* __restrict__ gb, float alpha, const float* __restrict__ w,
                                 float eps, AT* __restrict__ out, int ldo, int D) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  float* xr = x + r * D;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    float v = alpha * xr[i];
    if (y) {
      float a = y[r * ldy + i];
      if (P) a *= sigmoidf_(P[r * ldp + g_off + i] + gb[i]);
      v += a;
    }
    xr[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float k = 1.0f / sqrtf(ss / (float)D + eps);
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    const float v = xr[i] * k * w[i];
    xr[i] = v;
    if (out) stf(out + r * ldo + i, v);
  }
}

// ------------------------------------------------------------------ biases + RoPE + per-head RMS division + paged write
// cos_sin [rows, R]: row p = [cos(p f_0 .. f_{R/2-1}) | sin(...)].  Pair (i, i + R/2), i < R/2; dims >= R pass.
// A wave per q / k head (d <= 256: four dims a lane); the values are written by all threads afterwards.
template <typename AT>
__global__ __launch_bounds__(256) void qk_norm_rope_store_k(
    const float* __restrict__ P, int ldp, const float* __restrict__ bias, int q_off, int k_off, int v_off, int H, int G,
    int d, int dv, int R, const int* __restrict__ pos, const float* __restrict__ cos_sin, const int64_t* __restrict__ slots,
    float eps, int qk_norm, AT* __restrict__ q_out, AT* __restrict__ k_cache, AT* __restrict__ v_cache, int Gv) {
  const int t = blockIdx.x;
  const float* row = P + (int64_t)t * ldp;
  const float* cs = cos_sin + (int64_t)pos[t] * R;
  const int half = R >> 1;
  const int64_t slot = slots[t];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int heads = H + (k_off >= 0 ? G : 0);
  for (int head = wave; head < heads; head += nw) {
    const bool isq = head < H;
    const int c0 = isq ? q_off + head * d : k_off + (head - H) * d;
    auto at = [&](int i) { return row[c0 + i] + (bias ? bias[c0 + i] : 0.0f); };
    float v[4];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int i = lane + 64 * c;
      v[c] = 0.0f;
      if (i >= d) continue;
      float a = at(i);
      if (i < half) {
        a = a * cs[i] - at(i + half) * cs[half + i];
      } else if (i < R) {
        const int j = i - half;
        a = a * cs[j] + at(j) * cs[half + j];
      }
      v[c] = a;
      ss += a * a;
    }
    float kn = 1.0f;
    if (qk_norm) kn = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int i = lane + 64 * c;
      if (i >= d) continue;
      if (isq) {
        stf(q_out + ((int64_t)t * H + head) * d + i, v[c] * kn);
      } else if (slot >= 0) {
        const int64_t pg = (slot / PAGE_TOK) * G + (head - H);
        stf(k_cache + (pg * PAGE_TOK + (slot % PAGE_TOK)) * d + i, v[c] * kn);
      }
    }
  }
  if (k_off >= 0 && slot >= 0) {
    for (int e = threadIdx.x; e < Gv * dv; e += blockDim.x) {  // (Gv value heads: G, or fewer when key heads share values)
      const int g = e / dv, i = e - g * dv;
      const int64_t pg = (slot / PAGE_TOK) * Gv + g;
      stf(v_cache + (pg * dv + i) * PAGE_TOK + (slot % PAGE_TOK), row[v_off + e] + (bias ? bias[v_off + e] : 0.0f));
    }
  }
}

// ------------------------------------------------------------------ pooled keys and values
// Block j holds the positions j pool .. j pool + pool - 1; its mean key / value is stored with the page of its last
// token, entry j - floor(64 page / pool): kp [pages, G, per, d], vp [pages, G, per, dv].  Workgroup = (completed
// block of the step, sequence, kv head); the means are taken over the caches' contents as they hold them.
template <typename AT>
__global__ void kv_pool_update_k(const AT* __restrict__ k_cache, const AT* __restrict__ v_cache, AT* __restrict__ kp,
                                 AT* __restrict__ vp, const int* __restrict__ block_tables, int width,
                                 const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, int pool, int per, int G,
                                 int d, int dv) {
  const int b = blockIdx.y, g = blockIdx.z;
  const int ctx = ctx_lens[b], nq = cu_q[b + 1] - cu_q[b];
  if (ctx <= 0 || nq <= 0) return;
  const int blk = (ctx - nq) / pool + blockIdx.x;  // first block whose last token is new, onwards
  const int first = blk * pool, lastp = first + pool - 1;
  if (lastp >= ctx) return;
  const int* bt = block_tables + (int64_t)b * width;
  const int pgi = lastp / PAGE_TOK;
  const int64_t dst = (int64_t)bt[pgi] * G + g;
  const int e = blk - (pgi * PAGE_TOK) / pool;
  const float np = (float)pool;
  for (int i = threadIdx.x; i < d + dv; i += blockDim.x) {
    float acc = 0.0f;
    if (i < d) {
      for (int p = first; p <= lastp; ++p)
        acc += ldf(k_cache + (((int64_t)bt[p / PAGE_TOK] * G + g) * PAGE_TOK + (p % PAGE_TOK)) * d + i);
      stf(kp + (dst * per + e) * d + i, acc / np);
    } else {
      const int iv = i - d;
      for (int p = first; p <= lastp; ++p)
        acc += ldf(v_cache + (((int64_t)bt[p / PAGE_TOK] * G + g) * dv + iv) * PAGE_TOK + (p % PAGE_TOK));
      stf(vp + (dst * per + e) * dv + iv, acc / np);
    }
  }
}

// ------------------------------------------------------------------ window + pooled-block attention with a sink
// A query at position i sees the tokens j with 0 <= i - j < window (window 0: all j <= i) and the pooled blocks b with
// b pool + pool - 1 <= i - window; the softmax's denominator also holds exp(sink[head]).
//
// Workgroup per (token, REP query heads of one kv head) (any d, dv <= 256, bf16 or fp32), WATT_WAVES waves: the key
// tiles are dealt to the waves in turn; a lane loads a key row once and scores it against the REP heads, and a V^T run
// of 8 keys once for the REP weighted sums.  A wave's running maxima start at -inf (wave 0: at the sinks' logits with
// denominators of one); at the end the waves' (maximum, denominator, sums) are merged through LDS.
constexpr int WATT_WAVES = 8;

template <typename AT, typename OT, int REP>
__global__ __launch_bounds__(64 * WATT_WAVES) void attn_window_pool_k(
    const AT* __restrict__ q, const AT* __restrict__ k_cache, const AT* __restrict__ v_cache, const AT* __restrict__ kp,
    const AT* __restrict__ vp, const int* __restrict__ block_tables, int width, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_lens, int B, const float* __restrict__ sink, float scale, int window, int pool, int per,
    OT* __restrict__ out, int ldo, int H, int G, int d, int dv, int Gv) {
  constexpr int TILE = REP >= 8 ? 128 : 256;
  extern __shared__ float sm[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* qs = sm;                                          // [REP][d]
  float* ws = sm + REP * d + wave * REP * TILE;            // [REP][TILE] per wave
  float* mg = sm + REP * d + WATT_WAVES * REP * TILE;      // merge: [waves][REP][2 + dv]
  const int t = blockIdx.x, h0 = blockIdx.y * REP;
  const int b = seq_of(cu_q, B, t);
  const int ctx = ctx_lens[b];
  if (ctx <= 0) return;  // padding row of a captured decode batch
  const int pos = ctx - (cu_q[b + 1] - cu_q[b]) + (t - cu_q[b]);
  const int g = h0 / (H / G);
  const int gv = g / (G / Gv);  // the value head of this key head (G / Gv neighbouring key heads share one)
  for (int i = threadIdx.x; i < REP * d; i += blockDim.x) qs[i] = ldf(q + ((int64_t)t * H + h0) * d + i);
  __syncthreads();
  const int* bt = block_tables + (int64_t)b * width;
  float m[REP], l[REP], acc[REP][4];  // value dims lane, lane + 64, ...
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    m[r] = (sink && wave == 0) ? sink[h0 + r] : -INFINITY;
    l[r] = (sink && wave == 0) ? 1.0f : 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;
  }
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int nbv = (pool > 0 && window > 0 && pos - window + 1 >= pool) ? (pos - window + 1) / pool : 0;

  auto score = [&](const AT* kr, float* s) {
#pragma unroll
    for (int r = 0; r < REP; ++r) s[r] = 0.0f;
    if (d & 7) {
      for (int i = 0; i < d; ++i) {
        const float kv = ldf(kr + i);
#pragma unroll
        for (int r = 0; r < REP; ++r) s[r] += qs[r * d + i] * kv;
      }
    } else {
      for (int i = 0; i < d; i += 8) {
        float kv[8];
        ld8(kr + i, kv);
#pragma unroll
        for (int r = 0; r < REP; ++r)
#pragma unroll
          for (int e = 0; e < 8; ++e) s[r] += qs[r * d + i + e] * kv[e];
      }
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) s[r] *= scale;
  };
  // one tile of this wave: scores of the keys a0 + [0, n) (those outside [p0, p1) weigh nothing) -> softmax weights in
  // ws, the running maxima / denominators / accumulators rescaled.  ws is the wave's own: its lanes' LDS accesses
  // are ordered by the wave-level fences.
  auto weigh = [&](int a0, int n, int p0, int p1, auto&& key_row) {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    float mx[REP];
#pragma unroll
    for (int r = 0; r < REP; ++r) mx[r] = -INFINITY;
    for (int p = a0 + lane; p < a0 + n; p += 64) {
      float s[REP];
      if (p >= p0 && p < p1) {
        score(key_row(p), s);
      } else {
#pragma unroll
        for (int r = 0; r < REP; ++r) s[r] = -INFINITY;
      }
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        ws[r * TILE + p - a0] = s[r];
        mx[r] = fmaxf(mx[r], s[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      const float mn = fmaxf(m[r], wave_max(mx[r]));
      float ls = 0.0f;
      for (int p = a0 + lane; p < a0 + n; p += 64) {
        const float s = ws[r * TILE + p - a0];
        const float w = s == -INFINITY ? 0.0f : expf(s - mn);
        ws[r * TILE + p - a0] = w;
        ls += w;
      }
      const float corr = m[r] == -INFINITY ? 0.0f : expf(m[r] - mn);
      l[r] = l[r] * corr + wave_sum(ls);
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[r][c] *= corr;
      m[r] = mn;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  int tile = 0;  // tiles are dealt to the waves in turn
  // pooled blocks [0, nbv)
  for (int a0 = 0; a0 < nbv; a0 += TILE, ++tile) {
    if (tile % WATT_WAVES != wave) continue;
    const int n = min(TILE, nbv - a0);
    weigh(a0, n, 0, nbv, [&](int j) {
      const int pgi = (j * pool + pool - 1) / PAGE_TOK;
      return kp + (((int64_t)bt[pgi] * G + g) * per + (j - (pgi * PAGE_TOK) / pool)) * d;
    });
    for (int j = a0; j < a0 + n; ++j) {
      const int pgi = (j * pool + pool - 1) / PAGE_TOK;
      const AT* vr = vp + (((int64_t)bt[pgi] * G + g) * per + (j - (pgi * PAGE_TOK) / pool)) * dv;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int i = lane + 64 * c;
        if (i < dv) {
          const float vv = ldf(vr + i);
#pragma unroll
          for (int r = 0; r < REP; ++r) acc[r][c] += ws[r * TILE + j - a0] * vv;
        }
      }
    }
  }
  // tokens [lo, pos], tiles aligned to 8 keys
  for (int a0 = lo & ~7; a0 <= pos; a0 += TILE, ++tile) {
    if (tile % WATT_WAVES != wave) continue;
    const int a1 = min(a0 + TILE, (pos + 8) & ~7);
    weigh(a0, a1 - a0, lo, pos + 1, [&](int p) {
      return k_cache + (((int64_t)bt[p / PAGE_TOK] * G + g) * PAGE_TOK + (p % PAGE_TOK)) * d;
    });
    for (int p = a0; p < a1; p += 8) {  // 8 keys of one page per step
      const AT* vq = v_cache + ((int64_t)bt[p / PAGE_TOK] * Gv + gv) * dv * PAGE_TOK + (p % PAGE_TOK);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int i = lane + 64 * c;
        if (i < dv) {
          float vv[8];
          ld8(vq + (int64_t)i * PAGE_TOK, vv);
#pragma unroll
          for (int r = 0; r < REP; ++r)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float w = ws[r * TILE + p - a0 + e];
              acc[r][c] += w != 0.0f ? w * vv[e] : 0.0f;  // (a slot no token has written yet may hold anything)
            }
        }
      }
    }
  }
  // merge the waves: M = max m_w, out = sum_w acc_w e^(m_w - M) / sum_w l_w e^(m_w - M)
  const int ms = 2 + dv;
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    float* mine = mg + (wave * REP + r) * ms;
    if (lane == 0) {
      mine[0] = m[r];
      mine[1] = l[r];
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int i = lane + 64 * c;
      if (i < dv) mine[2 + i] = acc[r][c];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < REP * dv; e += blockDim.x) {
    const int r = e / dv, i = e - r * dv;
    float M = -INFINITY;
    for (int w = 0; w < WATT_WAVES; ++w) M = fmaxf(M, mg[(w * REP + r) * ms]);
    float L = 0.0f, a = 0.0f;
    for (int w = 0; w < WATT_WAVES; ++w) {
      const float* o = mg + (w * REP + r) * ms;
      if (o[0] != -INFINITY) {
        const float f = expf(o[0] - M);
        L += o[1] * f;
        a += o[2 + i] * f;
      }
    }
    stf(out + (int64_t)t * ldo + (h0 + r) * dv + i, L > 0.0f ? a / L : 0.0f);
  }
}

// MFMA kernel (bf16 caches; key size 32 NK, value size 32 NV; output bf16 or fp32): a workgroup owns 128 consecutive queries of one (sequence, head), 32 per wave, and
// walks first the pooled blocks that its last query sees, then the tokens from its first query's window on, a tile of
// KT keys at a time: the K rows and V^T runs of the tile are staged in LDS and shared by the four waves (pooled
// entries are gathered row by row and their values transposed on the way in).  Scores are computed transposed,
// S^T = K Q^T (keys x queries), so a lane's accumulator rows are consecutive keys of ONE query: the running maximum and
// denominator are per lane (the four lanes of a query agree on the maximum through two shuffles and keep partial
// denominators), and the exponentials, rounded to bf16, are as they lie the B operand of O^T += V^T P^T, whose k slots
// (g, j) are read as keys {4g .. 4g+3, 16+4g .. 16+4g+3} on both operands.  Scores, maxima and sums are fp32 (base-2
// exponentials of scores scaled by log2 e); the sink's logit starts the running maximum with a denominator of one.
template <int NK, int NV, typename OT>
__global__ __launch_bounds__(256) void attn_window_pool_mfma_k(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    const uint16_t* __restrict__ kp, const uint16_t* __restrict__ vp, const int* __restrict__ block_tables, int width,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, const float* __restrict__ sink, float scale, int window,
    int pool, int per, OT* __restrict__ out, int ldo, int H, int G, int Gv) {
  // key size D = 32 NK, value size DV = 32 NV (pooled blocks: NK == NV); G / Gv neighbouring key heads share a value head
  constexpr int D = NK * 32, DV = NV * 32, ND = NV * 2, QT = 2;
  constexpr int KT = (D > 192 || DV > 192) ? 32 : 64;  // keys per tile (a page holds a whole number of tiles)
  constexpr int KP = D + 8, VP = KT + 8;
  constexpr float L2E = 1.4426950408889634f;
  __shared__ __attribute__((aligned(16))) uint16_t sK[KT][KP], sV[DV][VP];
  const int b = blockIdx.x, h = blockIdx.z;
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, c = l & 15, g4 = l >> 4;
  const int t0 = cu_q[b], qlen = cu_q[b + 1] - t0, ctx = ctx_lens[b];
  const int wq0 = blockIdx.y * 128;
  if (ctx <= 0 || wq0 >= qlen) return;
  const int q0 = wq0 + wave * 32;
  const bool active = q0 < qlen;
  const int nq = active ? min(32, qlen - q0) : 0;
  const int pos0 = ctx - qlen + q0;  // position of the wave's first query
  const int gk = h / (H / G), gv = gk / (G / Gv);
  // pooled blocks a query at position p sees: those that end at or before p - window
  auto blocks_seen = [&](int p) { return (pool > 0 && p - window + 1 >= pool) ? (p - window + 1) / pool : 0; };
  s16x8 qf[QT][NK];
  int qpos[QT], qnb[QT];
  float m[QT], lsum[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int local = qt * 16 + c;
    const bool ok = local < nq;
    qpos[qt] = pos0 + local;
    qnb[qt] = blocks_seen(qpos[qt]);
    const uint16_t* qp = q + ((int64_t)(t0 + q0 + local) * H + h) * D + 8 * g4;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) qf[qt][ks] = ok ? ld16(qp + ks * 32) : s16x8{0, 0, 0, 0, 0, 0, 0, 0};
    m[qt] = sink ? sink[h] * L2E : -INFINITY;
    lsum[qt] = (sink && g4 == 0) ? 1.0f : 0.0f;  // (partial denominators: one of the query's four lanes counts the sink)
  }
  f32x4 o[QT][ND];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt)
#pragma unroll
    for (int db = 0; db < ND; ++db) o[qt][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float sc2 = scale * L2E;
  const int* bt = block_tables + (int64_t)b * width;
  const int wlast = ctx - qlen + wq0 + min(128, qlen - wq0) - 1;  // the workgroup's last query
  const int wpos0 = ctx - qlen + wq0;
  const int last = active ? pos0 + nq - 1 : -1;                  // the wave's last query
  constexpr int NCHUNK = KT * (D / 8), NCH = (NCHUNK + 255) / 256;
  constexpr int NCHUNKV = KT * (DV / 8), NCHV = (NCHUNKV + 255) / 256;
  s16x8 rk[NCH], rv[NCHV];

  // one staged tile: scores, mask, running softmax, O^T += V^T P^T.  pooled: key index = block index.
  auto consume = [&](int tb, bool pooled) {
#pragma unroll
    for (int sub = 0; sub < KT / 32; ++sub) {
      const int kb = tb + sub * 32;
      bool full;
      if (pooled) {
        if (!active || kb >= blocks_seen(last)) continue;  // (wave-uniform) none of these blocks is seen by this wave
        full = kb + 32 <= blocks_seen(pos0);
      } else {
        const int k_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
        if (!active || kb > last || kb + 31 < k_lo) continue;
        full = kb + 31 <= pos0 && (window <= 0 || kb > last - window);
      }
      f32x4 s[2][QT];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) s[kt][qt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NK; ++ks)
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          const s16x8 a = ld16(&sK[sub * 32 + kt * 16 + c][ks * 32 + 8 * g4]);
#pragma unroll
          for (int qt = 0; qt < QT; ++qt) s[kt][qt] = mfma16(a, qf[qt][ks], s[kt][qt]);
        }
      s16x8 pf[QT];
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float t = s[kt][qt][r] * sc2;
            if (!full) {
              const int kpos = kb + kt * 16 + 4 * g4 + r;
              const bool vis = pooled ? kpos < qnb[qt] : (kpos <= qpos[qt] && (window <= 0 || qpos[qt] - kpos < window));
              t = vis ? t : -INFINITY;
            }
            s[kt][qt][r] = t;
            mx = fmaxf(mx, t);
          }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m[qt], mx);
        const float ms = mn == -INFINITY ? 0.0f : mn;  // (nothing seen yet: every weight below is exp2(-inf) = 0)
        const float corr = __builtin_amdgcn_exp2f(m[qt] - ms);
        m[qt] = mn;
        float ps = 0.0f;
        u32x4 packed;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r2 = 0; r2 < 2; ++r2) {
            const float p0 = __builtin_amdgcn_exp2f(s[kt][qt][2 * r2] - ms), p1 = __builtin_amdgcn_exp2f(s[kt][qt][2 * r2 + 1] - ms);
            ps += p0 + p1;
            // two bf16 (rounded half up: the weights are in [0, 1]) in one dword
            packed[kt * 2 + r2] = __builtin_amdgcn_perm(__float_as_uint(p1) + 0x8000u, __float_as_uint(p0) + 0x8000u, 0x07060302u);
          }
        pf[qt] = __builtin_bit_cast(s16x8, packed);
        lsum[qt] = lsum[qt] * corr + ps;
#pragma unroll
        for (int db = 0; db < ND; ++db) o[qt][db] *= corr;
      }
      // (slots no token has written yet hold zeros or an earlier request's finite values; their weight is 0)
#pragma unroll
      for (int db = 0; db < ND; ++db) {
        const s16x4 v0 = *reinterpret_cast<const s16x4*>(&sV[db * 16 + c][sub * 32 + 4 * g4]);
        const s16x4 v1 = *reinterpret_cast<const s16x4*>(&sV[db * 16 + c][sub * 32 + 16 + 4 * g4]);
        const s16x8 a = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) o[qt][db] = mfma16(a, pf[qt], o[qt][db]);
      }
    }
  };

  // ---- pooled blocks [0, nbw): rows gathered from the pages that hold them, values transposed into sV
  const int nbw = NK == NV ? blocks_seen(wlast) : 0;
  for (int tb = 0; tb < nbw; tb += KT) {
    __syncthreads();  // the previous tile has been consumed
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int ch = threadIdx.x + 256 * j;
      if (NCHUNK % 256 != 0 && ch >= NCHUNK) break;
      const int row = ch / (D / 8), cc = ch - row * (D / 8);
      const int blk = min(tb + row, nbw - 1);  // (rows past the last block repeat it; their weight is 0)
      const int pgi = (blk * pool + pool - 1) / PAGE_TOK;
      const int64_t e = ((int64_t)bt[pgi] * G + gk) * per + (blk - (pgi * PAGE_TOK) / pool);
      st16(&sK[row][cc * 8], ld16(kp + e * D + cc * 8));
      const s16x8 v = ld16(vp + e * D + cc * 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) sV[cc * 8 + i][row] = (uint16_t)v[i];
    }
    __syncthreads();
    consume(tb, true);
  }

  // ---- tokens from the first query's window on
  const int t_lo = (window > 0 ? max(0, wpos0 - window + 1) : 0) & ~(KT - 1);
  auto fetch = [&](int tb) {
    const int64_t pg = (int64_t)bt[tb >> 6] * G + gk, pgv = (int64_t)bt[tb >> 6] * Gv + gv;
    const int koff = tb & 63;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int ch = threadIdx.x + 256 * j;
      if (NCHUNK % 256 != 0 && ch >= NCHUNK) break;
      const int row = ch / (D / 8), cc = ch - row * (D / 8);
      rk[j] = ld16(k_cache + ((pg * PAGE_TOK) + koff + row) * D + cc * 8);
    }
#pragma unroll
    for (int j = 0; j < NCHV; ++j) {
      const int ch = threadIdx.x + 256 * j;
      if (NCHUNKV % 256 != 0 && ch >= NCHUNKV) break;
      const int vrow = ch / (KT / 8), vc = ch - vrow * (KT / 8);
      rv[j] = ld16(v_cache + (pgv * DV + vrow) * PAGE_TOK + koff + vc * 8);
    }
  };
  fetch(t_lo);
  for (int tb = t_lo; tb <= wlast; tb += KT) {
    __syncthreads();  // the previous tile has been consumed
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int ch = threadIdx.x + 256 * j;
      if (NCHUNK % 256 != 0 && ch >= NCHUNK) break;
      const int row = ch / (D / 8), cc = ch - row * (D / 8);
      st16(&sK[row][cc * 8], rk[j]);
    }
#pragma unroll
    for (int j = 0; j < NCHV; ++j) {
      const int ch = threadIdx.x + 256 * j;
      if (NCHUNKV % 256 != 0 && ch >= NCHUNKV) break;
      const int vrow = ch / (KT / 8), vc = ch - vrow * (KT / 8);
      st16(&sV[vrow][vc * 8], rv[j]);
    }
    __syncthreads();
    if (tb + KT <= wlast) fetch(tb + KT);  // in flight while this tile is consumed
    consume(tb, false);
  }
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    float ls = lsum[qt];
    ls += __shfl_xor(ls, 16, 64);
    ls += __shfl_xor(ls, 32, 64);
    if (qt * 16 + c >= nq) continue;
    const float inv = ls > 0.0f ? 1.0f / ls : 0.0f;
    OT* op = out + (int64_t)(t0 + q0 + qt * 16 + c) * ldo + h * DV + 4 * g4;
#pragma unroll
    for (int db = 0; db < ND; ++db) {
      if constexpr (sizeof(OT) == 4) {
        *reinterpret_cast<f32x4*>(op + db * 16) = f32x4{o[qt][db][0] * inv, o[qt][db][1] * inv, o[qt][db][2] * inv, o[qt][db][3] * inv};
      } else {
        s16x4 w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = (short)f2bf(o[qt][db][r] * inv);
        *reinterpret_cast<s16x4*>(op + db * 16) = w;
      }
    }
  }
}

// ------------------------------------------------------------------ SSD inputs
// Channels [x: H dv | B: G N | C: G N] at P[:, x_off ...]; conv_w [C, taps] (last column: the current token), bias
// conv_b; conv_state [slots, taps - 1, C] holds the inputs before this step (zeros for a new sequence).
// xbc [T, C] = silu(conv + bias); dt = softplus(P[dt_off + h] + dt_bias[h]); v [T, H dv] = dt x;
// decay [T, H] = exp(-exp(A_log[h]) dt).
__global__ void ssd_prep_k(const float* __restrict__ P, int ldp, int x_off, int dt_off, const float* __restrict__ conv_w,
                           const float* __restrict__ conv_b, int taps, int C, const float* __restrict__ conv_state,
                           const int* __restrict__ state_slots, const int* __restrict__ cu_q, int B,
                           const float* __restrict__ A_log, const float* __restrict__ dt_bias, int H, int dv,
                           float* __restrict__ xbc, float* __restrict__ v, float* __restrict__ decay) {
  const int t = blockIdx.x;
  const int b = seq_of(cu_q, B, t);
  const int slot = state_slots[b];
  if (slot < 0) return;
  const int tstart = cu_q[b], local = t - tstart;
  const float* row = P + (int64_t)t * ldp;
  const float* st = conv_state + (int64_t)slot * (taps - 1) * C;
  const int inner = H * dv;
  extern __shared__ float dts[];  // [H] step sizes of this token
  for (int h = threadIdx.x; h < H; h += blockDim.x) dts[h] = softplusf_(row[dt_off + h] + dt_bias[h]);
  __syncthreads();
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float acc = conv_b[c];
    for (int j = 0; j < taps; ++j) {
      const int sidx = local - (taps - 1 - j);
      const float x = sidx >= 0 ? P[(int64_t)(tstart + sidx) * ldp + x_off + c] : st[(int64_t)(taps - 1 + sidx) * C + c];
      acc += conv_w[c * taps + j] * x;
    }
    const float y = siluf_(acc);
    xbc[(int64_t)t * C + c] = y;
    if (c < inner) v[(int64_t)t * inner + c] = dts[c / dv] * y;
  }
  if (blockIdx.y == 0)
    for (int h = threadIdx.x; h < H; h += blockDim.x) decay[(int64_t)t * H + h] = expf(-expf(A_log[h]) * dts[h]);
}

// the last taps - 1 convolution inputs of every sequence -> its state slot (after every token of the step has read
// the old state: a launch of its own)
__global__ void conv_tail_store_k(const float* __restrict__ P, int ldp, int x_off, int C, int taps,
                                  float* __restrict__ conv_state, const int* __restrict__ state_slots,
                                  const int* __restrict__ cu_q) {
  const int b = blockIdx.x;
  const int slot = state_slots[b];
  const int n = cu_q[b + 1] - cu_q[b];
  if (slot < 0 || n <= 0) return;
  float* st = conv_state + (int64_t)slot * (taps - 1) * C;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    // ascending: entry idx takes the old entry idx + n (> idx) or a token of this step
    for (int idx = 0; idx < taps - 1; ++idx) {
      const int s = n - (taps - 1) + idx;
      st[(int64_t)idx * C + c] = s >= 0 ? P[(int64_t)(cu_q[b] + s) * ldp + x_off + c] : st[(int64_t)(idx + n) * C + c];
    }
  }
}

// ------------------------------------------------------------------ SSD output: skip, gate, grouped RMS norm, weight
// workgroup = (token, norm group)
template <typename AT>
__global__ void ssd_gate_norm_k(const float* __restrict__ o, const float* __restrict__ xbc, int C,
                                const float* __restrict__ skip, const float* __restrict__ P, int ldp, int z_off,
                                const float* __restrict__ w, float eps, AT* __restrict__ out, int ldo, int inner, int dv,
                                int gs) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int c0 = blockIdx.y * gs;
  auto val = [&](int c) {
    return (o[t * inner + c] + skip[c / dv] * xbc[t * C + c]) * siluf_(P[t * ldp + z_off + c]);
  };
  float ss = 0.0f;
  for (int i = threadIdx.x; i < gs; i += blockDim.x) {
    const float y = val(c0 + i);
    ss += y * y;
  }
  ss = block_sum(ss, red);
  const float k = 1.0f / sqrtf(ss / (float)gs + eps);
  for (int i = threadIdx.x; i < gs; i += blockDim.x) stf(out + t * ldo + c0 + i, val(c0 + i) * k * w[c0 + i]);
}

// ------------------------------------------------------------------ PolyNorm
// One workgroup per token.  Rows of at most PN_REG values a thread are read once and kept in registers between the
// three sums and the polynomial; longer rows are read twice.
constexpr int PN_REG = 16;

template <typename AT>
__global__ void polynorm_act_k(const float* __restrict__ P, int ldp, int up_off, int F, const float* __restrict__ coef,
                               float eps, AT* __restrict__ out, int ldo) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float* z = P + t * ldp + up_off;
  const bool held = F <= PN_REG * (int)blockDim.x;
  float zr[PN_REG];
  float s2 = 0.0f, s4 = 0.0f, s6 = 0.0f;
  if (held) {
#pragma unroll
    for (int j = 0; j < PN_REG; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      const float a = i < F ? z[i] : 0.0f, a2 = a * a, a3 = a2 * a;
      zr[j] = a;
      s2 += a2;
      s4 += a2 * a2;
      s6 += a3 * a3;
    }
  } else {
    for (int i = threadIdx.x; i < F; i += blockDim.x) {
      const float a = z[i], a2 = a * a, a3 = a2 * a;
      s2 += a2;
      s4 += a2 * a2;
      s6 += a3 * a3;
    }
  }
  s2 = block_sum(s2, red);
  s4 = block_sum(s4, red);
  s6 = block_sum(s6, red);
  const float k1 = coef[0] / sqrtf(s2 / (float)F + eps), k2 = coef[1] / sqrtf(s4 / (float)F + eps),
              k3 = coef[2] / sqrtf(s6 / (float)F + eps), e = coef[3];
  if (held) {
#pragma unroll
    for (int j = 0; j < PN_REG; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      const float a = zr[j], a2 = a * a;
      if (i < F) stf(out + t * ldo + i, k1 * a + k2 * a2 + k3 * a2 * a + e);
    }
  } else {
    for (int i = threadIdx.x; i < F; i += blockDim.x) {
      const float a = z[i], a2 = a * a;
      stf(out + t * ldo + i, k1 * a + k2 * a2 + k3 * a2 * a + e);
    }
  }
}

template <typename AT>
__global__ void relu2_k(const float* __restrict__ P, int ldp, int off, int F, AT* __restrict__ out, int ldo, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t t = idx / F;
  const int i = (int)(idx - t * F);
  const float z = fmaxf(P[t * ldp + off + i], 0.0f);
  stf(out + t * ldo + i, z * z);
}

// ------------------------------------------------------------------ routed experts' weighted sum + gated shared expert
// y [splits * slots, >= D]: the down projection's K slices (summed here in a fixed order)
__global__ void moe_weighted_sum_k(const float* __restrict__ y, int ldy, const int* __restrict__ slot_of,
                                   const float* __restrict__ topw, int k, int splits, int64_t slots,
                                   const float* __restrict__ sh, int lds, const float* __restrict__ P, int ldp, int shg_off,
                                   float* __restrict__ out, int D) {
  const int64_t t = blockIdx.x;
  const float sg = !sh ? 0.0f : (P ? sigmoidf_(P[t * ldp + shg_off]) : 1.0f);  // (no gate: the shared expert is added as it is)
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    float acc = 0.0f;
    for (int j = 0; j < k; ++j) {
      const int64_t r = slot_of[t * k + j];
      float ys = 0.0f;
      for (int sp = 0; sp < splits; ++sp) ys += y[(sp * slots + r) * ldy + i];
      acc += topw[t * k + j] * ys;
    }
    if (sh) acc += sg * sh[t * lds + i];
    out[t * D + i] = acc;
  }
}

// ------------------------------------------------------------------ host side
// XOT_WATT_MFMA=0 keeps prompt portions on the wave-per-token attention kernel (A/B runs)
const bool WATT_MFMA = []() { const char* e = getenv("XOT_WATT_MFMA"); return !(e && e[0] == '0'); }();

void gated_postnorm(at::Tensor& x, const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& P, int64_t g_off,
                    const c10::optional<at::Tensor>& gate_b, double alpha, const at::Tensor& w, double eps,
                    const c10::optional<at::Tensor>& out) {
  f32c(x, "x");
  f32c(w, "w");
  MCHECK(x.dim() == 2, "x must be [T, D]");
  const int64_t T = x.size(0), D = x.size(1);
  if (T == 0) return;
  MCHECK(w.numel() == D, "the norm weight must hold D numbers");
  int ldy = 0, ldp = 0, ldo = 0;
  if (y.has_value()) {
    ldy = ld_of(*y, "y");
    MCHECK(y->size(0) == T && y->size(1) >= D, "the sublayer's result must be fp32 [T, >= D] rows");
  }
  if (P.has_value()) {
    MCHECK(y.has_value() && gate_b.has_value(), "a gate needs the sublayer's result and the gate's bias");
    ldp = ld_of(*P, "P");
    MCHECK(P->size(0) == T, "P must have T rows");
    cols_ok(*P, g_off, D, "gate");
    f32c(*gate_b, "gate_b");
    MCHECK(gate_b->numel() == D, "the gate's bias must hold D numbers");
  }
  if (out.has_value()) ldo = act_ld_min(*out, T, D, "out");
  const float* yp = y.has_value() ? y->data_ptr<float>() : nullptr;
  const float* pp = P.has_value() ? P->data_ptr<float>() : nullptr;
  const float* gp = P.has_value() ? gate_b->data_ptr<float>() : nullptr;
  if (out.has_value() && out->scalar_type() == at::kBFloat16)
    gated_postnorm_k<uint16_t><<<T, 256, 0, stream()>>>(x.data_ptr<float>(), yp, ldy, pp, ldp, (int)g_off, gp, (float)alpha,
                                                        w.data_ptr<float>(), (float)eps, (uint16_t*)out->data_ptr(), ldo, (int)D);
  else
    gated_postnorm_k<float><<<T, 256, 0, stream()>>>(x.data_ptr<float>(), yp, ldy, pp, ldp, (int)g_off, gp, (float)alpha,
                                                     w.data_ptr<float>(), (float)eps,
                                                     out.has_value() ? out->data_ptr<float>() : nullptr, ldo, (int)D);
}

void check_kv(const at::Tensor& k_cache, const at::Tensor& v_cache, at::ScalarType dt, int64_t G, int64_t d, int64_t dv) {
  MCHECK(k_cache.is_cuda() && k_cache.scalar_type() == dt && k_cache.is_contiguous() && k_cache.dim() == 4 &&
             k_cache.size(1) == G && k_cache.size(2) == PAGE_TOK && k_cache.size(3) == d,
         "k_cache must be [pages, G, 64, d] of the activations' dtype");
  MCHECK(v_cache.is_cuda() && v_cache.scalar_type() == dt && v_cache.is_contiguous() && v_cache.dim() == 4 &&
             v_cache.size(0) == k_cache.size(0) && v_cache.size(1) >= 1 && G % v_cache.size(1) == 0 && v_cache.size(2) == dv &&
             v_cache.size(3) == PAGE_TOK,
         "v_cache must be [pages, Gv, dv, 64] of the activations' dtype, Gv = G or a divisor of it (key heads that share values)");
}

void qk_norm_rope_store(const at::Tensor& P, const c10::optional<at::Tensor>& bias, int64_t q_off, int64_t k_off,
                        int64_t v_off, int64_t H, int64_t G, int64_t d, int64_t dv, int64_t R, const at::Tensor& pos,
                        const at::Tensor& cos_sin, const at::Tensor& slots, double eps, bool qk_norm, at::Tensor& q_out,
                        at::Tensor& k_cache, at::Tensor& v_cache) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  int64_t Gv = G;
  if (T == 0) return;
  i32c(pos, "pos");
  f32c(cos_sin, "cos_sin");
  MCHECK(slots.is_cuda() && slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.numel() == T && pos.numel() == T,
         "pos / slots must hold one entry per token");
  MCHECK(R % 2 == 0 && R >= 0 && R <= d && (R == 0 || (cos_sin.dim() == 2 && cos_sin.size(1) == R)), "bad rotary dims");
  MCHECK(H > 0 && G > 0 && H % G == 0 && d > 0 && d <= 256 && dv > 0 && dv <= 256, "head counts / sizes (at most 256)");
  cols_ok(P, q_off, H * d, "q");
  if (k_off >= 0) {
    MCHECK(v_off >= 0, "keys without values");
    cols_ok(P, k_off, G * d, "k");
    check_kv(k_cache, v_cache, q_out.scalar_type(), G, d, dv);
    Gv = v_cache.size(1);
    cols_ok(P, v_off, Gv * dv, "v");
  }
  const float* bp = nullptr;
  if (bias.has_value()) {
    f32c(*bias, "bias");
    MCHECK(bias->numel() >= std::max(q_off + H * d, std::max(k_off + G * d, v_off + Gv * dv)), "bias must cover the q / k / v columns");
    bp = bias->data_ptr<float>();
  }
  MCHECK(q_out.is_cuda() && is_act(q_out) && q_out.is_contiguous() && q_out.numel() == T * H * d, "q_out must be [T, H, d]");
  // positions and slots are checked on the host by their producer (the block manager hands out slots < pages * 64
  // and the runner bounds positions by the table's rows)
  if (q_out.scalar_type() == at::kBFloat16)
    qk_norm_rope_store_k<uint16_t><<<T, 256, 0, stream()>>>(
        P.data_ptr<float>(), ldp, bp, (int)q_off, (int)k_off, (int)v_off, (int)H, (int)G, (int)d, (int)dv, (int)R,
        pos.data_ptr<int>(), cos_sin.data_ptr<float>(), slots.data_ptr<int64_t>(), (float)eps, (int)qk_norm,
        (uint16_t*)q_out.data_ptr(), (uint16_t*)k_cache.data_ptr(), (uint16_t*)v_cache.data_ptr(), (int)Gv);
  else
    qk_norm_rope_store_k<float><<<T, 256, 0, stream()>>>(
        P.data_ptr<float>(), ldp, bp, (int)q_off, (int)k_off, (int)v_off, (int)H, (int)G, (int)d, (int)dv, (int)R,
        pos.data_ptr<int>(), cos_sin.data_ptr<float>(), slots.data_ptr<int64_t>(), (float)eps, (int)qk_norm,
        q_out.data_ptr<float>(), k_cache.data_ptr<float>(), v_cache.data_ptr<float>(), (int)Gv);
}

void check_pools(const at::Tensor& k_cache, const at::Tensor& kp, const at::Tensor& vp, int64_t pool, int64_t G, int64_t d,
                 int64_t dv, int* per) {
  MCHECK(pool >= 1, "pool must be at least one token");
  *per = (int)((PAGE_TOK + pool - 1) / pool);
  MCHECK(kp.is_cuda() && kp.scalar_type() == k_cache.scalar_type() && kp.is_contiguous() && kp.dim() == 4 &&
             kp.size(0) == k_cache.size(0) && kp.size(1) == G && kp.size(2) == *per && kp.size(3) == d,
         "the pooled keys must be [pages, G, ceil(64 / pool), d] of the caches' dtype");
  MCHECK(vp.is_cuda() && vp.scalar_type() == k_cache.scalar_type() && vp.is_contiguous() && vp.dim() == 4 &&
             vp.size(0) == k_cache.size(0) && vp.size(1) == G && vp.size(2) == *per && vp.size(3) == dv,
         "the pooled values must be [pages, G, ceil(64 / pool), dv] of the caches' dtype");
}

void kv_pool_update(const at::Tensor& k_cache, const at::Tensor& v_cache, at::Tensor& kp, at::Tensor& vp,
                    const at::Tensor& block_tables, const at::Tensor& cu_q, const at::Tensor& ctx_lens, int64_t pool,
                    int64_t max_qlen) {
  MCHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && is_act(k_cache), "caches must be 4-D bf16 / fp32");
  const int64_t G = k_cache.size(1), d = k_cache.size(3), dv = v_cache.size(2), B = ctx_lens.numel();
  check_kv(k_cache, v_cache, k_cache.scalar_type(), G, d, dv);
  MCHECK(v_cache.size(1) == G, "pooled blocks need a value head per key head");
  int per;
  check_pools(k_cache, kp, vp, pool, G, d, dv, &per);
  i32c(block_tables, "block_tables");
  i32c(cu_q, "cu_q");
  i32c(ctx_lens, "ctx_lens");
  MCHECK(block_tables.dim() == 2 && block_tables.size(0) == B && cu_q.numel() == B + 1, "step tensors do not fit the batch");
  if (B == 0 || max_qlen <= 0) return;
  const dim3 grid((unsigned)(max_qlen / pool + 2), (unsigned)B, (unsigned)G);
  const int bs = (int)std::min<int64_t>(256, ((d + dv + 63) / 64) * 64);
  if (k_cache.scalar_type() == at::kBFloat16)
    kv_pool_update_k<uint16_t><<<grid, bs, 0, stream()>>>(
        (const uint16_t*)k_cache.data_ptr(), (const uint16_t*)v_cache.data_ptr(), (uint16_t*)kp.data_ptr(),
        (uint16_t*)vp.data_ptr(), block_tables.data_ptr<int>(), (int)block_tables.size(1), cu_q.data_ptr<int>(),
        ctx_lens.data_ptr<int>(), (int)pool, per, (int)G, (int)d, (int)dv);
  else
    kv_pool_update_k<float><<<grid, bs, 0, stream()>>>(
        k_cache.data_ptr<float>(), v_cache.data_ptr<float>(), kp.data_ptr<float>(), vp.data_ptr<float>(),
        block_tables.data_ptr<int>(), (int)block_tables.size(1), cu_q.data_ptr<int>(), ctx_lens.data_ptr<int>(), (int)pool,
        per, (int)G, (int)d, (int)dv);
}

template <int NK, int NV, typename OT>
void launch_wattn_mfma(dim3 grid, const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache, const uint16_t* kp,
                       const uint16_t* vp, const at::Tensor& block_tables, const at::Tensor& cu_q, const at::Tensor& ctx_lens,
                       const float* sink, float scale, int window, int pool, int per, at::Tensor& out, int ldo, int H, int G) {
  attn_window_pool_mfma_k<NK, NV, OT><<<grid, 256, 0, stream()>>>(
      (const uint16_t*)q.data_ptr(), (const uint16_t*)k_cache.data_ptr(), (const uint16_t*)v_cache.data_ptr(), kp, vp,
      block_tables.data_ptr<int>(), (int)block_tables.size(1), cu_q.data_ptr<int>(), ctx_lens.data_ptr<int>(), sink, scale,
      window, pool, per, (OT*)out.data_ptr(), ldo, H, G, (int)v_cache.size(1));
}

// max_qlen: the longest run of new tokens of one sequence in this step (below 16: single decoded tokens and short
// portions -> the wave-per-token kernel; the MFMA kernel takes bf16 with d == dv in {32, 64, 128}).
void attn_window_pool(const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                      const c10::optional<at::Tensor>& kp, const c10::optional<at::Tensor>& vp, const at::Tensor& block_tables,
                      const at::Tensor& cu_q, const at::Tensor& ctx_lens, const c10::optional<at::Tensor>& sink, double scale,
                      int64_t window, int64_t pool, at::Tensor& out, int64_t max_qlen) {
  MCHECK(q.is_cuda() && is_act(q) && q.is_contiguous() && q.dim() == 3, "q must be contiguous [T, H, d]");
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2), B = ctx_lens.numel();
  if (T == 0 || B == 0) return;
  MCHECK(k_cache.dim() == 4 && v_cache.dim() == 4, "caches must be 4-D");
  const int64_t G = k_cache.size(1), dv = v_cache.size(2);
  check_kv(k_cache, v_cache, q.scalar_type(), G, d, dv);
  MCHECK(G > 0 && H % G == 0 && d <= 256 && dv <= 256, "head counts / sizes (at most 256)");
  MCHECK(window >= 0 && pool >= 0, "window / pool must not be negative");
  int per = 0;
  const bool pooled = pool > 0 && window > 0;
  if (pooled) {
    MCHECK(kp.has_value() && vp.has_value(), "pooled blocks need the pooled caches");
    check_pools(k_cache, *kp, *vp, pool, G, d, dv, &per);
  }
  i32c(block_tables, "block_tables");
  i32c(cu_q, "cu_q");
  i32c(ctx_lens, "ctx_lens");
  MCHECK(block_tables.dim() == 2 && block_tables.size(0) == B && cu_q.numel() == B + 1, "step tensors do not fit the batch");
  const float* sp = nullptr;
  if (sink.has_value()) {
    f32c(*sink, "sink");
    MCHECK(sink->numel() == H, "sink must hold one logit per head");
    sp = sink->data_ptr<float>();
  }
  const int64_t Gv = v_cache.size(1);
  MCHECK(out.scalar_type() == q.scalar_type() || out.scalar_type() == at::kFloat, "out must have q's dtype or be fp32");
  MCHECK(!pooled || Gv == G, "pooled blocks need a value head per key head");
  const int ldo = act_ld(out, T, H * dv, "out");
  const bool o32 = out.scalar_type() == at::kFloat;
  // the MFMA kernel: bf16 caches, runs of 16 tokens or more, value size = key size in {32, 64, 128} (bf16 or fp32 output)
  // or twice the key size in {32, 64} with fp32 output (differential attention's maps); pooled blocks need equal sizes
  const bool same = d == dv && (d == 32 || d == 64 || d == 128), twice = dv == 2 * d && (d == 32 || d == 64) && o32 && !pooled;
  if (q.scalar_type() == at::kBFloat16 && max_qlen >= 16 && (same || twice) && ldo % 4 == 0 && WATT_MFMA) {
    const dim3 grid((unsigned)B, (unsigned)((max_qlen + 127) / 128), (unsigned)H);
    const uint16_t* kpp = pooled ? (const uint16_t*)kp->data_ptr() : nullptr;
    const uint16_t* vpp = pooled ? (const uint16_t*)vp->data_ptr() : nullptr;
    const int pl = pooled ? (int)pool : 0;
#define WATT_MFMA_GO(NK, NV, OT)                                                                                            \
  launch_wattn_mfma<NK, NV, OT>(grid, q, k_cache, v_cache, kpp, vpp, block_tables, cu_q, ctx_lens, sp, (float)scale,       \
                                (int)window, pl, per, out, ldo, (int)H, (int)G)
    if (twice && d == 32) WATT_MFMA_GO(1, 2, float);
    else if (twice) WATT_MFMA_GO(2, 4, float);
    else if (d == 32 && o32) WATT_MFMA_GO(1, 1, float);
    else if (d == 32) WATT_MFMA_GO(1, 1, uint16_t);
    else if (d == 64 && o32) WATT_MFMA_GO(2, 2, float);
    else if (d == 64) WATT_MFMA_GO(2, 2, uint16_t);
    else if (o32) WATT_MFMA_GO(4, 4, float);
    else WATT_MFMA_GO(4, 4, uint16_t);
#undef WATT_MFMA_GO
    return;
  }
  // query heads of one kv head share a workgroup (each key row and value run is loaded once for all of them)
  const int rep_all = (int)(H / G);
  int rep = rep_all % 8 == 0 ? 8 : rep_all % 4 == 0 ? 4 : rep_all % 2 == 0 ? 2 : 1;
  auto lds_of = [&](int r) {
    return (size_t)(r * d + WATT_WAVES * r * (r >= 8 ? 128 : 256) + WATT_WAVES * r * (2 + dv)) * sizeof(float);
  };
  // (the default limit of dynamic LDS per workgroup is 64 KB; a small step keeps a workgroup per head to fill the chip)
  while (rep > 1 && (lds_of(rep) > 60 * 1024 || T * (H / rep) < 256)) rep /= 2;
  const dim3 grid((unsigned)T, (unsigned)(H / rep));
  const size_t lds = lds_of(rep);
#define WATT_GO(AT, OT, R)                                                                                                 \
  attn_window_pool_k<AT, OT, R><<<grid, 64 * WATT_WAVES, lds, stream()>>>(                                                 \
      (const AT*)q.data_ptr(), (const AT*)k_cache.data_ptr(), (const AT*)v_cache.data_ptr(),                               \
      pooled ? (const AT*)kp->data_ptr() : nullptr, pooled ? (const AT*)vp->data_ptr() : nullptr,                          \
      block_tables.data_ptr<int>(), (int)block_tables.size(1), cu_q.data_ptr<int>(), ctx_lens.data_ptr<int>(), (int)B, sp, \
      (float)scale, (int)window, pooled ? (int)pool : 0, per, (OT*)out.data_ptr(), ldo, (int)H, (int)G, (int)d, (int)dv,  \
      (int)Gv)
#define WATT_REP(AT, OT)                   \
  switch (rep) {                           \
    case 8: WATT_GO(AT, OT, 8); break;     \
    case 4: WATT_GO(AT, OT, 4); break;     \
    case 2: WATT_GO(AT, OT, 2); break;     \
    default: WATT_GO(AT, OT, 1); break;    \
  }
  if (q.scalar_type() == at::kBFloat16 && o32) {
    WATT_REP(uint16_t, float)
  } else if (q.scalar_type() == at::kBFloat16) {
    WATT_REP(uint16_t, uint16_t)
  } else {
    WATT_REP(float, float)
  }
#undef WATT_REP
#undef WATT_GO
}

void ssd_prep(const at::Tensor& P, int64_t x_off, int64_t dt_off, const at::Tensor& conv_w, const at::Tensor& conv_b,
              at::Tensor& conv_state, const at::Tensor& state_slots, const at::Tensor& cu_q, const at::Tensor& A_log,
              const at::Tensor& dt_bias, int64_t H, int64_t dv, at::Tensor& xbc, at::Tensor& v, at::Tensor& decay) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0) return;
  f32c(conv_w, "conv_w");
  f32c(conv_b, "conv_b");
  f32c(conv_state, "conv_state");
  f32c(A_log, "A_log");
  f32c(dt_bias, "dt_bias");
  f32c(xbc, "xbc");
  f32c(v, "v");
  f32c(decay, "decay");
  i32c(state_slots, "state_slots");
  i32c(cu_q, "cu_q");
  MCHECK(conv_w.dim() == 2, "conv_w must be [C, taps]");
  const int64_t C = conv_w.size(0), taps = conv_w.size(1), B = state_slots.numel();
  MCHECK(taps >= 1 && conv_b.numel() == C && C >= H * dv, "ssd_prep: convolution shapes");
  MCHECK(taps == 1 || (conv_state.dim() == 3 && conv_state.size(1) == taps - 1 && conv_state.size(2) == C),
         "conv_state must be [slots, taps - 1, C]");
  MCHECK(cu_q.numel() == B + 1 && A_log.numel() == H && dt_bias.numel() == H, "ssd_prep: shape mismatch");
  MCHECK(xbc.numel() == T * C && v.numel() == T * H * dv && decay.numel() == T * H, "ssd_prep: output shape mismatch");
  cols_ok(P, x_off, C, "conv inputs");
  cols_ok(P, dt_off, H, "dt");
  // few tokens (decode steps): the channels are spread over workgroups too
  const dim3 pgrid((unsigned)T, (unsigned)(T >= 2048 ? 1 : std::min<int64_t>((C + 255) / 256, 32)));
  ssd_prep_k<<<pgrid, 256, H * sizeof(float), stream()>>>(P.data_ptr<float>(), ldp, (int)x_off, (int)dt_off, conv_w.data_ptr<float>(),
                                      conv_b.data_ptr<float>(), (int)taps, (int)C, conv_state.data_ptr<float>(),
                                      state_slots.data_ptr<int>(), cu_q.data_ptr<int>(), (int)B, A_log.data_ptr<float>(),
                                      dt_bias.data_ptr<float>(), (int)H, (int)dv, xbc.data_ptr<float>(), v.data_ptr<float>(),
                                      decay.data_ptr<float>());
  if (taps > 1) {
    const dim3 grid((unsigned)B, (unsigned)((C + 255) / 256));
    conv_tail_store_k<<<grid, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)x_off, (int)C, (int)taps,
                                                  conv_state.data_ptr<float>(), state_slots.data_ptr<int>(),
                                                  cu_q.data_ptr<int>());
  }
}

void ssd_gate_norm(const at::Tensor& o, const at::Tensor& xbc, const at::Tensor& skip_d, const at::Tensor& P, int64_t z_off,
                   const at::Tensor& w, int64_t groups, double eps, at::Tensor& out) {
  f32c(o, "o");
  f32c(xbc, "xbc");
  f32c(skip_d, "skip_d");
  f32c(w, "w");
  const int ldp = ld_of(P, "P");
  MCHECK(o.dim() == 2 && xbc.dim() == 2, "o [T, inner], xbc [T, C]");
  const int64_t T = o.size(0), inner = o.size(1), C = xbc.size(1), H = skip_d.numel();
  if (T == 0) return;
  MCHECK(P.size(0) == T && xbc.size(0) == T && C >= inner && H > 0 && inner % H == 0 && w.numel() == inner && groups >= 1 &&
             inner % groups == 0,
         "ssd_gate_norm: shape mismatch");
  cols_ok(P, z_off, inner, "gate");
  const int ldo = act_ld_min(out, T, inner, "out");
  const dim3 grid((unsigned)T, (unsigned)groups);
  if (out.scalar_type() == at::kBFloat16)
    ssd_gate_norm_k<uint16_t><<<grid, 256, 0, stream()>>>(o.data_ptr<float>(), xbc.data_ptr<float>(), (int)C,
                                                          skip_d.data_ptr<float>(), P.data_ptr<float>(), ldp, (int)z_off,
                                                          w.data_ptr<float>(), (float)eps, (uint16_t*)out.data_ptr(), ldo,
                                                          (int)inner, (int)(inner / H), (int)(inner / groups));
  else
    ssd_gate_norm_k<float><<<grid, 256, 0, stream()>>>(o.data_ptr<float>(), xbc.data_ptr<float>(), (int)C,
                                                       skip_d.data_ptr<float>(), P.data_ptr<float>(), ldp, (int)z_off,
                                                       w.data_ptr<float>(), (float)eps, out.data_ptr<float>(), ldo, (int)inner,
                                                       (int)(inner / H), (int)(inner / groups));
}

void polynorm_act(const at::Tensor& P, int64_t up_off, int64_t F, const at::Tensor& coef, double eps, at::Tensor& out) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0) return;
  f32c(coef, "coef");
  MCHECK(coef.numel() == 4 && F > 0, "PolyNorm takes four coefficients");
  cols_ok(P, up_off, F, "up");
  const int ldo = act_ld_min(out, T, F, "out");
  const int bs = F > 256 * PN_REG ? 1024 : 256;
  if (out.scalar_type() == at::kBFloat16)
    polynorm_act_k<uint16_t><<<T, bs, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)up_off, (int)F, coef.data_ptr<float>(),
                                                     (float)eps, (uint16_t*)out.data_ptr(), ldo);
  else
    polynorm_act_k<float><<<T, bs, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)up_off, (int)F, coef.data_ptr<float>(),
                                                  (float)eps, out.data_ptr<float>(), ldo);
}

void relu2(const at::Tensor& P, int64_t off, int64_t F, at::Tensor& out) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  cols_ok(P, off, F, "relu2 input");
  const int ldo = act_ld_min(out, T, F, "out");
  const int64_t total = T * F;
  if (total == 0) return;
  const int blocks = (int)((total + 255) / 256);
  if (out.scalar_type() == at::kBFloat16)
    relu2_k<uint16_t><<<blocks, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)off, (int)F, (uint16_t*)out.data_ptr(), ldo,
                                                    total);
  else
    relu2_k<float><<<blocks, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)off, (int)F, out.data_ptr<float>(), ldo, total);
}

void moe_weighted_sum(const at::Tensor& y, const at::Tensor& slot_of, const at::Tensor& topw, int64_t k,
                      const c10::optional<at::Tensor>& sh_y, const c10::optional<at::Tensor>& P, int64_t shg_off,
                      at::Tensor& out, int64_t splits) {
  const int ldy = ld_of(y, "y");
  f32c(out, "out");
  f32c(topw, "topw");
  i32c(slot_of, "slot_of");
  MCHECK(out.dim() == 2, "out must be [T, D]");
  const int64_t T = out.size(0), D = out.size(1);
  if (T == 0) return;
  MCHECK(k >= 1 && splits >= 1 && topw.numel() == T * k && slot_of.numel() == T * k && y.size(0) == splits * T * k &&
             y.size(1) >= D,
         "moe_weighted_sum: shape mismatch");
  const float *sp = nullptr, *pp = nullptr;
  int lds = 0, ldp = 0;
  if (sh_y.has_value()) {
    lds = ld_of(*sh_y, "sh_y");
    MCHECK(sh_y->size(0) == T && sh_y->size(1) >= D, "a shared expert needs its result [T, >= D]");
    sp = sh_y->data_ptr<float>();
    if (P.has_value()) {
      ldp = ld_of(*P, "P");
      MCHECK(P->size(0) == T, "P must have T rows");
      cols_ok(*P, shg_off, 1, "shared gate");
      pp = P->data_ptr<float>();
    }
  }
  // (slot_of comes from the routing kernel: every entry is a row of y)
  moe_weighted_sum_k<<<T, 256, 0, stream()>>>(y.data_ptr<float>(), ldy, slot_of.data_ptr<int>(), topw.data_ptr<float>(), (int)k,
                                              (int)splits, (int64_t)(T * k), sp, lds, pp, ldp, (int)shg_off,
                                              out.data_ptr<float>(), (int)D);
}

}  // namespace

void bind_hybrid(pybind11::module& m) {
  namespace py = pybind11;
  m.def("gated_postnorm", &gated_postnorm);
  m.def("qk_norm_rope_store", &qk_norm_rope_store);
  m.def("kv_pool_update", &kv_pool_update);
  m.def("attn_window_pool", &attn_window_pool);
  m.def("ssd_prep", &ssd_prep);
  m.def("ssd_gate_norm", &ssd_gate_norm);
  m.def("polynorm_act", &polynorm_act);
  m.def("relu2", &relu2);
  m.def("moe_weighted_sum", &moe_weighted_sum, py::arg("y"), py::arg("slot_of"), py::arg("topw"), py::arg("k"),
        py::arg("sh_y"), py::arg("P"), py::arg("shg_off"), py::arg("out"), py::arg("splits") = 1);
}

}  // namespace xot
