// Token mixers beside softmax attention, and the fp32-residual layer plumbing around them (gfx950).
//
//   resid_scale_norm   x += s1 * y1 (+ s2 * y2) on the fp32 residual stream, then RMS norm with one scalar gain
//   gelu_mul           gelu_tanh(gate) * up out of a fused projection's columns
//   rope_kv_store      partial rotate-half RoPE on q and k, paged write of the rotated key and of the value
//                      (the value may be the un-rotated key)
//   attn_gated_chunk   chunk-local attention with sigmoid(score + bias[head]) weights, no normalisation: an MFMA
//                      kernel for prompt portions (bf16), a (token, kv head, key split) kernel for single tokens
//                      and fp32, a wave per (token, head) for groups above 8 query heads
//   delta_prep         short causal convolutions + SiLU, unit-norm q / k, sigmoid write strength, scalar decay
//   conv_state_update  the last taps-1 convolution inputs of every sequence -> its state slot
//   gla_prep           per-key-channel decay sigmoid(low-rank z)^(1/tau)
//   linear_recurrence  S <- decay * S, delta-rule or outer-product write, o = S^T q; fp32 state per slot
//   gated_rmsnorm      per-head RMS norm of o, weight, SiLU gate
//
// A fused projection's output P is fp32 [T, ldp]; "column offset" arguments address its slices.  Activations that
// feed the next GEMM (AT) are bf16 or fp32; everything that enters a norm, a score or a recurrence is fp32.
#include "mixer_util.h"

namespace xot {
namespace {
using namespace mix;

// ------------------------------------------------------------------ residual + scalar-gain RMS norm
template <typename AT>
__global__ void resid_scale_norm_k(float* __restrict__ x, const float* __restrict__ y1, const float* __restrict__ s1,
                                   const float* __restrict__ y2, const float* __restrict__ s2,
                                   const float* __restrict__ gain, float eps, AT* __restrict__ out, int D, int ld1,
                                   int ld2, int ldo) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  float* xr = x + r * D;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    float v = xr[i];
    if (y1) {
      float a = s1[i] * y1[r * ld1 + i];
      if (y2) a += s2[i] * y2[r * ld2 + i];
      v += a;
      xr[i] = v;
    }
    ss += v * v;
  }
  if (!out) return;
  ss = block_sum(ss, red);
  const float k = gain[0] / sqrtf(ss / (float)D + eps);
  for (int i = threadIdx.x; i < D; i += blockDim.x) stf(out + r * ldo + i, xr[i] * k);
}

// ------------------------------------------------------------------ gelu_tanh(gate) * up
template <typename AT>
__global__ void gelu_mul_k(const float* __restrict__ P, int ldp, int gate_off, int up_off, int F, AT* __restrict__ out,
                           int ldo, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t t = idx / F;
  const int i = (int)(idx - t * F);
  const float z = P[t * ldp + gate_off + i], u = P[t * ldp + up_off + i];
  const float g = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  stf(out + t * ldo + i, g * u);
}

// ------------------------------------------------------------------ RoPE + paged key / value write
// cos_sin [rows, R]: row p = [cos(p f_0 .. f_{R/2-1}) | sin(...)].  Pair (i, i + R/2), i < R/2; dims >= R pass.
template <typename AT>
__global__ void rope_kv_store_k(const float* __restrict__ P, int ldp, int q_off, int k_off, int v_off, int H, int G, int d,
                                int R, const int* __restrict__ pos, const float* __restrict__ cos_sin,
                                const int64_t* __restrict__ slots, AT* __restrict__ q_out, AT* __restrict__ k_cache,
                                AT* __restrict__ v_cache) {
  const int t = blockIdx.x;
  const float* row = P + (int64_t)t * ldp;
  const float* cs = cos_sin + (int64_t)pos[t] * R;
  const int half = R >> 1;
  const int64_t slot = slots[t];
  const int n = (H + G) * d;
  for (int e = threadIdx.x; e < n; e += blockDim.x) {
    const int head = e / d, i = e - head * d;
    const bool isq = head < H;
    const float* x = row + (isq ? q_off + head * d : k_off + (head - H) * d);
    float v = x[i];
    const float raw = v;
    if (i < half) {
      v = x[i] * cs[i] - x[i + half] * cs[half + i];
    } else if (i < R) {
      const int j = i - half;
      v = x[i] * cs[j] + x[j] * cs[half + j];
    }
    if (isq) {
      stf(q_out + ((int64_t)t * H + head) * d + i, v);
    } else if (slot >= 0) {
      const int g = head - H;
      const int64_t pg = (slot / PAGE_TOK) * G + g;
      stf(k_cache + (pg * PAGE_TOK + (slot % PAGE_TOK)) * d + i, v);
      stf(v_cache + (pg * d + i) * PAGE_TOK + (slot % PAGE_TOK), v_off >= 0 ? row[v_off + g * d + i] : raw);
    }
  }
}

// ------------------------------------------------------------------ chunk-local gated attention
// Caches: K [pages, G, 64, d] (a key's dims contiguous), V^T [pages, G, d, 64] (a dim's 64 keys of the page
// contiguous: the PV product streams 4 / 8 consecutive keys of one dim per load).
// out[t, h * d + i] = out_scale * sum_j sigmoid(q.k_j * scale + pb[h]) v_j[i] over the keys j <= i's position of
// the query's chunk.
//
// Wave-per-(token, head) kernel (any d <= 256, bf16 or fp32; the fallback for more than 8 query heads per kv head):
// lanes over keys for the scores, then lanes over value dims for the weighted sum.
constexpr int ATT_TILE = 512;

template <typename AT>
__global__ void attn_gated_chunk_k(const AT* __restrict__ q, const AT* __restrict__ k_cache, const AT* __restrict__ v_cache,
                                   const int* __restrict__ block_tables, int width, const int* __restrict__ cu_q,
                                   const int* __restrict__ ctx_lens, int B, const float* __restrict__ pb, float scale,
                                   int chunk, float out_scale, AT* __restrict__ out, int ldo, int H, int G, int d) {
  extern __shared__ float sm[];
  float* qs = sm;            // [d]
  float* ws = sm + d;        // [ATT_TILE + 8]: weights of positions a0 .. (a0 = the tile's start rounded down to 8)
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int b = seq_of(cu_q, B, t);
  const int ctx = ctx_lens[b];
  if (ctx <= 0) return;  // padding row of a captured decode batch
  const int pos = ctx - (cu_q[b + 1] - cu_q[b]) + (t - cu_q[b]);
  const int lo = (pos / chunk) * chunk;
  const int g = h / (H / G);
  for (int i = lane; i < d; i += 64) qs[i] = ldf(q + ((int64_t)t * H + h) * d + i);
  const float bias = pb[h];
  const int* bt = block_tables + (int64_t)b * width;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};  // value dims lane, lane + 64, ... (d <= 256)
  for (int p0 = lo; p0 <= pos; p0 += ATT_TILE) {
    const int p1 = min(p0 + ATT_TILE, pos + 1);  // keys [p0, p1)
    const int a0 = p0 & ~7, a1 = (p1 + 7) & ~7;  // 8-aligned cover; positions outside [p0, p1) weigh 0
    __syncthreads();
    for (int p = a0 + lane; p < a1; p += 64) {
      float w = 0.0f;
      if (p >= p0 && p < p1) {
        const AT* kr = k_cache + (((int64_t)bt[p / PAGE_TOK] * G + g) * PAGE_TOK + (p % PAGE_TOK)) * d;
        float s = 0.0f;
        if (d & 7) {
          for (int i = 0; i < d; ++i) s += qs[i] * ldf(kr + i);
        } else {
          for (int i = 0; i < d; i += 8) {
            float kv[8];
            ld8(kr + i, kv);
#pragma unroll
            for (int e = 0; e < 8; ++e) s += qs[i + e] * kv[e];
          }
        }
        w = sigmoidf_(s * scale + bias);
      }
      ws[p - a0] = w;
    }
    __syncthreads();
    for (int p = a0; p < a1; p += 8) {  // 8 keys of one page per step
      const AT* vp = v_cache + ((int64_t)bt[p / PAGE_TOK] * G + g) * d * PAGE_TOK + (p % PAGE_TOK);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int i = lane + 64 * c;
        if (i < d) {
          float vv[8];
          ld8(vp + (int64_t)i * PAGE_TOK, vv);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float w = ws[p - a0 + e];
            acc[c] += w != 0.0f ? w * vv[e] : 0.0f;  // (a slot no token has written yet may hold anything)
          }
        }
      }
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int i = lane + 64 * c;
    if (i < d) stf(out + (int64_t)t * ldo + h * d + i, acc[c] * out_scale);
  }
}

// Single tokens and fp32 steps, query heads sharing a kv head (at most 8): workgroup = (token, kv head, key split).
// Scores: a thread per key loads its K row once and scores it against every query head of the group.  Sum: threads
// = value dims x key slices, 8 keys per 16-byte V^T load, one accumulator per query head; slices are reduced through
// LDS.  With key splits each workgroup writes an fp32 partial and attn_split_sum_k adds them in a fixed order.
constexpr int ATG_TILE = 256;
constexpr int ATG_HEADS = 8;

template <typename AT>
__global__ __launch_bounds__(256) void attn_gated_chunk_gqa_k(
    const AT* __restrict__ q, const AT* __restrict__ k_cache, const AT* __restrict__ v_cache,
    const int* __restrict__ block_tables, int width, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, int B,
    const float* __restrict__ pb, float scale, int chunk, float out_scale, AT* __restrict__ out, int ldo,
    float* __restrict__ part, int T, int H, int G, int d, int dpad, int KS) {
  extern __shared__ float sm[];
  const int hpg = H / G;
  float* qs = sm;                               // [hpg][d]
  float* ws = qs + hpg * d;                     // [hpg][ATG_TILE + 8]
  float* red = ws + hpg * (ATG_TILE + 8);       // [slices][hpg][dpad]
  const int t = blockIdx.x, g = blockIdx.y, ks = blockIdx.z, tid = threadIdx.x;
  const int b = seq_of(cu_q, B, t);
  const int ctx = ctx_lens[b];
  if (ctx <= 0) return;  // padding row of a captured decode batch
  const int pos = ctx - (cu_q[b + 1] - cu_q[b]) + (t - cu_q[b]);
  const int lo = (pos / chunk) * chunk;
  // this split's keys [k0, k1): equal 8-aligned shares of [lo, pos]
  const int share = (((pos - lo + 1) + KS - 1) / KS + 7) & ~7;
  const int k0 = lo + ks * share, k1 = min(k0 + share, pos + 1);
  for (int e = tid; e < hpg * d; e += 256) qs[e] = ldf(q + ((int64_t)t * H + g * hpg) * d + e);
  const int nsl = 256 / dpad, di = tid % dpad, sl = tid / dpad;
  const int* bt = block_tables + (int64_t)b * width;
  float acc[ATG_HEADS];
#pragma unroll
  for (int hq = 0; hq < ATG_HEADS; ++hq) acc[hq] = 0.0f;
  for (int p0 = k0; p0 < k1; p0 += ATG_TILE) {
    const int p1 = min(p0 + ATG_TILE, k1);
    const int a0 = p0 & ~7, a1 = (p1 + 7) & ~7;  // 8-aligned cover (<= ATG_TILE + 8 keys); outside [p0, p1) weighs 0
    __syncthreads();
    for (int p = a0 + tid; p < a1; p += 256) {
      float sc[ATG_HEADS];
#pragma unroll
      for (int hq = 0; hq < ATG_HEADS; ++hq) sc[hq] = 0.0f;
      const bool in = p >= p0 && p < p1;
      if (in) {
        const AT* kr = k_cache + (((int64_t)bt[p / PAGE_TOK] * G + g) * PAGE_TOK + (p % PAGE_TOK)) * d;
        if (d & 7) {
          for (int i = 0; i < d; ++i) {
            const float kv = ldf(kr + i);
#pragma unroll
            for (int hq = 0; hq < ATG_HEADS; ++hq)
              if (hq < hpg) sc[hq] += qs[hq * d + i] * kv;
          }
        } else {
          for (int i = 0; i < d; i += 8) {
            float kv[8];
            ld8(kr + i, kv);
#pragma unroll
            for (int hq = 0; hq < ATG_HEADS; ++hq)
              if (hq < hpg) {
#pragma unroll
                for (int e = 0; e < 8; ++e) sc[hq] += qs[hq * d + i + e] * kv[e];
              }
          }
        }
      }
#pragma unroll
      for (int hq = 0; hq < ATG_HEADS; ++hq)
        if (hq < hpg) ws[hq * (ATG_TILE + 8) + p - a0] = in ? sigmoidf_(sc[hq] * scale + pb[g * hpg + hq]) : 0.0f;
    }
    __syncthreads();
    if (di < d) {
      for (int p = a0 + 8 * sl; p < a1; p += 8 * nsl) {  // 8 keys of one page per step
        float vv[8];
        ld8(v_cache + (((int64_t)bt[p / PAGE_TOK] * G + g) * d + di) * PAGE_TOK + (p % PAGE_TOK), vv);
#pragma unroll
        for (int hq = 0; hq < ATG_HEADS; ++hq)
          if (hq < hpg) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float w = ws[hq * (ATG_TILE + 8) + p - a0 + e];
              acc[hq] += w != 0.0f ? w * vv[e] : 0.0f;  // (a slot no token has written yet may hold anything)
            }
          }
      }
    }
  }
#pragma unroll
  for (int hq = 0; hq < ATG_HEADS; ++hq)
    if (hq < hpg) red[(sl * hpg + hq) * dpad + di] = acc[hq];
  __syncthreads();
  for (int e = tid; e < hpg * d; e += 256) {
    const int hq = e / d, i = e - hq * d;
    float o = 0.0f;
    for (int s2 = 0; s2 < nsl; ++s2) o += red[(s2 * hpg + hq) * dpad + i];
    if (KS == 1)
      stf(out + (int64_t)t * ldo + (g * hpg + hq) * d + i, o * out_scale);
    else
      part[((int64_t)ks * T + t) * H * d + (g * hpg + hq) * d + i] = o;
  }
}

template <typename AT>
__global__ void attn_split_sum_k(const float* __restrict__ part, int KS, int T, int HD, float out_scale, AT* __restrict__ out,
                                 int ldo, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, int B) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)T * HD) return;
  const int t = (int)(idx / HD), i = (int)(idx - (int64_t)t * HD);
  if (ctx_lens[seq_of(cu_q, B, t)] <= 0) return;  // padding row: no partials were written
  float o = 0.0f;
  for (int ks = 0; ks < KS; ++ks) o += part[((int64_t)ks * T + t) * HD + i];
  stf(out + (int64_t)t * ldo + i, o * out_scale);
}

// MFMA kernel (bf16, d = 32 NK): a workgroup owns 128 consecutive queries of one (sequence, head), 32 per wave, and
// walks the keys of their chunk(s) a tile of KT keys at a time: the K rows and V^T runs of the tile are staged in LDS
// with whole-line loads and shared by the four waves.  Scores are computed transposed, S^T = K Q^T (keys x queries),
// so a lane's four accumulator rows are four consecutive keys of ONE query: after the sigmoid they are, as they lie,
// the B operand of O^T += V^T P^T, whose k slots (g, j) are read as keys {4g .. 4g+3, 16+4g .. 16+4g+3} on both
// operands.  LDS rows are padded by 16 B so the fragment reads of 16 rows hit distinct banks.
template <int NK>
__global__ __launch_bounds__(256) void attn_gated_chunk_mfma_k(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    const int* __restrict__ block_tables, int width, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    const float* __restrict__ pb, float scale, int chunk, float out_scale, uint16_t* __restrict__ out, int ldo, int H, int G) {
  constexpr int D = NK * 32, ND = NK * 2, QT = 2;
  constexpr int KT = D > 192 ? 32 : 64;  // keys per tile (a page holds a whole number of tiles)
  constexpr int KP = D + 8, VP = KT + 8;
  __shared__ __attribute__((aligned(16))) uint16_t sK[KT][KP], sV[D][VP];
  const int b = blockIdx.x, h = blockIdx.z;
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, c = l & 15, g4 = l >> 4;
  const int t0 = cu_q[b], qlen = cu_q[b + 1] - t0, ctx = ctx_lens[b];
  const int wq0 = blockIdx.y * 128;
  if (ctx <= 0 || wq0 >= qlen) return;
  const int q0 = wq0 + wave * 32;
  const bool active = q0 < qlen;
  const int nq = active ? min(32, qlen - q0) : 0;
  const int pos0 = ctx - qlen + q0;  // position of the wave's first query
  const int gk = h / (H / G);
  const float bias = pb[h];
  s16x8 qf[QT][NK];
  int qpos[QT], qcs[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int local = qt * 16 + c;
    const bool ok = local < nq;
    qpos[qt] = pos0 + local;
    qcs[qt] = (qpos[qt] / chunk) * chunk;
    const uint16_t* qp = q + ((int64_t)(t0 + q0 + local) * H + h) * D + 8 * g4;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) qf[qt][ks] = ok ? ld16(qp + ks * 32) : s16x8{0, 0, 0, 0, 0, 0, 0, 0};
  }
  f32x4 o[QT][ND];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt)
#pragma unroll
    for (int db = 0; db < ND; ++db) o[qt][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  // the wave's keys [k_lo, k_hi]; the workgroup's tiles cover the union over its waves
  const int k_lo = active ? (pos0 / chunk) * chunk : 0x7fffffff, k_hi = active ? pos0 + nq - 1 : -1;
  const int cs_last = active ? (k_hi / chunk) * chunk : 0;  // a block at or after it and wholly before pos0 needs no mask
  const int wpos0 = ctx - qlen + wq0;
  const int t_lo = ((wpos0 / chunk) * chunk) & ~(KT - 1), t_hi = wpos0 + min(128, qlen - wq0) - 1;
  const int* bt = block_tables + (int64_t)b * width;
  // sigmoid(s scale + bias) = 1 / (1 + 2^(s ea + eb))
  const float ea = -scale * 1.4426950408889634f, eb = -bias * 1.4426950408889634f;
  // a thread's share of a tile: NCH 16-byte chunks of K and of V^T, fetched one tile ahead into registers
  constexpr int NCHUNK = KT * (D / 8), NCH = (NCHUNK + 255) / 256;
  s16x8 rk[NCH], rv[NCH];
  auto fetch = [&](int tb) {
    const int64_t pg = (int64_t)bt[tb >> 6] * G + gk;
    const int koff = tb & 63;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int ch = threadIdx.x + 256 * j;
      if (NCHUNK % 256 != 0 && ch >= NCHUNK) break;
      const int row = ch / (D / 8), cc = ch - row * (D / 8);
      rk[j] = ld16(k_cache + ((pg * PAGE_TOK) + koff + row) * D + cc * 8);
      const int vrow = ch / (KT / 8), vc = ch - vrow * (KT / 8);
      rv[j] = ld16(v_cache + (pg * D + vrow) * PAGE_TOK + koff + vc * 8);
    }
  };
  fetch(t_lo);
  for (int tb = t_lo; tb <= t_hi; tb += KT) {
    __syncthreads();  // the previous tile has been consumed
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int ch = threadIdx.x + 256 * j;
      if (NCHUNK % 256 != 0 && ch >= NCHUNK) break;
      const int row = ch / (D / 8), cc = ch - row * (D / 8);
      st16(&sK[row][cc * 8], rk[j]);
      const int vrow = ch / (KT / 8), vc = ch - vrow * (KT / 8);
      st16(&sV[vrow][vc * 8], rv[j]);
    }
    __syncthreads();
    if (tb + KT <= t_hi) fetch(tb + KT);  // in flight while this tile is consumed
#pragma unroll
    for (int sub = 0; sub < KT / 32; ++sub) {
      const int kb = tb + sub * 32;
      if (kb > k_hi || kb + 31 < k_lo) continue;  // (wave-uniform) none of these keys is visible to this wave
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
      const bool full = kb + 31 <= pos0 && kb >= cs_last;  // every key of the block is visible to every query
      s16x8 pf[QT];
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        u32x4 packed;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r2 = 0; r2 < 2; ++r2) {
            float pr[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const int r = 2 * r2 + e;
              float p = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(s[kt][qt][r] * ea + eb));
              if (!full) {
                const int kpos = kb + kt * 16 + 4 * g4 + r;
                p = (kpos <= qpos[qt] && kpos >= qcs[qt]) ? p : 0.0f;
              }
              pr[e] = p;
            }
            // two bf16 (rounded half up: the weights are positive and finite) in one dword
            packed[kt * 2 + r2] = __builtin_amdgcn_perm(__float_as_uint(pr[1]) + 0x8000u, __float_as_uint(pr[0]) + 0x8000u,
                                                        0x07060302u);
          }
        pf[qt] = __builtin_bit_cast(s16x8, packed);
      }
      // (slots of the page no token has written yet hold zeros or an earlier request's finite values; their weight is 0)
#pragma unroll
      for (int db = 0; db < ND; ++db) {
        const s16x4 v0 = *reinterpret_cast<const s16x4*>(&sV[db * 16 + c][sub * 32 + 4 * g4]);
        const s16x4 v1 = *reinterpret_cast<const s16x4*>(&sV[db * 16 + c][sub * 32 + 16 + 4 * g4]);
        const s16x8 a = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) o[qt][db] = mfma16(a, pf[qt], o[qt][db]);
      }
    }
  }
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    if (qt * 16 + c >= nq) continue;
    uint16_t* op = out + (int64_t)(t0 + q0 + qt * 16 + c) * ldo + h * D + 4 * g4;
#pragma unroll
    for (int db = 0; db < ND; ++db) {
      s16x4 w;
#pragma unroll
      for (int r = 0; r < 4; ++r) w[r] = (short)f2bf(o[qt][db][r] * out_scale);
      *reinterpret_cast<s16x4*>(op + db * 16) = w;
    }
  }
}

// ------------------------------------------------------------------ delta-rule inputs
// Channels [q: G d | k: G d | v: H dv] at P[:, x_off ...]; conv_w [C, taps] (last column: the current token);
// conv_state [slots, taps - 1, C] holds the inputs before this step (zeros for a new sequence).
// qkv [T, C]: q = unit(silu(conv q)) * d^-1/2, k = unit(silu(conv k)), v = silu(conv v);
// beta [T, H] = sigmoid(P[b_off + h]); decay [T, H] = exp(-exp(A_log[h]) softplus(P[a_off + h] + dt_bias[h])).
__global__ void delta_prep_k(const float* __restrict__ P, int ldp, int x_off, int b_off, int a_off,
                             const float* __restrict__ conv_w, int taps, const float* __restrict__ conv_state,
                             const int* __restrict__ state_slots, const int* __restrict__ cu_q, int B,
                             const float* __restrict__ A_log, const float* __restrict__ dt_bias, int H, int G, int d, int dv,
                             float* __restrict__ qkv, float* __restrict__ beta, float* __restrict__ decay, int T, int tpb) {
  // workgroup = (tpb <= 8 consecutive tokens, unit): units 0 .. G-1 the q heads, G .. 2G-1 the k heads, then H value
  // heads, then the gates.  A thread owns one channel of the unit for all the tokens: their convolution inputs are
  // loaded together and the tokens' sums of squares are reduced in one pass.  tpb is 1 for decode steps.
  constexpr int TPB = 8;
  __shared__ float red[TPB][4];
  const int unit = blockIdx.y;
  const int C = 2 * G * d + H * dv;
  const int tbase = blockIdx.x * tpb;
  if (unit == 2 * G + H) {
    for (int e = threadIdx.x; e < tpb * H; e += blockDim.x) {
      const int t = tbase + e / H, h = e % H;
      if (t >= T || state_slots[seq_of(cu_q, B, t)] < 0) continue;
      const float* row = P + (int64_t)t * ldp;
      beta[(int64_t)t * H + h] = sigmoidf_(row[b_off + h]);
      decay[(int64_t)t * H + h] = expf(-expf(A_log[h]) * softplusf_(row[a_off + h] + dt_bias[h]));
    }
    return;
  }
  const bool qk = unit < 2 * G;
  const int c0 = qk ? unit * d : 2 * G * d + (unit - 2 * G) * dv, n = qk ? d : dv;
  const int i = threadIdx.x;  // the launch gives a thread per channel of the widest unit (n <= blockDim.x <= 256)
  const int c = c0 + i;
  float y[TPB];
  bool ok[TPB];
#pragma unroll
  for (int tt = 0; tt < TPB; ++tt) {
    const int t = tbase + tt;
    y[tt] = 0.0f;
    ok[tt] = false;
    if (tt >= tpb || t >= T) continue;
    const int b = seq_of(cu_q, B, t);
    const int slot = state_slots[b];
    if (slot < 0) continue;
    ok[tt] = true;
    if (i >= n) continue;
    const int local = t - cu_q[b], tstart = cu_q[b];
    const float* st = conv_state + (int64_t)slot * (taps - 1) * C;
    float acc = 0.0f;
    for (int j = 0; j < taps; ++j) {
      const int sidx = local - (taps - 1 - j);
      const float x = sidx >= 0 ? P[(int64_t)(tstart + sidx) * ldp + x_off + c] : st[(int64_t)(taps - 1 + sidx) * C + c];
      acc += conv_w[c * taps + j] * x;
    }
    y[tt] = siluf_(acc);
  }
  if (qk) {
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
#pragma unroll
    for (int tt = 0; tt < TPB; ++tt) {
      const float ss = wave_sum(y[tt] * y[tt]);
      if ((threadIdx.x & 63) == 0) red[tt][wave] = ss;
    }
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < TPB; ++tt) {
      float ss = 0.0f;
      for (int w = 0; w < nw; ++w) ss += red[tt][w];
      float kn = 1.0f / sqrtf(ss + 1e-6f);
      if (unit < G) kn *= 1.0f / sqrtf((float)d);
      y[tt] *= kn;
    }
  }
  if (i < n) {
#pragma unroll
    for (int tt = 0; tt < TPB; ++tt)
      if (ok[tt]) qkv[(int64_t)(tbase + tt) * C + c] = y[tt];
  }
}

__global__ void conv_state_update_k(const float* __restrict__ P, int ldp, int x_off, int C, int taps,
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

// ------------------------------------------------------------------ GLA decay
// decay [T, HD] = exp(logsigmoid(z) / tau), z[c] = a2_b[c] + sum_r a2[c, r] P[t, a1_off + r]
__global__ void gla_prep_k(const float* __restrict__ P, int ldp, int a1_off, int rank, const float* __restrict__ a2,
                           const float* __restrict__ a2_b, float inv_tau, int HD, float* __restrict__ decay) {
  extern __shared__ float ys[];  // [rank]
  const int t = blockIdx.x;
  for (int r = threadIdx.x; r < rank; r += blockDim.x) ys[r] = P[(int64_t)t * ldp + a1_off + r];
  __syncthreads();
  for (int c = threadIdx.x; c < HD; c += blockDim.x) {
    float z = 0.0f;
    for (int r = 0; r < rank; ++r) z += a2[(int64_t)c * rank + r] * ys[r];
    z += a2_b[c];
    decay[(int64_t)t * HD + c] = expf(logsigmoidf_(z) * inv_tau);
  }
}

// ------------------------------------------------------------------ the recurrence
// State in memory: S^T [slots, H, dv, d] (a value channel's d key rows contiguous).
// Workgroup = (sequence, value head, 256 / RS value channels); 256 threads = channels x RS row groups, the row group
// in the low lane bits: the two dot products reduce inside DPP rows, register to register.  A thread keeps the KR
// consecutive key rows rg KR .. rg KR + KR - 1 of its channel in registers (d <= RS KR), so state loads and stores are
// contiguous runs and a token's k / q slices are vector LDS reads.  The launcher uses RS = 16 (a whole DPP row per
// value channel).  Tokens are staged through LDS TB at a time, double-buffered: the next block's global loads are in flight
// while the current one is consumed.
// MODE 1 (delta rule): S *= g; u = beta (v - S^T k); S += k u^T; o = S^T q.   MODE 0: S = diag(a) S + k v^T; o = S^T q
// (a decay per key channel).   MODE 2: S = g S + k v^T; o = S^T q (one decay per head: the state-space-duality form
// with k = B, q = C, v = dt x).   MODE 3: MODE 2 with an input scale b per head and token and a normaliser: the state has
// one value channel more than v (dvin + 1), fed with ones, S = g S + k (b [v | 1])^T, so the last channel is n = g n + b k
// and the last output n . q (the stabilised matrix memory of xLSTM, g and b computed by its gate kernel).
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int m = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
  return v + __int_as_float(m);
}
// sum over RS adjacent lanes, result in each of them: lanes ^1 and ^2 by quad permutes, then (RS 16) the mirrored
// half row and the mirrored row, whose lanes already hold equal quad / half-row sums
template <int RS>
__device__ __forceinline__ float group_sum(float v) {
  v = dpp_add<0xB1>(v);  // quad_perm [1, 0, 3, 2]
  v = dpp_add<0x4E>(v);  // quad_perm [2, 3, 0, 1]
  if (RS >= 8) v = dpp_add<0x141>(v);   // row_half_mirror
  if (RS == 16) v = dpp_add<0x140>(v);  // row_mirror
  return v;
}

template <int KR, int RS, int MODE>
__global__ __launch_bounds__(256) void linear_recurrence_k(
    const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk, const float* __restrict__ v, int ldv,
    const float* __restrict__ decay, const float* __restrict__ beta, float q_scale, float* __restrict__ state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_q, int H, int G, int d, int dv, int dvin, int dstride,
    float* __restrict__ out) {
  constexpr int DP = KR * RS;  // padded key dim
  constexpr bool DELTA = MODE == 1, SCALAR = MODE != 0, NORMCH = MODE == 3;
  constexpr int COLS = 256 / RS;
  constexpr int TB = DP >= 256 ? 8 : 16;
  constexpr int NQ = TB * DP / 256, NV = (TB * COLS + 255) / 256;
  __shared__ __attribute__((aligned(16))) float sq[2][TB][DP], sk[2][TB][DP], sa[2][TB][SCALAR ? 4 : DP];
  __shared__ float sv[2][TB][COLS], sg[2][TB][2];
  const int b = blockIdx.x, h = blockIdx.y, cb = blockIdx.z;
  const int slot = state_slots[b];
  const int t0 = cu_q[b], n = cu_q[b + 1] - t0;
  if (slot < 0 || n <= 0) return;
  const int tid = threadIdx.x, rg = tid % RS, cl = tid / RS, col = cb * COLS + cl;
  const bool live = col < dv;
  const int hk = h / (H / G);
  float* S = state + (((int64_t)slot * H + h) * dv + (live ? col : 0)) * d + rg * KR;
  float s[KR];
  // 16-byte state loads / stores where the thread's rows are whole float4s inside d (d and KR multiples of 4)
  const bool vec = KR % 4 == 0 && (d & 3) == 0;
#pragma unroll
  for (int m = 0; m < KR; m += (KR % 4 == 0 ? 4 : 1)) {
    if (KR % 4 == 0 && vec) {
      const bool in = live && rg * KR + m + 4 <= d;
      const f32x4 x = in ? *reinterpret_cast<const f32x4*>(S + m) : f32x4{0.f, 0.f, 0.f, 0.f};
      s[m] = x[0];
      s[m + 1] = x[1];
      s[m + 2] = x[2];
      s[m + 3] = x[3];
    } else {
#pragma unroll
      for (int e = 0; e < (KR % 4 == 0 ? 4 : 1); ++e) s[m + e] = (live && rg * KR + m + e < d) ? S[m + e] : 0.0f;
    }
  }

  float pq[NQ], pk[NQ], pa[SCALAR ? 1 : NQ], pv[NV], pg0 = 0.0f, pg1 = 0.0f;
  auto fetch = [&](int tb) {  // global -> registers: tokens tb .. tb + TB - 1 of the sequence (zeros past its end)
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      const int e = tid + 256 * j, tt = e / DP, i = e - tt * DP;
      const int64_t t = t0 + tb + tt;
      const bool in = i < d && tb + tt < n;
      pq[j] = in ? q[t * ldq + hk * d + i] * q_scale : 0.0f;
      pk[j] = in ? k[t * ldk + hk * d + i] : 0.0f;
      if (!SCALAR) pa[j] = in ? decay[(t * H + h) * d + i] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = tid + 256 * j, tt = e / COLS, c = cb * COLS + e % COLS;
      pv[j] = (e < TB * COLS && c < dvin && tb + tt < n) ? v[(int64_t)(t0 + tb + tt) * ldv + h * dvin + c] : 0.0f;
      if (NORMCH && e < TB * COLS && c == dvin && tb + tt < n) pv[j] = 1.0f;
    }
    if (SCALAR && tid < TB && tb + tid < n) {
      pg0 = decay[(int64_t)(t0 + tb + tid) * dstride + h];  // (dstride 0: one fixed decay per head, decay [H])
      if (DELTA || NORMCH) pg1 = beta[(int64_t)(t0 + tb + tid) * H + h];
    }
  };
  auto stage = [&](int buf) {  // registers -> LDS
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      const int e = tid + 256 * j, tt = e / DP, i = e - tt * DP;
      sq[buf][tt][i] = pq[j];
      sk[buf][tt][i] = pk[j];
      if (!SCALAR) sa[buf][tt][i] = pa[j];
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = tid + 256 * j;
      if (e < TB * COLS) sv[buf][e / COLS][e % COLS] = pv[j];
    }
    if (SCALAR && tid < TB) {
      sg[buf][tid][0] = pg0;
      sg[buf][tid][1] = pg1;
    }
  };
  fetch(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int tb = 0; tb < n; tb += TB, buf ^= 1) {
    const int nt = min(TB, n - tb);
    const bool more = tb + TB < n;
    if (more) fetch(tb + TB);
#pragma unroll 2
    for (int tt = 0; tt < nt; ++tt) {
      const float vc = NORMCH ? sv[buf][tt][cl] * sg[buf][tt][1] : sv[buf][tt][cl];
      float kk[KR], qq[KR];
#pragma unroll
      for (int m = 0; m < KR; ++m) {
        kk[m] = sk[buf][tt][rg * KR + m];
        qq[m] = sq[buf][tt][rg * KR + m];
      }
      float o0 = 0.0f, o1 = 0.0f, o2 = 0.0f, o3 = 0.0f;
      if (DELTA) {
        const float g = sg[buf][tt][0], bt = sg[buf][tt][1];
        float d0 = 0.0f, d1 = 0.0f, d2 = 0.0f, d3 = 0.0f;
#pragma unroll
        for (int m = 0; m < KR; ++m) {
          s[m] *= g;
          const float p = s[m] * kk[m];
          if ((m & 3) == 0) d0 += p; else if ((m & 3) == 1) d1 += p; else if ((m & 3) == 2) d2 += p; else d3 += p;
        }
        const float u = bt * (vc - group_sum<RS>((d0 + d1) + (d2 + d3)));
#pragma unroll
        for (int m = 0; m < KR; ++m) {
          s[m] += kk[m] * u;
          const float p = s[m] * qq[m];
          if ((m & 3) == 0) o0 += p; else if ((m & 3) == 1) o1 += p; else if ((m & 3) == 2) o2 += p; else o3 += p;
        }
      } else if (SCALAR) {
        const float g = sg[buf][tt][0];
#pragma unroll
        for (int m = 0; m < KR; ++m) {
          s[m] = g * s[m] + kk[m] * vc;
          const float p = s[m] * qq[m];
          if ((m & 3) == 0) o0 += p; else if ((m & 3) == 1) o1 += p; else if ((m & 3) == 2) o2 += p; else o3 += p;
        }
      } else {
#pragma unroll
        for (int m = 0; m < KR; ++m) {
          s[m] = sa[buf][tt][rg * KR + m] * s[m] + kk[m] * vc;
          const float p = s[m] * qq[m];
          if ((m & 3) == 0) o0 += p; else if ((m & 3) == 1) o1 += p; else if ((m & 3) == 2) o2 += p; else o3 += p;
        }
      }
      const float o = group_sum<RS>((o0 + o1) + (o2 + o3));
      if (live && rg == 0) out[(int64_t)(t0 + tb + tt) * H * dv + h * dv + col] = o;
    }
    if (more) stage(buf ^ 1);  // (its last readers passed the barrier that ended the previous block)
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int m = 0; m < KR; m += (KR % 4 == 0 ? 4 : 1)) {
      if (KR % 4 == 0 && vec) {
        if (rg * KR + m + 4 <= d) *reinterpret_cast<f32x4*>(S + m) = f32x4{s[m], s[m + 1], s[m + 2], s[m + 3]};
      } else {
#pragma unroll
        for (int e = 0; e < (KR % 4 == 0 ? 4 : 1); ++e)
          if (rg * KR + m + e < d) S[m + e] = s[m + e];
      }
    }
  }
}

// ------------------------------------------------------------------ per-head RMS norm * weight * silu(gate)
template <typename AT>
__global__ void gated_rmsnorm_k(const float* __restrict__ o, const float* __restrict__ w, const float* __restrict__ P, int ldp,
                                int g_off, float eps, float out_scale, AT* __restrict__ out, int ldo, int H, int dv) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* x = o + ((int64_t)t * H + h) * dv;
  float ss = 0.0f;
  for (int i = lane; i < dv; i += 64) ss += x[i] * x[i];
  ss = wave_sum(ss);
  const float k = out_scale / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += 64) {
    const float gate = P[(int64_t)t * ldp + g_off + h * dv + i];
    stf(out + (int64_t)t * ldo + h * dv + i, x[i] * k * w[i] * siluf_(gate));
  }
}

// ------------------------------------------------------------------ host side
void resid_scale_norm(at::Tensor& x, const c10::optional<at::Tensor>& y1, const c10::optional<at::Tensor>& s1,
                      const c10::optional<at::Tensor>& y2, const c10::optional<at::Tensor>& s2,
                      const c10::optional<at::Tensor>& gain, double eps, const c10::optional<at::Tensor>& out) {
  f32c(x, "x");
  MCHECK(x.dim() == 2, "x must be [T, D]");
  const int64_t T = x.size(0), D = x.size(1);
  if (T == 0) return;
  auto chk = [&](const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& s) {
    if (!y.has_value()) return;
    MCHECK(ld_of(*y, "y") >= D && y->size(0) == T && y->size(1) >= D, "residual branch must be fp32 [T, >= D] rows");
    MCHECK(s.has_value(), "a residual branch needs its scale");
    f32c(*s, "scale");
    MCHECK(s->numel() == D, "residual branch scale must hold D numbers");
  };
  chk(y1, s1);
  chk(y2, s2);
  MCHECK(y1.has_value() || !y2.has_value(), "y2 without y1");
  if (out.has_value()) {
    MCHECK(gain.has_value(), "a normed output needs the gain");
    f32c(*gain, "gain");
    MCHECK(gain->numel() == 1, "gain must hold one number");
    MCHECK(out->is_cuda() && is_act(*out) && out->dim() == 2 && out->size(0) == T && out->size(1) >= D && out->stride(1) == 1,
           "out must be [T, >= D] rows");
  }
  const int ld1 = y1.has_value() ? (int)y1->stride(0) : 0, ld2 = y2.has_value() ? (int)y2->stride(0) : 0;
  const int ldo = out.has_value() ? (int)out->stride(0) : 0;
  const float* p1 = y1.has_value() ? y1->data_ptr<float>() : nullptr;
  const float* q1 = y1.has_value() ? s1->data_ptr<float>() : nullptr;
  const float* p2 = y2.has_value() ? y2->data_ptr<float>() : nullptr;
  const float* q2 = y2.has_value() ? s2->data_ptr<float>() : nullptr;
  const float* g = out.has_value() ? gain->data_ptr<float>() : nullptr;
  if (out.has_value() && out->scalar_type() == at::kBFloat16)
    resid_scale_norm_k<uint16_t><<<T, 256, 0, stream()>>>(x.data_ptr<float>(), p1, q1, p2, q2, g, (float)eps,
                                                          (uint16_t*)out->data_ptr(), (int)D, ld1, ld2, ldo);
  else
    resid_scale_norm_k<float><<<T, 256, 0, stream()>>>(x.data_ptr<float>(), p1, q1, p2, q2, g, (float)eps,
                                                       out.has_value() ? out->data_ptr<float>() : nullptr, (int)D, ld1, ld2, ldo);
}

void gelu_mul(const at::Tensor& P, int64_t gate_off, int64_t up_off, int64_t F, at::Tensor& out) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  MCHECK(out.is_cuda() && is_act(out) && out.dim() == 2 && out.size(0) == T && out.size(1) >= F && out.stride(1) == 1,
         "out must be [T, >= F] rows");
  const int ldo = (int)out.stride(0);
  cols_ok(P, gate_off, F, "gate");
  cols_ok(P, up_off, F, "up");
  const int64_t total = T * F;
  if (total == 0) return;
  const int blocks = (int)((total + 255) / 256);
  if (out.scalar_type() == at::kBFloat16)
    gelu_mul_k<uint16_t><<<blocks, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)gate_off, (int)up_off, (int)F,
                                                       (uint16_t*)out.data_ptr(), ldo, total);
  else
    gelu_mul_k<float><<<blocks, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)gate_off, (int)up_off, (int)F,
                                                    out.data_ptr<float>(), ldo, total);
}

void rope_kv_store(const at::Tensor& P, int64_t q_off, int64_t k_off, int64_t v_off, int64_t H, int64_t G, int64_t d,
                   int64_t R, const at::Tensor& pos, const at::Tensor& cos_sin, const at::Tensor& slots, at::Tensor& q_out,
                   at::Tensor& k_cache, at::Tensor& v_cache) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0) return;
  i32c(pos, "pos");
  f32c(cos_sin, "cos_sin");
  MCHECK(slots.is_cuda() && slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.numel() == T && pos.numel() == T,
         "pos / slots must hold one entry per token");
  MCHECK(R % 2 == 0 && R >= 0 && R <= d && (R == 0 || (cos_sin.dim() == 2 && cos_sin.size(1) == R)), "bad rotary dims");
  cols_ok(P, q_off, H * d, "q");
  cols_ok(P, k_off, G * d, "k");
  if (v_off >= 0) cols_ok(P, v_off, G * d, "v");
  MCHECK(q_out.is_cuda() && is_act(q_out) && q_out.is_contiguous() && q_out.numel() == T * H * d, "q_out must be [T, H, d]");
  MCHECK(k_cache.is_cuda() && k_cache.scalar_type() == q_out.scalar_type() && k_cache.is_contiguous() && k_cache.dim() == 4 &&
             k_cache.size(1) == G && k_cache.size(2) == PAGE_TOK && k_cache.size(3) == d,
         "k_cache must be [pages, G, 64, d] of q_out's dtype");
  MCHECK(v_cache.is_cuda() && v_cache.scalar_type() == q_out.scalar_type() && v_cache.is_contiguous() && v_cache.dim() == 4 &&
             v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G && v_cache.size(2) == d && v_cache.size(3) == PAGE_TOK,
         "v_cache must be [pages, G, d, 64] of q_out's dtype");
  // positions and slots are checked on the host by their producer (the block manager hands out slots < pages * 64
  // and the runner bounds positions by the table's rows)
  if (q_out.scalar_type() == at::kBFloat16)
    rope_kv_store_k<uint16_t><<<T, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)q_off, (int)k_off, (int)v_off, (int)H,
                                                       (int)G, (int)d, (int)R, pos.data_ptr<int>(), cos_sin.data_ptr<float>(),
                                                       slots.data_ptr<int64_t>(), (uint16_t*)q_out.data_ptr(),
                                                       (uint16_t*)k_cache.data_ptr(), (uint16_t*)v_cache.data_ptr());
  else
    rope_kv_store_k<float><<<T, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)q_off, (int)k_off, (int)v_off, (int)H, (int)G,
                                                    (int)d, (int)R, pos.data_ptr<int>(), cos_sin.data_ptr<float>(),
                                                    slots.data_ptr<int64_t>(), q_out.data_ptr<float>(),
                                                    k_cache.data_ptr<float>(), v_cache.data_ptr<float>());
}

template <int NK>
void launch_attn_mfma(dim3 grid, const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                      const at::Tensor& block_tables, const at::Tensor& cu_q, const at::Tensor& ctx_lens, const at::Tensor& pb,
                      float scale, int chunk, float out_scale, at::Tensor& out, int ldo, int H, int G) {
  attn_gated_chunk_mfma_k<NK><<<grid, 256, 0, stream()>>>(
      (const uint16_t*)q.data_ptr(), (const uint16_t*)k_cache.data_ptr(), (const uint16_t*)v_cache.data_ptr(),
      block_tables.data_ptr<int>(), (int)block_tables.size(1), cu_q.data_ptr<int>(), ctx_lens.data_ptr<int>(),
      pb.data_ptr<float>(), scale, chunk, out_scale, (uint16_t*)out.data_ptr(), ldo, H, G);
}

// max_qlen: the longest run of new tokens of one sequence in this step (1: single decoded tokens -> the wave-per-token
// kernel; the MFMA kernel takes bf16 with d a multiple of 32).
void attn_gated_chunk(const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache, const at::Tensor& block_tables,
                      const at::Tensor& cu_q, const at::Tensor& ctx_lens, const at::Tensor& pb, double scale, int64_t chunk,
                      double out_scale, at::Tensor& out, int64_t max_qlen) {
  MCHECK(q.is_cuda() && is_act(q) && q.is_contiguous() && q.dim() == 3, "q must be [T, H, d]");
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2);
  if (T == 0) return;
  MCHECK(k_cache.is_cuda() && k_cache.scalar_type() == q.scalar_type() && k_cache.is_contiguous() && k_cache.dim() == 4 &&
             k_cache.size(2) == PAGE_TOK && k_cache.size(3) == d, "k_cache must be [pages, G, 64, d] of q's dtype");
  const int64_t G = k_cache.size(1);
  MCHECK(v_cache.is_cuda() && v_cache.scalar_type() == q.scalar_type() && v_cache.is_contiguous() && v_cache.dim() == 4 &&
             v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G && v_cache.size(2) == d && v_cache.size(3) == PAGE_TOK,
         "v_cache must be [pages, G, d, 64] of q's dtype");
  MCHECK(G > 0 && H % G == 0 && d <= 256 && chunk > 0, "attn_gated_chunk: heads must be a multiple of kv heads, d <= 256");
  i32c(block_tables, "block_tables");
  i32c(cu_q, "cu_q");
  i32c(ctx_lens, "ctx_lens");
  f32c(pb, "pb");
  const int64_t B = ctx_lens.numel();
  MCHECK(block_tables.dim() == 2 && block_tables.size(0) == B && cu_q.numel() == B + 1 && pb.numel() == H, "batch shape mismatch");
  const int ldo = act_ld(out, T, H * d, "out");
  MCHECK(out.scalar_type() == q.scalar_type(), "out must have q's dtype");
  const bool bf = q.scalar_type() == at::kBFloat16;
  if (bf && max_qlen > 1 && d % 32 == 0 && ldo % 4 == 0 && reinterpret_cast<uintptr_t>(out.data_ptr()) % 8 == 0) {
    const dim3 grid((unsigned)B, (unsigned)((max_qlen + 127) / 128), (unsigned)H);
#define ATT_CASE(N)                                                                                                         \
  case N:                                                                                                                   \
    launch_attn_mfma<N>(grid, q, k_cache, v_cache, block_tables, cu_q, ctx_lens, pb, (float)scale, (int)chunk, (float)out_scale, \
                        out, ldo, (int)H, (int)G);                                                                          \
    break;
    switch (d / 32) {
      ATT_CASE(1) ATT_CASE(2) ATT_CASE(3) ATT_CASE(4) ATT_CASE(5) ATT_CASE(6) ATT_CASE(7) ATT_CASE(8)
    }
#undef ATT_CASE
    return;
  }
  if (H / G <= ATG_HEADS) {
    const int hpg = (int)(H / G);
    int dpad = 16;
    while (dpad < d) dpad *= 2;
    // key splits: enough workgroups to cover the chip (about four per CU), at least 64 keys each
    // (64 tokens x 4 kv heads, about 530 keys each: 61 / 46 / 35 / 45 us when aiming at 256 / 512 / 1024 / 2048 workgroups)
    const int64_t want_wgs = 1024;
    int KS = (int)std::min<int64_t>(std::min<int64_t>(8, (chunk + 63) / 64), (want_wgs + T * G - 1) / (T * G));
    KS = std::max(KS, 1);
    at::Tensor part;
    if (KS > 1) part = at::empty({KS, T, H * d}, q.options().dtype(at::kFloat));
    const dim3 grid((unsigned)T, (unsigned)G, (unsigned)KS);
    const size_t lds = ((size_t)hpg * d + (size_t)hpg * (ATG_TILE + 8) + (size_t)(256 / dpad) * hpg * dpad) * sizeof(float);
    float* pp = KS > 1 ? part.data_ptr<float>() : nullptr;
    const int blocks = (int)((T * H * d + 255) / 256);
    if (bf) {
      attn_gated_chunk_gqa_k<uint16_t><<<grid, 256, lds, stream()>>>(
          (const uint16_t*)q.data_ptr(), (const uint16_t*)k_cache.data_ptr(), (const uint16_t*)v_cache.data_ptr(),
          block_tables.data_ptr<int>(), (int)block_tables.size(1), cu_q.data_ptr<int>(), ctx_lens.data_ptr<int>(), (int)B,
          pb.data_ptr<float>(), (float)scale, (int)chunk, (float)out_scale, (uint16_t*)out.data_ptr(), ldo, pp, (int)T, (int)H,
          (int)G, (int)d, dpad, KS);
      if (KS > 1)
        attn_split_sum_k<uint16_t><<<blocks, 256, 0, stream()>>>(pp, KS, (int)T, (int)(H * d), (float)out_scale,
                                                                 (uint16_t*)out.data_ptr(), ldo, cu_q.data_ptr<int>(),
                                                                 ctx_lens.data_ptr<int>(), (int)B);
    } else {
      attn_gated_chunk_gqa_k<float><<<grid, 256, lds, stream()>>>(
          q.data_ptr<float>(), k_cache.data_ptr<float>(), v_cache.data_ptr<float>(), block_tables.data_ptr<int>(),
          (int)block_tables.size(1), cu_q.data_ptr<int>(), ctx_lens.data_ptr<int>(), (int)B, pb.data_ptr<float>(), (float)scale,
          (int)chunk, (float)out_scale, out.data_ptr<float>(), ldo, pp, (int)T, (int)H, (int)G, (int)d, dpad, KS);
      if (KS > 1)
        attn_split_sum_k<float><<<blocks, 256, 0, stream()>>>(pp, KS, (int)T, (int)(H * d), (float)out_scale,
                                                              out.data_ptr<float>(), ldo, cu_q.data_ptr<int>(),
                                                              ctx_lens.data_ptr<int>(), (int)B);
    }
    return;
  }
  const dim3 grid((unsigned)T, (unsigned)H);
  const size_t lds = (d + ATT_TILE + 8) * sizeof(float);
  if (bf)
    attn_gated_chunk_k<uint16_t><<<grid, 64, lds, stream()>>>(
        (const uint16_t*)q.data_ptr(), (const uint16_t*)k_cache.data_ptr(), (const uint16_t*)v_cache.data_ptr(),
        block_tables.data_ptr<int>(), (int)block_tables.size(1), cu_q.data_ptr<int>(), ctx_lens.data_ptr<int>(), (int)B,
        pb.data_ptr<float>(), (float)scale, (int)chunk, (float)out_scale, (uint16_t*)out.data_ptr(), ldo, (int)H, (int)G, (int)d);
  else
    attn_gated_chunk_k<float><<<grid, 64, lds, stream()>>>(
        q.data_ptr<float>(), k_cache.data_ptr<float>(), v_cache.data_ptr<float>(), block_tables.data_ptr<int>(),
        (int)block_tables.size(1), cu_q.data_ptr<int>(), ctx_lens.data_ptr<int>(), (int)B, pb.data_ptr<float>(), (float)scale,
        (int)chunk, (float)out_scale, out.data_ptr<float>(), ldo, (int)H, (int)G, (int)d);
}

void delta_prep(const at::Tensor& P, int64_t x_off, int64_t b_off, int64_t a_off, const at::Tensor& conv_w,
                at::Tensor& conv_state, const at::Tensor& state_slots, const at::Tensor& cu_q, const at::Tensor& A_log,
                const at::Tensor& dt_bias, int64_t H, int64_t G, int64_t d, int64_t dv, at::Tensor& qkv, at::Tensor& beta,
                at::Tensor& decay) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0), C = 2 * G * d + H * dv;
  if (T == 0) return;
  f32c(conv_w, "conv_w");
  f32c(conv_state, "conv_state");
  f32c(A_log, "A_log");
  f32c(dt_bias, "dt_bias");
  f32c(qkv, "qkv");
  f32c(beta, "beta");
  f32c(decay, "decay");
  i32c(state_slots, "state_slots");
  i32c(cu_q, "cu_q");
  MCHECK(conv_w.dim() == 2 && conv_w.size(0) == C, "conv_w must be [C, taps]");
  const int64_t taps = conv_w.size(1), B = state_slots.numel();
  MCHECK(taps >= 1 && conv_state.dim() == 3 && conv_state.size(1) == taps - 1 && conv_state.size(2) == C,
         "conv_state must be [slots, taps - 1, C]");
  MCHECK(cu_q.numel() == B + 1 && A_log.numel() == H && dt_bias.numel() == H && H % G == 0, "delta_prep: shape mismatch");
  MCHECK(qkv.numel() == T * C && beta.numel() == T * H && decay.numel() == T * H, "delta_prep: output shape mismatch");
  cols_ok(P, x_off, C, "conv inputs");
  cols_ok(P, b_off, H, "beta");
  cols_ok(P, a_off, H, "decay");
  MCHECK(d <= 256 && dv <= 256, "delta_prep: head sizes above 256");
  const int bs = (int)(((std::max(d, dv) + 63) / 64) * 64);
  const int tpb = T > 256 ? 8 : 1;
  delta_prep_k<<<dim3((unsigned)((T + tpb - 1) / tpb), (unsigned)(2 * G + H + 1)), bs, 0, stream()>>>(
      P.data_ptr<float>(), ldp, (int)x_off, (int)b_off, (int)a_off, conv_w.data_ptr<float>(), (int)taps,
      conv_state.data_ptr<float>(), state_slots.data_ptr<int>(), cu_q.data_ptr<int>(), (int)B, A_log.data_ptr<float>(),
      dt_bias.data_ptr<float>(), (int)H, (int)G, (int)d, (int)dv, qkv.data_ptr<float>(), beta.data_ptr<float>(),
      decay.data_ptr<float>(), (int)T, tpb);
  if (taps > 1) {
    const dim3 grid((unsigned)B, (unsigned)((C + 255) / 256));
    conv_state_update_k<<<grid, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)x_off, (int)C, (int)taps,
                                                    conv_state.data_ptr<float>(), state_slots.data_ptr<int>(),
                                                    cu_q.data_ptr<int>());
  }
}

void gla_prep(const at::Tensor& P, int64_t a1_off, const at::Tensor& a2, const at::Tensor& a2_b, double tau, at::Tensor& decay) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0) return;
  f32c(a2, "a2");
  f32c(a2_b, "a2_b");
  f32c(decay, "decay");
  MCHECK(a2.dim() == 2, "a2 must be [H d, rank]");
  const int64_t HD = a2.size(0), rank = a2.size(1);
  MCHECK(a2_b.numel() == HD && decay.numel() == T * HD && tau > 0, "gla_prep: shape mismatch");
  cols_ok(P, a1_off, rank, "decay projection");
  gla_prep_k<<<T, 256, rank * sizeof(float), stream()>>>(P.data_ptr<float>(), ldp, (int)a1_off, (int)rank, a2.data_ptr<float>(),
                                                         a2_b.data_ptr<float>(), (float)(1.0 / tau), (int)HD,
                                                         decay.data_ptr<float>());
}

template <int RS, int MODE>
void launch_rec(int KR, dim3 grid, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* decay,
                const float* beta, float q_scale, float* state, const int* slots, const int* cu, int H, int G, int d, int dv,
                int dvin, int dstride, float* out) {
#define REC_CASE(DPAD)                                                                                                 \
  case DPAD:                                                                                                           \
    linear_recurrence_k<DPAD / RS, RS, MODE><<<grid, 256, 0, stream()>>>(q, ldq, k, ldk, v, ldv, decay, beta, q_scale, \
                                                                          state, slots, cu, H, G, d, dv, dvin, dstride, out); \
    break;
  switch (KR * RS) {  // padded key dim
    REC_CASE(16)
    REC_CASE(32)
    REC_CASE(64)
    REC_CASE(128)
    REC_CASE(256)
    default:
      MCHECK(false, "linear_recurrence: key dim above 256");
  }
#undef REC_CASE
}

// q / k [T, G d], v [T, H dv]: fp32 rows of unit inner stride (column slices allowed).  decay [T, H] (delta rule, or
// without beta: one decay per head and a plain outer-product write; a 1-D [H]: the same decay at every token) or [T, H d]
// (per key channel); beta [T, H] (delta
// only; an input scale for a state with a normaliser channel: then v is [T, H (dv - 1)]).  state [slots, H, dv, d] (S^T: key
// rows contiguous).
void linear_recurrence(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& decay,
                       const c10::optional<at::Tensor>& beta, double q_scale, at::Tensor& state, const at::Tensor& state_slots,
                       const at::Tensor& cu_q, at::Tensor& out) {
  const int ldq = ld_of(q, "q"), ldk = ld_of(k, "k"), ldv = ld_of(v, "v");
  f32c(decay, "decay");
  f32c(state, "state");
  f32c(out, "out");
  i32c(state_slots, "state_slots");
  i32c(cu_q, "cu_q");
  MCHECK(state.dim() == 4, "state must be [slots, H, dv, d]");
  const int64_t T = q.size(0), H = state.size(1), dv = state.size(2), d = state.size(3), B = state_slots.numel();
  if (T == 0 || B == 0) return;
  MCHECK(q.size(1) % d == 0 && q.size(1) == k.size(1), "q / k must be [T, G d]");
  const int64_t G = q.size(1) / d;
  const bool normch = v.size(1) == H * (dv - 1);  // the state's last value channel is a normaliser, beta an input scale
  const int64_t dvin = normch ? dv - 1 : dv;
  MCHECK(G > 0 && H % G == 0 && k.size(0) == T && v.size(0) == T && v.size(1) == H * dvin && out.numel() == T * H * dv,
         "linear_recurrence: shape mismatch");
  MCHECK(cu_q.numel() == B + 1, "cu_q must hold B + 1 offsets");
  MCHECK(!normch || beta.has_value(), "a state with a normaliser channel needs the input scales");
  const bool delta = beta.has_value() && !normch;
  if (beta.has_value()) {
    f32c(*beta, "beta");
    MCHECK(beta->numel() == T * H && decay.numel() == T * H, "delta rule: beta / decay must be [T, H]");
  } else if (decay.numel() != T * H && !(decay.dim() == 1 && decay.numel() == H)) {
    MCHECK(decay.numel() == T * H * d && G == H, "per-channel decay must be [T, H d] with one q / k head per value head");
  }
  // one decay per head (and token: [T, H]; or fixed: a 1-D [H]), q / k shared by H / G heads
  const bool fixed = !delta && !normch && decay.dim() == 1 && decay.numel() == H;
  const bool scalar = !delta && !normch && (fixed || decay.numel() == T * H);
  int DP = 16;
  while (DP < d) DP *= 2;
  MCHECK(DP <= 256, "linear_recurrence: key dim above 256");
  // 16 row groups per value channel (4 and 8, with more rows per thread, measured slower at 8 x 2048 tokens and 16
  // heads: d 64 / dv 128 0.89 / 0.75 / 0.70 ms with 4 / 8 / 16, d 128 / dv 128 1.57 / 1.28 / 1.23)
  const int RS = 16;
  const int cols = 256 / RS;
  const dim3 grid((unsigned)B, (unsigned)H, (unsigned)((dv + cols - 1) / cols));
  const float* bp = beta.has_value() ? beta->data_ptr<float>() : nullptr;
#define REC_GO(R, D)                                                                                                          \
  launch_rec<R, D>(DP / R, grid, q.data_ptr<float>(), ldq, k.data_ptr<float>(), ldk, v.data_ptr<float>(), ldv,              \
                   decay.data_ptr<float>(), bp, (float)q_scale, state.data_ptr<float>(), state_slots.data_ptr<int>(),        \
                   cu_q.data_ptr<int>(), (int)H, (int)G, (int)d, (int)dv, (int)dvin, fixed ? 0 : (int)H,         \
                   out.data_ptr<float>())
  if (delta) REC_GO(16, 1); else if (normch) REC_GO(16, 3); else if (scalar) REC_GO(16, 2); else REC_GO(16, 0);
#undef REC_GO
}

void gated_rmsnorm(const at::Tensor& o, const at::Tensor& w, const at::Tensor& P, int64_t g_off, double eps, double out_scale,
                   at::Tensor& out) {
  f32c(o, "o");
  f32c(w, "w");
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0), dv = w.numel();
  if (T == 0) return;
  MCHECK(dv > 0 && o.numel() % (T * dv) == 0, "o must be [T, H, dv]");
  const int64_t H = o.numel() / (T * dv);
  cols_ok(P, g_off, H * dv, "gate");
  const int ldo = act_ld(out, T, H * dv, "out");
  const dim3 grid((unsigned)T, (unsigned)H);
  if (out.scalar_type() == at::kBFloat16)
    gated_rmsnorm_k<uint16_t><<<grid, 64, 0, stream()>>>(o.data_ptr<float>(), w.data_ptr<float>(), P.data_ptr<float>(), ldp,
                                                         (int)g_off, (float)eps, (float)out_scale, (uint16_t*)out.data_ptr(),
                                                         ldo, (int)H, (int)dv);
  else
    gated_rmsnorm_k<float><<<grid, 64, 0, stream()>>>(o.data_ptr<float>(), w.data_ptr<float>(), P.data_ptr<float>(), ldp,
                                                      (int)g_off, (float)eps, (float)out_scale, out.data_ptr<float>(), ldo,
                                                      (int)H, (int)dv);
}

}  // namespace

void bind_mixers(pybind11::module& m) {
  m.def("resid_scale_norm", &resid_scale_norm);
  m.def("gelu_mul", &gelu_mul);
  m.def("rope_kv_store", &rope_kv_store);
  m.def("attn_gated_chunk", &attn_gated_chunk);
  m.def("delta_prep", &delta_prep);
  m.def("gla_prep", &gla_prep);
  m.def("linear_recurrence", &linear_recurrence);
  m.def("gated_rmsnorm", &gated_rmsnorm);
}

}  // namespace xot
