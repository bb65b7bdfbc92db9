// Kernels of sandwich-block models with latent attention (fp32 residual stream; activations AT = bf16 or fp32).
//
//   sandwich_add_norm   x += mult * norm(y), and the next sublayer's input norm(x) in the GEMM operand dtype (RMS norms with
//                       a weight, or layer norms with weight and bias)
//   latent_kv_store     kv latent RMS norm + RoPE of the shared rotated key part -> one cache row per token; the query
//                       latent's RMS norm
//   latent_q_rope       queries: unrotated parts per head [H, T, dn] (operand of q . W_uk), rotated parts after RoPE
//   latent_attn         softmax attention of absorbed queries over the cached rows [latent | rotated key part], the
//                       latent being key and value; sliding window, per-head sink logit
//   latent_out_gate     heads' outputs [H, T, dv] -> token-major rows, times sigmoid gates (per element or per head)
//   glu_act             silu(g) u, or the clamped form g' sigmoid(1.702 g') (u' + 1)
//
// Cache: [pages, 1, 64, R + dr] (R = latent size, dr = rotated key dims), a page's 64 rows contiguous.  Attention is
// multi-query over these rows: head h's query is [q_lat,h (R) | q_pe,h (dr)], its output o_lat,h = sum_j w_j c_j (R).
#include "mixer_util.h"

namespace xot {
namespace {
using namespace mix;

typedef __attribute__((address_space(3))) s16x4* lds_s16x4_t;
// transposed LDS read (gfx950): within each group of 16 lanes, lane 4 q + p gives the address of 4 consecutive 16-bit
// elements (row q, columns 4 p .. 4 p + 3 of a 4 x 16 block); lane c receives column c of rows 0 .. 3
__device__ __forceinline__ s16x4 tr_read(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)(p));
}

constexpr float LOG2E_F = 1.4426950408889634f;

// ------------------------------------------------------------------ residual add of a normed sublayer result + next norm
// norm of one row held in global memory: v / rms(v) * w, or with a bias the layer norm (v - mean) / sqrt(var + eps) * w + b
// (the variance as the mean of the squared deviations, in a pass of its own).  Returns (shift, scale).
__device__ __forceinline__ void row_norm_stats(const float* v, int D, bool center, float eps, float* red, float* shift,
                                               float* scale) {
  float mean = 0.0f;
  if (center) {
    float s = 0.0f;
    for (int i = threadIdx.x; i < D; i += blockDim.x) s += v[i];
    mean = block_sum(s, red) / D;
  }
  float ss = 0.0f;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    const float c = v[i] - mean;
    ss += c * c;
  }
  ss = block_sum(ss, red);
  *shift = mean;
  *scale = 1.0f / sqrtf(ss / D + eps);
}

template <typename AT>
__global__ __launch_bounds__(256) void sandwich_add_norm_k(float* __restrict__ x, const float* __restrict__ y, int ldy,
                                                           const float* __restrict__ wb, const float* __restrict__ bb,
                                                           const float* __restrict__ wn, const float* __restrict__ bn,
                                                           float mult, float eps, AT* __restrict__ out, int ldo, int D) {
  __shared__ float red[8];
  const int64_t t = blockIdx.x;
  float* xr = x + t * D;
  if (y) {
    const float* yr = y + t * ldy;
    float mu, r;
    row_norm_stats(yr, D, bb != nullptr, eps, red, &mu, &r);
    for (int i = threadIdx.x; i < D; i += blockDim.x) xr[i] += mult * ((yr[i] - mu) * r * wb[i] + (bb ? bb[i] : 0.0f));
  }
  if (wn) {  // (a thread re-reads the elements it wrote itself)
    float mu, r;
    row_norm_stats(xr, D, bn != nullptr, eps, red, &mu, &r);
    for (int i = threadIdx.x; i < D; i += blockDim.x) stf(out + t * ldo + i, (xr[i] - mu) * r * wn[i] + (bn ? bn[i] : 0.0f));
  }
}

// element i of a vector whose first `rot` dims are rotated: pairs (2i, 2i + 1) (inter) or (i, i + rot / 2);
// cs = (cos | sin) of the token's position, rot / 2 each
__device__ __forceinline__ float rope_elem(const float* __restrict__ v, int i, int rot, int inter, const float* __restrict__ cs) {
  if (i >= rot) return v[i];
  const int half = rot >> 1;
  int fi, partner;
  bool first;
  if (inter) {
    fi = i >> 1;
    first = !(i & 1);
    partner = i ^ 1;
  } else {
    first = i < half;
    fi = first ? i : i - half;
    partner = first ? i + half : i - half;
  }
  const float a = v[i], b = v[partner], c = cs[fi], s = cs[half + fi];
  return first ? a * c - b * s : a * c + b * s;
}

template <typename AT>
__global__ __launch_bounds__(256) void latent_kv_store_k(const float* __restrict__ P, int ldp, int ckv_off, int R, int dr,
                                                         const float* __restrict__ kv_norm, int q_off, int q_rank,
                                                         const float* __restrict__ q_norm, float eps, int rot, int inter,
                                                         const int* __restrict__ pos, const float* __restrict__ cs,
                                                         const int64_t* __restrict__ slots, AT* __restrict__ cache,
                                                         AT* __restrict__ qa, int ldqa) {
  __shared__ float red[8];
  const int64_t t = blockIdx.x;
  const float* pr = P + t * ldp;
  const int64_t slot = slots[t];
  float ss = 0.0f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) ss += pr[ckv_off + i] * pr[ckv_off + i];
  ss = block_sum(ss, red);
  if (slot >= 0) {
    AT* row = cache + slot * (R + dr);
    const float r = 1.0f / sqrtf(ss / R + eps);
    for (int i = threadIdx.x; i < R; i += blockDim.x) stf(row + i, pr[ckv_off + i] * r * kv_norm[i]);
    const float* c = cs + (int64_t)pos[t] * rot;
    for (int i = threadIdx.x; i < dr; i += blockDim.x) stf(row + R + i, rope_elem(pr + ckv_off + R, i, rot, inter, c));
  }
  if (q_rank > 0) {
    float sq = 0.0f;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) sq += pr[q_off + i] * pr[q_off + i];
    sq = block_sum(sq, red);
    const float r = 1.0f / sqrtf(sq / q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) stf(qa + t * ldqa + i, pr[q_off + i] * r * q_norm[i]);
  }
}

template <typename AT>
__global__ __launch_bounds__(256) void latent_q_rope_k(const float* __restrict__ Q, int ldq, int q_off, int T, int H, int dn,
                                                       int dr, int rot, int inter, const int* __restrict__ pos,
                                                       const float* __restrict__ cs, AT* __restrict__ qn,
                                                       AT* __restrict__ qpe) {
  const int64_t t = blockIdx.x;
  const int d = dn + dr;
  const float* c = cs + (int64_t)pos[t] * rot;
  for (int e = threadIdx.x; e < H * d; e += blockDim.x) {
    const int h = e / d, i = e - h * d;
    const float* qh = Q + t * ldq + q_off + h * d;
    if (i < dn)
      stf(qn + ((int64_t)h * T + t) * dn + i, qh[i]);
    else
      stf(qpe + (t * H + h) * dr + (i - dn), rope_elem(qh + dn, i - dn, rot, inter, c));
  }
}

template <typename AT>
__global__ __launch_bounds__(256) void latent_out_gate_k(const AT* __restrict__ o, const float* __restrict__ P, int ldp,
                                                         int g_off, int gate, int T, int H, int dv, AT* __restrict__ out,
                                                         int ldo) {
  const int64_t t = blockIdx.x;
  for (int e = threadIdx.x; e < H * dv; e += blockDim.x) {
    const int h = e / dv, i = e - h * dv;
    float v = ldf(o + ((int64_t)h * T + t) * dv + i);
    if (gate == 1) v *= sigmoidf_(P[t * ldp + g_off + e]);
    if (gate == 2) v *= sigmoidf_(P[t * ldp + g_off + h]);
    stf(out + t * ldo + e, v);
  }
}

template <typename AT>
__global__ void glu_act_k(const float* __restrict__ P, int ldp, int gate_off, int up_off, int F, int clamped, float limit,
                          AT* __restrict__ out, int ldo, int64_t total) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int64_t t = e / F;
  const int i = (int)(e - t * F);
  float g = P[t * ldp + gate_off + i], u = P[t * ldp + up_off + i];
  float y;
  if (clamped) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    y = g * sigmoidf_(1.702f * g) * (u + 1.0f);
  } else {
    y = siluf_(g) * u;
  }
  stf(out + t * ldo + i, y);
}

// ------------------------------------------------------------------ attention over the latent rows: any sizes, bf16 / fp32
// Workgroup per (token, REP heads), LATT_WAVES waves: key tiles are dealt to the waves in turn; a lane scores one key
// row against the REP absorbed queries (fp32 dot products, the row loaded once for all of them), then the wave sums the
// weighted latents, a lane owning the value dims lane, lane + 64, ...  A wave's running maxima start at -inf (wave 0: at
// the sinks' logits with denominators of one); the waves' (maximum, denominator, sums) are merged through LDS.
constexpr int LATT_WAVES = 8;
constexpr int LATT_TILE = 64;

template <typename AT, int REP, int NC>
__global__ __launch_bounds__(64 * LATT_WAVES) void latent_attn_k(
    const AT* __restrict__ q_lat, const AT* __restrict__ q_pe, const AT* __restrict__ cache,
    const int* __restrict__ block_tables, int width, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, int B,
    int T, const float* __restrict__ sink, float scale, int window, AT* __restrict__ out, int H, int R, int dr) {
  extern __shared__ float sm[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int d = R + dr;
  float* qs = sm;                                              // [REP][d]
  float* ws = sm + REP * d + wave * REP * LATT_TILE;           // [REP][TILE] per wave
  float* mg = sm + REP * d + LATT_WAVES * REP * LATT_TILE;     // merge: [waves][REP][2 + R]
  const int t = blockIdx.x, h0 = blockIdx.y * REP;
  const int b = seq_of(cu_q, B, t);
  const int ctx = ctx_lens[b];
  if (ctx <= 0) {  // padding row of a captured decode batch: zeros, so that nothing downstream reads stale memory
    for (int e = threadIdx.x; e < REP * R; e += blockDim.x)
      if (h0 + e / R < H) stf(out + ((int64_t)(h0 + e / R) * T + t) * R + e % R, 0.0f);
    return;
  }
  const int pos = ctx - (cu_q[b + 1] - cu_q[b]) + (t - cu_q[b]);
  for (int i = threadIdx.x; i < REP * d; i += blockDim.x) {
    const int r = i / d, e = i - r * d, h = min(h0 + r, H - 1);
    qs[i] = e < R ? ldf(q_lat + ((int64_t)h * T + t) * R + e) : ldf(q_pe + ((int64_t)t * H + h) * dr + (e - R));
  }
  __syncthreads();
  const int* bt = block_tables + (int64_t)b * width;
  float m[REP], l[REP], acc[REP][NC];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    const bool sk = sink && wave == 0;
    m[r] = sk ? sink[min(h0 + r, H - 1)] : -INFINITY;
    l[r] = sk ? 1.0f : 0.0f;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[r][c] = 0.0f;
  }
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  int tile = 0;
  for (int a0 = lo; a0 <= pos; a0 += LATT_TILE, ++tile) {
    if (tile % LATT_WAVES != wave) continue;
    const int n = min(LATT_TILE, pos + 1 - a0);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    float s[REP];
#pragma unroll
    for (int r = 0; r < REP; ++r) s[r] = -INFINITY;
    if (lane < n) {
      const int p = a0 + lane;
      const AT* kr = cache + ((int64_t)bt[p / PAGE_TOK] * PAGE_TOK + (p % PAGE_TOK)) * d;
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
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      const float mn = fmaxf(m[r], wave_max(s[r]));
      const float w = s[r] == -INFINITY ? 0.0f : expf(s[r] - mn);
      ws[r * LATT_TILE + lane] = w;
      const float corr = m[r] == -INFINITY ? 0.0f : expf(m[r] - mn);
      l[r] = l[r] * corr + wave_sum(w);
#pragma unroll
      for (int c = 0; c < NC; ++c) acc[r][c] *= corr;
      m[r] = mn;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int j = 0; j < n; ++j) {
      const int p = a0 + j;
      const AT* vr = cache + ((int64_t)bt[p / PAGE_TOK] * PAGE_TOK + (p % PAGE_TOK)) * d;
      float vv[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) vv[c] = lane + 64 * c < R ? ldf(vr + lane + 64 * c) : 0.0f;
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        const float w = ws[r * LATT_TILE + j];
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[r][c] += w * vv[c];
      }
    }
  }
  // merge the waves: M = max m_w, out = sum_w acc_w e^(m_w - M) / sum_w l_w e^(m_w - M)
  const int ms = 2 + R;
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    float* mine = mg + (wave * REP + r) * ms;
    if (lane == 0) {
      mine[0] = m[r];
      mine[1] = l[r];
    }
#pragma unroll
    for (int c = 0; c < NC; ++c)
      if (lane + 64 * c < R) mine[2 + lane + 64 * c] = acc[r][c];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < REP * R; e += blockDim.x) {
    const int r = e / R, i = e - r * R;
    if (h0 + r >= H) continue;
    float M = -INFINITY;
    for (int w = 0; w < LATT_WAVES; ++w) M = fmaxf(M, mg[(w * REP + r) * ms]);
    float L = 0.0f, a = 0.0f;
    for (int w = 0; w < LATT_WAVES; ++w) {
      const float* o = mg + (w * REP + r) * ms;
      if (o[0] != -INFINITY) {
        const float f = expf(o[0] - M);
        L += o[1] * f;
        a += o[2 + i] * f;
      }
    }
    stf(out + ((int64_t)(h0 + r) * T + t) * R + i, L > 0.0f ? a / L : 0.0f);
  }
}

// ------------------------------------------------------------------ MFMA kernel (bf16): prompt portions and single tokens
// Columns of a wave's 16x16 tiles are 16 (query, head) pairs that share the keys: in a prompt portion (DEC false) a
// workgroup of four waves owns 64 consecutive new tokens of one (sequence, head), 16 per wave; for single tokens (DEC
// true) a one-wave workgroup owns one token's block of 16 heads and one share of its pages (key split), and writes
// (maximum, denominator, sums) partials that latent_attn_merge_k adds up.  A page's 64 rows are staged in LDS row-major
// (row length padded with zeros to a multiple of 32); the queries sit in registers as B operands.
// Scores are computed transposed, S^T = K Q^T (keys x columns, 16x16x32 MFMA), so a lane's accumulator rows are keys
// of ONE column: running maximum and denominator are per lane (the four lanes of a column agree on the maximum through
// two shuffles and keep partial denominators), and the exponentials, rounded to bf16, are as they lie the B operand of
// O^T += V^T P^T, whose k slots (g, j) are read as keys {4g .. 4g+3, 16+4g .. 16+4g+3} on both operands.  The V^T
// operand comes straight out of the row-major page image by the transposed LDS read (4 keys x 16 dims per 16 lanes).
// Scores, maxima and sums are fp32 (base-2 exponentials of scores scaled by log2 e); a sink's logit starts the
// running maximum with a denominator of one.  NV: compile-time bound on R / 16 (output accumulators); the row length
// is at most 32 (NV / 2 + 2).
constexpr int LM_PAD = 8;

template <int NV, bool DEC>
__global__ __launch_bounds__(256) void latent_attn_mfma_k(
    const uint16_t* __restrict__ q_lat, const uint16_t* __restrict__ q_pe, const uint16_t* __restrict__ cache,
    const int* __restrict__ block_tables, int width, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, int B,
    int T, const float* __restrict__ sink, float scale_l2, int window, uint16_t* __restrict__ out, float* __restrict__ part,
    int nsplit, int H, int R, int dr) {
  // (row length and output tiles are the template's bounds: columns past the real sizes hold zeros, output tiles past
  // the latent are computed and dropped, so the MFMA loops have no run-time conditions and pipeline their LDS reads)
  constexpr int NQ = NV / 2 + 2, NT = 256, QROWS = DEC ? 16 : 64, DKp = NQ * 32, LDK = DKp + LM_PAD;
  extern __shared__ __attribute__((aligned(16))) uint16_t lsm[];
  const int DK = R + dr, nv = R >> 4;
  uint16_t* Qs = lsm;                 // [QROWS][LDK]
  uint16_t* Ks = Qs + QROWS * LDK;    // [2][64][LDK]: the page in use and the next one
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, lq = lane & 15;
  int b, h0 = 0, t0 = 0, ql = 0, q0 = 0, base = 0, tok = 0;
  if constexpr (DEC) {
    tok = blockIdx.z;
    h0 = blockIdx.y * 16;
    b = tok;  // (a step of single tokens: token t is sequence t's)
  } else {
    b = blockIdx.y;
    h0 = blockIdx.z;
    q0 = blockIdx.x * 64;
  }
  const int n = ctx_lens[b];
  t0 = cu_q[b];
  ql = cu_q[b + 1] - t0;
  base = n - ql;
  const int head = DEC ? min(h0 + lq, H - 1) : h0;
  if constexpr (DEC) {
    if (n <= 0) {  // padding row of a captured decode batch: zeros, an empty partial
      if (h0 + lq < H && wave == 0) {
        if (nsplit == 1) {
          for (int i = g; i < R; i += 4) out[((int64_t)head * T + tok) * R + i] = 0;
        } else {
          float* pr = part + (((int64_t)tok * H + head) * nsplit + blockIdx.x) * (2 + R);
          for (int i = g; i < 2 + R; i += 4) pr[i] = i == 0 ? -INFINITY : 0.0f;
        }
      }
      return;
    }
  } else {
    if (n <= 0 || q0 >= ql) return;
  }
  const int* bt = block_tables + (int64_t)b * width;
  // this lane's column: its query's position, whether it is a real one
  const int qi = DEC ? 0 : q0 + 16 * wave + lq;
  const bool valid = DEC ? (h0 + lq < H) : (qi < ql);
  const int qp = DEC ? base + (tok - t0) : base + qi;
  const int wq_lo = DEC ? qp : base + q0 + 16 * wave;                       // the wave's positions
  const int wq_hi = DEC ? qp : base + min(q0 + 16 * wave + 15, ql - 1);
  const int first = DEC ? (window > 0 ? max(0, qp - window + 1) : 0) : (window > 0 ? max(0, base + q0 - window + 1) : 0);
  const int last = DEC ? qp : base + min(q0 + 63, ql - 1);
  int pg0 = first / PAGE_TOK, pg1 = last / PAGE_TOK + 1;
  if constexpr (DEC) {
    const int per = (pg1 - pg0 + nsplit - 1) / nsplit;
    pg0 += blockIdx.x * per;
    pg1 = min(pg1, pg0 + per);
  }
  float m = -INFINITY, l = 0.0f;
  if (sink && (!DEC || blockIdx.x == 0)) {
    m = sink[head] * LOG2E_F;
    l = g == 0 ? 1.0f : 0.0f;
  }
  f32x4 acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  const int kchunks = DK >> 3;
  const int q4 = lq >> 2, p4 = lq & 3;
  // a page's rows travel global -> registers -> LDS, a thread's chunks all in flight at once; the next page is
  // fetched into registers before this page's MFMAs and written to the other buffer after them
  s16x8 pre[NQ];
  auto fetch = [&](int pg) {
    const uint16_t* src = cache + (int64_t)bt[pg] * PAGE_TOK * DK;
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int idx = tid + NT * u;
      if (idx < 64 * kchunks) {
        const int row = idx / kchunks, dim = (idx - row * kchunks) << 3;
        pre[u] = ld16(src + row * DK + dim);
      }
    }
  };
  auto commit = [&](uint16_t* dst) {
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int idx = tid + NT * u;
      if (idx < 64 * kchunks) {
        const int row = idx / kchunks, dim = (idx - row * kchunks) << 3;
        st16(dst + row * LDK + dim, pre[u]);
      }
    }
  };
  if (pg0 < pg1) fetch(pg0);  // (in flight while the queries are staged)
  // queries -> LDS (rows without a query and the padding columns: zero), then into registers as B operands
  const int chunks = DKp >> 3;
  for (int idx = tid; idx < QROWS * chunks; idx += NT) {
    const int row = idx / chunks, dim = (idx - row * chunks) << 3;
    s16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    const bool has = DEC ? (h0 + row < H) : (q0 + row < ql);
    if (has && dim < DK) {
      const int64_t t = DEC ? tok : t0 + q0 + row;
      const int hh = DEC ? h0 + row : h0;
      v = dim < R ? ld16(q_lat + ((int64_t)hh * T + t) * R + dim) : ld16(q_pe + (t * H + hh) * dr + (dim - R));
    }
    st16(Qs + row * LDK + dim, v);
  }
  for (int idx = tid; idx < 128 * ((DKp - DK) >> 3); idx += NT) {  // the keys' padding columns stay zero
    const int pc = (DKp - DK) >> 3, row = idx / pc, dim = DK + ((idx - row * pc) << 3);
    st16(Ks + row * LDK + dim, s16x8{0, 0, 0, 0, 0, 0, 0, 0});
  }
  if (pg0 < pg1) commit(Ks);
  __syncthreads();
  s16x8 qreg[NQ];
  {
    const uint16_t* qb = Qs + ((DEC ? 0 : 16 * wave) + lq) * LDK + 8 * g;
#pragma unroll
    for (int i = 0; i < NQ; ++i) qreg[i] = ld16(qb + 32 * i);
  }
  for (int pg = pg0; pg < pg1; ++pg) {
    const uint16_t* Kc = Ks + ((pg - pg0) & 1) * 64 * LDK;
    const bool more = pg + 1 < pg1;
    if (more) fetch(pg + 1);
    if (!DEC || wave == 0) {
    const int k0 = pg * PAGE_TOK;
    // scores of the page's four 16-key sub-tiles that some column of this wave sees
    f32x4 S[4];
    bool live[4];
    float mx = -INFINITY;
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      const int ks = k0 + 16 * sub;
      live[sub] = ks <= wq_hi && (window == 0 || ks + 15 > wq_lo - window) && wq_lo <= wq_hi;
      S[sub] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      if (!live[sub]) continue;
      const uint16_t* ka = Kc + (16 * sub + lq) * LDK + 8 * g;
#pragma unroll
      for (int i = 0; i < NQ; ++i) S[sub] = mfma16(ld16(ka + 32 * i), qreg[i], S[sub]);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kp = ks + 4 * g + r;
        const bool vis = valid && kp <= qp && (window == 0 || qp - kp < window);
        S[sub][r] = vis ? S[sub][r] * scale_l2 : -INFINITY;
        mx = fmaxf(mx, S[sub][r]);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const float corr = m == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m - mn);
    m = mn;
    float ls = 0.0f;
    s16x8 pb[2];
#pragma unroll
    for (int sub = 0; sub < 4; ++sub)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float sv = live[sub] ? S[sub][r] : -INFINITY;
        const float p = sv == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(sv - mn);
        const uint16_t pbits = f2bf(p);
        ls += bf2f(pbits);
        pb[sub >> 1][(sub & 1) * 4 + r] = (short)pbits;
      }
    l = l * corr + ls;
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] *= corr;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      if (!live[2 * kk] && !live[2 * kk + 1]) continue;
      // V^T fragments by transposed LDS reads: lane 4 q4 + p4 of group g addresses key 32 kk (+ 16) + 4 g + q4, dims
      // 16 i + 4 p4 .. + 3; lane lq receives dim 16 i + lq of those four keys
      const uint16_t* vb = Kc + (32 * kk + 4 * g + q4) * LDK + 4 * p4;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const s16x4 a0 = tr_read(vb + 16 * i), a1 = tr_read(vb + 16 * LDK + 16 * i);
        const s16x8 a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
        acc[i] = mfma16(a, pb[kk], acc[i]);
      }
    }
    }
    if (more) commit(Ks + (((pg - pg0) & 1) ^ 1) * 64 * LDK);
    __syncthreads();  // the next page is written, this one's readers are done
  }
  if (DEC && wave != 0) return;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!valid) return;
  if (DEC && nsplit > 1) {
    float* pr = part + (((int64_t)tok * H + head) * nsplit + blockIdx.x) * (2 + R);
    if (g == 0) {
      pr[0] = m;
      pr[1] = l;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (i >= nv) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) pr[2 + 16 * i + 4 * g + r] = acc[i][r];
    }
    return;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  uint16_t* orow = out + ((int64_t)head * T + (DEC ? tok : t0 + qi)) * R;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (i >= nv) continue;
    s16x4 o;
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = (short)f2bf(acc[i][r] * inv);
    *reinterpret_cast<s16x4*>(orow + 16 * i + 4 * g) = o;
  }
}

// partials of the key splits [T, H, nsplit, 2 + R] (base-2 maximum, denominator, sums) -> out [H, T, R]
__global__ __launch_bounds__(256) void latent_attn_merge_k(const float* __restrict__ part, int nsplit, int T, int H, int R,
                                                          uint16_t* __restrict__ out) {
  __shared__ float w[64];  // nsplit <= 64: the first wave weighs the splits
  const int64_t th = blockIdx.x;  // t * H + h
  const int t = (int)(th / H), h = (int)(th - (int64_t)t * H);
  const float* p = part + th * nsplit * (2 + R);
  if (threadIdx.x < 64) {
    const int sidx = threadIdx.x;
    const float ms = sidx < nsplit ? p[sidx * (2 + R)] : -INFINITY;
    const float ls = sidx < nsplit ? p[sidx * (2 + R) + 1] : 0.0f;
    const float M = wave_max(ms);
    const float f = ms == -INFINITY ? 0.0f : exp2f(ms - M);
    const float L = wave_sum(ls * f);
    w[sidx] = L > 0.0f ? f / L : 0.0f;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    float a = 0.0f;
#pragma unroll 4
    for (int sp = 0; sp < nsplit; ++sp) a += w[sp] * p[sp * (2 + R) + 2 + i];
    out[((int64_t)h * T + t) * R + i] = f2bf(a);
  }
}

// The same for rows of at most 256 R numbers: a thread keeps its R values of y and of x in registers, so each row is
// read once (the sums run over registers; the variance still after the mean, as the mean of the squared deviations).
template <typename AT, int R>
__global__ __launch_bounds__(256) void sandwich_add_norm_reg_k(float* __restrict__ x, const float* __restrict__ y, int ldy,
                                                               const float* __restrict__ wb, const float* __restrict__ bb,
                                                               const float* __restrict__ wn, const float* __restrict__ bn,
                                                               float mult, float eps, AT* __restrict__ out, int ldo, int D) {
  __shared__ float red[8];
  const int64_t t = blockIdx.x;
  float* xr = x + t * D;
  float xv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = threadIdx.x + 256 * r;
    xv[r] = i < D ? xr[i] : 0.0f;
  }
  // (shift, scale) of a row held in registers
  auto stats = [&](const float* v, bool center, float* mu, float* rs) {
    float mean = 0.0f;
    if (center) {
      float s = 0.0f;
#pragma unroll
      for (int r = 0; r < R; ++r) s += v[r];  // (entries past D are zero)
      mean = block_sum(s, red) / D;
    }
    float ss = 0.0f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float c = threadIdx.x + 256 * r < D ? v[r] - mean : 0.0f;
      ss += c * c;
    }
    ss = block_sum(ss, red);
    *mu = mean;
    *rs = 1.0f / sqrtf(ss / D + eps);
  };
  if (y) {
    const float* yr = y + t * ldy;
    float yv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = threadIdx.x + 256 * r;
      yv[r] = i < D ? yr[i] : 0.0f;
    }
    float mu, rs;
    stats(yv, bb != nullptr, &mu, &rs);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = threadIdx.x + 256 * r;
      if (i < D) {
        xv[r] += mult * ((yv[r] - mu) * rs * wb[i] + (bb ? bb[i] : 0.0f));
        xr[i] = xv[r];
      }
    }
  }
  if (wn) {
    float mu, rs;
    stats(xv, bn != nullptr, &mu, &rs);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = threadIdx.x + 256 * r;
      if (i < D) stf(out + t * ldo + i, (xv[r] - mu) * rs * wn[i] + (bn ? bn[i] : 0.0f));
    }
  }
}

// ------------------------------------------------------------------ host side
// XOT_LATT_MFMA=0 keeps prompt portions on the wave-per-tile attention kernel (A/B runs)
const bool LATT_MFMA = []() { const char* e = getenv("XOT_LATT_MFMA"); return !(e && e[0] == '0'); }();

void sandwich_add_norm(at::Tensor& x, const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& wb,
                       const c10::optional<at::Tensor>& wn, double eps, const c10::optional<at::Tensor>& out,
                       const c10::optional<at::Tensor>& bb, const c10::optional<at::Tensor>& bn, double mult) {
  f32c(x, "x");
  MCHECK(x.dim() == 2, "x must be [T, D]");
  const int64_t T = x.size(0), D = x.size(1);
  if (T == 0) return;
  const float *yp = nullptr, *bp = nullptr, *np = nullptr, *bbp = nullptr, *bnp = nullptr;
  int ldy = 0, ldo = 0;
  if (bb.has_value()) {
    f32c(*bb, "bb");
    MCHECK(bb->numel() == D && y.has_value(), "the result norm's bias must hold D numbers");
    bbp = bb->data_ptr<float>();
  }
  if (bn.has_value()) {
    f32c(*bn, "bn");
    MCHECK(bn->numel() == D && wn.has_value(), "the next norm's bias must hold D numbers");
    bnp = bn->data_ptr<float>();
  }
  if (y.has_value()) {
    ldy = ld_of(*y, "y");
    MCHECK(y->size(0) == T && y->size(1) >= D && wb.has_value(), "the sublayer's result must be fp32 [T, >= D] rows with a norm weight");
    f32c(*wb, "wb");
    MCHECK(wb->numel() == D, "the norm weight must hold D numbers");
    yp = y->data_ptr<float>();
    bp = wb->data_ptr<float>();
  }
  void* op = nullptr;
  bool bf = true;
  if (wn.has_value()) {
    f32c(*wn, "wn");
    MCHECK(wn->numel() == D && out.has_value(), "the next norm needs D weights and an output");
    ldo = act_ld_min(*out, T, D, "out");
    np = wn->data_ptr<float>();
    op = out->data_ptr();
    bf = out->scalar_type() == at::kBFloat16;
  }
  if (!yp && !np) return;
#define SAN_GO(KERNEL, AT)                                                                                              \
  KERNEL<<<T, 256, 0, stream()>>>(x.data_ptr<float>(), yp, ldy, bp, bbp, np, bnp, (float)mult, (float)eps, (AT*)op, ldo, \
                                  (int)D)
#define SAN_PICK(AT)                                                     \
  if (D <= 1024) SAN_GO((sandwich_add_norm_reg_k<AT, 4>), AT);           \
  else if (D <= 2048) SAN_GO((sandwich_add_norm_reg_k<AT, 8>), AT);      \
  else if (D <= 4096) SAN_GO((sandwich_add_norm_reg_k<AT, 16>), AT);     \
  else SAN_GO(sandwich_add_norm_k<AT>, AT)
  if (bf) {
    SAN_PICK(uint16_t);
  } else {
    SAN_PICK(float);
  }
#undef SAN_PICK
#undef SAN_GO
}

void check_rope(const at::Tensor& pos, const at::Tensor& cos_sin, int64_t T, int64_t rot, int64_t dr) {
  i32c(pos, "pos");
  f32c(cos_sin, "cos_sin");
  MCHECK(pos.numel() == T, "pos must hold one entry per token");
  MCHECK(rot >= 0 && rot % 2 == 0 && rot <= dr && (rot == 0 || (cos_sin.dim() == 2 && cos_sin.size(1) == rot)), "bad rotary dims");
}

void check_latent_cache(const at::Tensor& cache, at::ScalarType dt, int64_t d) {
  MCHECK(cache.is_cuda() && cache.scalar_type() == dt && cache.is_contiguous() && cache.dim() == 4 && cache.size(1) == 1 &&
             cache.size(2) == PAGE_TOK && cache.size(3) == d,
         "the latent cache must be [pages, 1, 64, latent + rotated dims] of the activations' dtype");
}

void latent_kv_store(const at::Tensor& P, int64_t ckv_off, int64_t R, int64_t dr, const at::Tensor& kv_norm, int64_t q_off,
                     int64_t q_rank, const c10::optional<at::Tensor>& q_norm, double eps, int64_t rot, bool inter,
                     const at::Tensor& pos, const at::Tensor& cos_sin, const at::Tensor& slots, at::Tensor& cache,
                     const c10::optional<at::Tensor>& qa) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0) return;
  MCHECK(R >= 1 && dr >= 0 && q_rank >= 0, "bad sizes");
  cols_ok(P, ckv_off, R + dr, "kv latent");
  check_rope(pos, cos_sin, T, rot, dr);
  f32c(kv_norm, "kv_norm");
  MCHECK(kv_norm.numel() == R, "kv_norm must hold one weight per latent dim");
  MCHECK(slots.is_cuda() && slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.numel() == T,
         "slots must hold one entry per token");
  MCHECK(is_act(cache), "cache must be bf16 / fp32");
  check_latent_cache(cache, cache.scalar_type(), R + dr);
  const float* qn = nullptr;
  void* qap = nullptr;
  int ldqa = 0;
  if (q_rank > 0) {
    cols_ok(P, q_off, q_rank, "query latent");
    MCHECK(q_norm.has_value() && qa.has_value(), "a query latent needs its norm weight and an output");
    f32c(*q_norm, "q_norm");
    MCHECK(q_norm->numel() == q_rank && qa->scalar_type() == cache.scalar_type(), "q_norm / qa do not fit");
    ldqa = act_ld_min(*qa, T, q_rank, "qa");
    qn = q_norm->data_ptr<float>();
    qap = qa->data_ptr();
  }
  // positions and slots are checked on the host by their producer (the block manager hands out slots < pages * 64
  // and the runner bounds positions by the table's rows)
  if (cache.scalar_type() == at::kBFloat16)
    latent_kv_store_k<uint16_t><<<T, 256, 0, stream()>>>(
        P.data_ptr<float>(), ldp, (int)ckv_off, (int)R, (int)dr, kv_norm.data_ptr<float>(), (int)q_off, (int)q_rank, qn,
        (float)eps, (int)rot, (int)inter, pos.data_ptr<int>(), cos_sin.data_ptr<float>(), slots.data_ptr<int64_t>(),
        (uint16_t*)cache.data_ptr(), (uint16_t*)qap, ldqa);
  else
    latent_kv_store_k<float><<<T, 256, 0, stream()>>>(
        P.data_ptr<float>(), ldp, (int)ckv_off, (int)R, (int)dr, kv_norm.data_ptr<float>(), (int)q_off, (int)q_rank, qn,
        (float)eps, (int)rot, (int)inter, pos.data_ptr<int>(), cos_sin.data_ptr<float>(), slots.data_ptr<int64_t>(),
        cache.data_ptr<float>(), (float*)qap, ldqa);
}

void latent_q_rope(const at::Tensor& Q, int64_t q_off, int64_t H, int64_t dn, int64_t dr, int64_t rot, bool inter,
                   const at::Tensor& pos, const at::Tensor& cos_sin, at::Tensor& qn, at::Tensor& qpe) {
  const int ldq = ld_of(Q, "Q");
  const int64_t T = Q.size(0);
  if (T == 0) return;
  MCHECK(H >= 1 && dn >= 0 && dr >= 0 && dn + dr >= 1, "bad sizes");
  cols_ok(Q, q_off, H * (dn + dr), "queries");
  check_rope(pos, cos_sin, T, rot, dr);
  MCHECK(qn.is_cuda() && is_act(qn) && qn.is_contiguous() && qn.numel() == H * T * dn, "qn must be [H, T, dn]");
  MCHECK(qpe.is_cuda() && qpe.scalar_type() == qn.scalar_type() && qpe.is_contiguous() && qpe.numel() == T * H * dr,
         "qpe must be [T, H, dr] of qn's dtype");
  if (qn.scalar_type() == at::kBFloat16)
    latent_q_rope_k<uint16_t><<<T, 256, 0, stream()>>>(Q.data_ptr<float>(), ldq, (int)q_off, (int)T, (int)H, (int)dn, (int)dr,
                                                       (int)rot, (int)inter, pos.data_ptr<int>(), cos_sin.data_ptr<float>(),
                                                       (uint16_t*)qn.data_ptr(), (uint16_t*)qpe.data_ptr());
  else
    latent_q_rope_k<float><<<T, 256, 0, stream()>>>(Q.data_ptr<float>(), ldq, (int)q_off, (int)T, (int)H, (int)dn, (int)dr,
                                                    (int)rot, (int)inter, pos.data_ptr<int>(), cos_sin.data_ptr<float>(),
                                                    qn.data_ptr<float>(), qpe.data_ptr<float>());
}

template <typename AT, int REP, int NC>
void launch_latt(dim3 grid, size_t lds, const at::Tensor& q_lat, const at::Tensor& q_pe, const at::Tensor& cache,
                 const at::Tensor& bt, const at::Tensor& cu_q, const at::Tensor& ctx, const float* sink, float scale,
                 int window, at::Tensor& out, int H, int R, int dr) {
  auto kern = latent_attn_k<AT, REP, NC>;
  if (lds > 64 * 1024) {
    static bool attr = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
    (void)attr;
  }
  kern<<<grid, 64 * LATT_WAVES, lds, stream()>>>(
      (const AT*)q_lat.data_ptr(), (const AT*)q_pe.data_ptr(), (const AT*)cache.data_ptr(), bt.data_ptr<int>(), (int)bt.size(1),
      cu_q.data_ptr<int>(), ctx.data_ptr<int>(), (int)ctx.numel(), (int)q_lat.size(1), sink, scale, window,
      (AT*)out.data_ptr(), H, R, dr);
}

template <int NV, bool DEC>
void launch_latt_mfma(dim3 grid, size_t lds, const at::Tensor& q_lat, const at::Tensor& q_pe, const at::Tensor& cache,
                      const at::Tensor& bt, const at::Tensor& cu_q, const at::Tensor& ctx, const float* sink, float scale,
                      int window, at::Tensor& out, float* part, int nsplit, int H, int R, int dr) {
  auto kern = latent_attn_mfma_k<NV, DEC>;
  if (lds > 64 * 1024) {
    static bool attr = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
    (void)attr;
  }
  kern<<<grid, 256, lds, stream()>>>(
      (const uint16_t*)q_lat.data_ptr(), (const uint16_t*)q_pe.data_ptr(), (const uint16_t*)cache.data_ptr(),
      bt.data_ptr<int>(), (int)bt.size(1), cu_q.data_ptr<int>(), ctx.data_ptr<int>(), (int)ctx.numel(), (int)q_lat.size(1),
      sink, scale * LOG2E_F, window, (uint16_t*)out.data_ptr(), part, nsplit, H, R, dr);
}

void latent_attn(const at::Tensor& q_lat, const at::Tensor& q_pe, const at::Tensor& cache, const at::Tensor& block_tables,
                 const at::Tensor& cu_q, const at::Tensor& ctx_lens, const c10::optional<at::Tensor>& sink, double scale,
                 int64_t window, at::Tensor& out, int64_t max_qlen) {
  MCHECK(q_lat.is_cuda() && is_act(q_lat) && q_lat.is_contiguous() && q_lat.dim() == 3, "q_lat must be [H, T, R] bf16 / fp32");
  const int64_t H = q_lat.size(0), T = q_lat.size(1), R = q_lat.size(2), B = ctx_lens.numel();
  if (T == 0) return;
  const auto dt = q_lat.scalar_type();
  MCHECK(q_pe.is_cuda() && q_pe.scalar_type() == dt && q_pe.is_contiguous() && q_pe.dim() == 3 && q_pe.size(0) == T &&
             q_pe.size(1) == H,
         "q_pe must be [T, H, dr] of q_lat's dtype");
  const int64_t dr = q_pe.size(2);
  MCHECK(R >= 1 && R <= 512 && dr >= 0 && dr <= 256 && window >= 0, "latent size (at most 512) / rotated dims (at most 256)");
  check_latent_cache(cache, dt, R + dr);
  MCHECK(out.is_cuda() && out.scalar_type() == dt && out.is_contiguous() && out.dim() == 3 && out.size(0) == H &&
             out.size(1) == T && out.size(2) == R,
         "out must be [H, T, R] of q_lat's dtype");
  i32c(block_tables, "block_tables");
  i32c(cu_q, "cu_q");
  i32c(ctx_lens, "ctx_lens");
  MCHECK(block_tables.dim() == 2 && block_tables.size(0) == B && cu_q.numel() == B + 1 && B >= 1, "step tensors do not fit the batch");
  const float* sp = nullptr;
  if (sink.has_value()) {
    f32c(*sink, "sink");
    MCHECK(sink->numel() == H, "one sink per head");
    sp = sink->data_ptr<float>();
  }
  const int d = (int)(R + dr);
  // (block tables, cu_q and ctx_lens come from the runner: tables cover ctx_lens, cu_q[B] == T)
  // matrix-core kernels (bf16, sizes in whole MFMA tiles): prompt portions of 16 tokens and more, and steps of single
  // tokens (a workgroup per token, block of 16 heads and share of the pages; the shares are merged afterwards)
  if (LATT_MFMA && dt == at::kBFloat16 && (max_qlen >= 16 || max_qlen == 1) && R % 16 == 0 && dr % 8 == 0 && R <= 256) {
    const int nv = (int)(R / 16), nq = (d + 31) / 32;
    const int NVT = (nv <= 4 && nq <= 4) ? 4 : ((nv <= 8 && nq <= 6) ? 8 : 16);
    const bool dec = max_qlen == 1;
    const size_t lds = (size_t)(dec ? 144 : 192) * ((NVT / 2 + 2) * 32 + LM_PAD) * 2;
    if (nq <= NVT / 2 + 2 && lds <= 160 * 1024 && (!dec || T == B)) {
      dim3 grid((unsigned)((max_qlen + 63) / 64), (unsigned)B, (unsigned)H);
      int nsplit = 1;
      float* part = nullptr;
      at::Tensor ws;
      if (dec) {
        const int64_t hb = (H + 15) / 16, units = T * hb;
        int64_t pages = block_tables.size(1);
        if (window > 0) pages = std::min<int64_t>(pages, window / PAGE_TOK + 2);
        nsplit = (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(pages, 64), (256 + units - 1) / units));
        if (nsplit > 1) {
          ws = at::empty({T * H * nsplit * (2 + R)}, q_lat.options().dtype(at::kFloat));
          part = ws.data_ptr<float>();
        }
        grid = dim3((unsigned)nsplit, (unsigned)hb, (unsigned)T);
      }
#define XOT_LM(NV, DEC) launch_latt_mfma<NV, DEC>(grid, lds, q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, sp, (float)scale, (int)window, out, part, nsplit, (int)H, (int)R, (int)dr)
      if (dec) {
        if (NVT == 4) XOT_LM(4, true);
        else if (NVT == 8) XOT_LM(8, true);
        else XOT_LM(16, true);
        if (nsplit > 1)
          latent_attn_merge_k<<<(unsigned)(T * H), 256, 0, stream()>>>(part, nsplit, (int)T, (int)H, (int)R, (uint16_t*)out.data_ptr());
      } else {
        if (NVT == 4) XOT_LM(4, false);
        else if (NVT == 8) XOT_LM(8, false);
        else XOT_LM(16, false);
      }
#undef XOT_LM
      return;
    }
  }
  // heads per workgroup: the fewest idle head slots, the larger group on a tie, within the LDS budget
  const int NC = R <= 128 ? 2 : (R <= 256 ? 4 : 8);
  int rep = 0;
  size_t lds = 0;
  for (int r : {8, 4, 2}) {
    const size_t need = ((size_t)r * d + (size_t)LATT_WAVES * r * LATT_TILE + (size_t)LATT_WAVES * r * (2 + R)) * 4;
    if (need > 160 * 1024) continue;
    const int64_t slots = (H + r - 1) / r * r;
    if (rep == 0 || slots < (H + rep - 1) / rep * rep) {
      rep = r;
      lds = need;
    }
  }
  MCHECK(rep > 0, "latent attention: sizes exceed the LDS budget");
  const dim3 grid((unsigned)T, (unsigned)((H + rep - 1) / rep));
#define XOT_LA(AT, REP, NCC) launch_latt<AT, REP, NCC>(grid, lds, q_lat, q_pe, cache, block_tables, cu_q, ctx_lens, sp, (float)scale, (int)window, out, (int)H, (int)R, (int)dr)
#define XOT_LA_NC(AT, REP)                 \
  do {                                     \
    if (NC == 2) XOT_LA(AT, REP, 2);       \
    else if (NC == 4) XOT_LA(AT, REP, 4);  \
    else XOT_LA(AT, REP, 8);               \
  } while (0)
#define XOT_LA_REP(AT)                     \
  do {                                     \
    if (rep == 8) XOT_LA_NC(AT, 8);        \
    else if (rep == 4) XOT_LA_NC(AT, 4);   \
    else XOT_LA_NC(AT, 2);                 \
  } while (0)
  if (dt == at::kBFloat16) XOT_LA_REP(uint16_t);
  else XOT_LA_REP(float);
#undef XOT_LA_REP
#undef XOT_LA_NC
#undef XOT_LA
}

void latent_out_gate(const at::Tensor& o, const c10::optional<at::Tensor>& P, int64_t g_off, int64_t gate, at::Tensor& out) {
  MCHECK(o.is_cuda() && is_act(o) && o.is_contiguous() && o.dim() == 3, "o must be [H, T, dv] bf16 / fp32");
  const int64_t H = o.size(0), T = o.size(1), dv = o.size(2);
  if (T == 0) return;
  MCHECK(out.scalar_type() == o.scalar_type(), "out must have o's dtype");
  const int ldo = act_ld_min(out, T, H * dv, "out");
  const float* pp = nullptr;
  int ldp = 0;
  MCHECK(gate >= 0 && gate <= 2, "gate: 0 none, 1 per element, 2 per head");
  if (gate) {
    MCHECK(P.has_value(), "a gate needs the projection that holds it");
    ldp = ld_of(*P, "P");
    MCHECK(P->size(0) == T, "P must have T rows");
    cols_ok(*P, g_off, gate == 1 ? H * dv : H, "output gate");
    pp = P->data_ptr<float>();
  }
  if (o.scalar_type() == at::kBFloat16)
    latent_out_gate_k<uint16_t><<<T, 256, 0, stream()>>>((const uint16_t*)o.data_ptr(), pp, ldp, (int)g_off, (int)gate, (int)T,
                                                         (int)H, (int)dv, (uint16_t*)out.data_ptr(), ldo);
  else
    latent_out_gate_k<float><<<T, 256, 0, stream()>>>(o.data_ptr<float>(), pp, ldp, (int)g_off, (int)gate, (int)T, (int)H,
                                                      (int)dv, out.data_ptr<float>(), ldo);
}

void glu_act(const at::Tensor& P, int64_t gate_off, int64_t up_off, int64_t F, bool clamped, double limit, at::Tensor& out) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0 || F == 0) return;
  cols_ok(P, gate_off, F, "gate");
  cols_ok(P, up_off, F, "up");
  const int ldo = act_ld_min(out, T, F, "out");
  const int64_t total = T * F;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (out.scalar_type() == at::kBFloat16)
    glu_act_k<uint16_t><<<blocks, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)gate_off, (int)up_off, (int)F, (int)clamped,
                                                      (float)limit, (uint16_t*)out.data_ptr(), ldo, total);
  else
    glu_act_k<float><<<blocks, 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)gate_off, (int)up_off, (int)F, (int)clamped,
                                                   (float)limit, out.data_ptr<float>(), ldo, total);
}

}  // namespace

void bind_latent(pybind11::module& m) {
  m.def("sandwich_add_norm", &sandwich_add_norm);
  m.def("latent_kv_store", &latent_kv_store);
  m.def("latent_q_rope", &latent_q_rope);
  m.def("latent_attn", &latent_attn);
  m.def("latent_out_gate", &latent_out_gate);
  m.def("glu_act", &glu_act);
}

}  // namespace xot
