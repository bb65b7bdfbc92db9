// Element-wise and per-head stages around the attention and recurrence kernels of layer-norm sandwich blocks (gfx950):
//
//   diff_attn_out      differential attention's combination: a_1 - lam a_2, per-head RMS division, scale, per-head gate
//   sigmoid_gate_mul   a * sigmoid(gate), element by element
//   silu_cols          silu of a column range of a fused projection, fp32 (lightning attention's q | k | v)
//   mlstm_gates        the mlstm's capped gates, the running maximum's scan over a step's tokens, decay and input scale
//   gated_group_norm   (stabilised division,) RMS norm in equal groups, weight, sigmoid gate
//   pair_norm_mean     the mean of two RMS-normed, weighted rows
//
// P is a fused projection's fp32 output [T, ldp]; "column offset" arguments address its slices.  Everything here is
// computed in fp32; outputs that feed the next GEMM (AT) are bf16 or fp32.
#include "mixer_util.h"

namespace xot {
namespace {
using namespace mix;

// ------------------------------------------------------------------ differential attention: combine, norm, gate
// a [T, 2 H dv]: heads ordered (kv head g, map m, head r of the group); head h = g rep + r.  Workgroup = (token, head).
template <typename AT>
__global__ void diff_attn_out_k(const float* __restrict__ a, const float* __restrict__ P, int ldp, int g_off, int H, int rep,
                                int dv, float lam, float post, float eps, AT* __restrict__ out, int ldo) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / rep, r = h - g * rep;
  const float* a1 = a + ((int64_t)t * 2 * H + (g * 2 + 0) * rep + r) * dv;
  const float* a2 = a + ((int64_t)t * 2 * H + (g * 2 + 1) * rep + r) * dv;
  float ss = 0.0f;
  for (int i = lane; i < dv; i += 64) {
    const float o = a1[i] - lam * a2[i];
    ss += o * o;
  }
  ss = wave_sum(ss);
  const float k = post / sqrtf(ss / (float)dv + eps) * sigmoidf_(P[(int64_t)t * ldp + g_off + h]);
  for (int i = lane; i < dv; i += 64) stf(out + (int64_t)t * ldo + h * dv + i, (a1[i] - lam * a2[i]) * k);
}

// (a and out may be the same rows: every element is read and written by one thread)
template <typename IT, typename AT>
__global__ void sigmoid_gate_mul_k(const IT* a, int lda, const float* __restrict__ P, int ldp, int g_off, int n, AT* out,
                                   int ldo, int64_t total) {
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = e / n;
    const int i = (int)(e - t * n);
    stf(out + t * ldo + i, ldf(a + t * lda + i) * sigmoidf_(P[t * ldp + g_off + i]));
  }
}

__global__ void silu_cols_k(const float* __restrict__ P, int ldp, int off, int n, float* __restrict__ out, int64_t total) {
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = e / n;
    out[e] = siluf_(P[t * ldp + off + (int)(e - t * n)]);
  }
}

// ------------------------------------------------------------------ mlstm gates and the running maximum
// One wave per (sequence, head).  The lanes take 64 consecutive tokens: each computes its token's capped gates, then
// the maximum m_t = max(f_t + m_(t-1), i_t) runs through the 64 tokens in order (the gates broadcast lane by lane), every
// lane keeping the maximum before and after its own token; decay, input scale and m_t are written in parallel.
__global__ __launch_bounds__(64) void mlstm_gates_k(const float* __restrict__ P, int ldp, int i_off, int f_off,
                                                    const float* __restrict__ gate_b, float cap, float* __restrict__ mstate,
                                                    const int* __restrict__ state_slots, const int* __restrict__ cu_q, int H,
                                                    float* __restrict__ decay, float* __restrict__ inscale,
                                                    float* __restrict__ mout) {
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int slot = state_slots[b];
  const int t0 = cu_q[b], n = cu_q[b + 1] - t0;
  if (slot < 0 || n <= 0) return;
  float m = mstate[(int64_t)slot * H + h];
  const float bi = gate_b[h], bf = gate_b[H + h], inv = 1.0f / cap;
  for (int tb = 0; tb < n; tb += 64) {
    const int nt = min(64, n - tb);
    float gi = 0.0f, gf = 0.0f;
    if (lane < nt) {
      const float* row = P + (int64_t)(t0 + tb + lane) * ldp;
      gi = cap * tanhf((row[i_off + h] + bi) * inv);
      gf = logsigmoidf_(cap * tanhf((row[f_off + h] + bf) * inv));
    }
    float before = 0.0f, after = 0.0f;
    for (int j = 0; j < nt; ++j) {
      const float fj = __shfl(gf, j, 64), ij = __shfl(gi, j, 64);
      const float mn = fmaxf(fj + m, ij);
      if (lane == j) {
        before = m;
        after = mn;
      }
      m = mn;
    }
    if (lane < nt) {
      const int64_t o = (int64_t)(t0 + tb + lane) * H + h;
      decay[o] = expf(gf + before - after);
      inscale[o] = expf(gi - after);
      mout[o] = after;
    }
  }
  if (lane == 0) mstate[(int64_t)slot * H + h] = m;
}

// ------------------------------------------------------------------ (stabilised division,) grouped RMS norm, weight, sigmoid gate
// o [T, groups * (gs + extra)]; extra = 1: each group's last channel is a normaliser n and the values are divided by
// max(|n|, exp(-m[t, group])) + 1e-6 first.  Workgroup = (token, group).
template <typename AT>
__global__ void gated_group_norm_k(const float* __restrict__ o, const float* __restrict__ m, const float* __restrict__ w,
                                   const float* __restrict__ P, int ldp, int g_off, int groups, int gs, float eps,
                                   AT* __restrict__ out, int ldo) {
  __shared__ float red[16];
  const int t = blockIdx.x, g = blockIdx.y;
  const int extra = m ? 1 : 0;
  const float* x = o + ((int64_t)t * groups + g) * (gs + extra);
  float div = 1.0f;
  if (m) div = 1.0f / (fmaxf(fabsf(x[gs]), expf(-m[(int64_t)t * groups + g])) + 1e-6f);
  float ss = 0.0f;
  for (int i = threadIdx.x; i < gs; i += blockDim.x) {
    const float v = x[i] * div;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float k = div / sqrtf(ss / (float)gs + eps);
  for (int i = threadIdx.x; i < gs; i += blockDim.x) {
    const int c = g * gs + i;
    stf(out + (int64_t)t * ldo + c, x[i] * k * w[c] * sigmoidf_(P[(int64_t)t * ldp + g_off + c]));
  }
}

// Groups of at most 64 GR values: a wave per (token, group), four groups a workgroup, the group's values in registers.
template <typename AT, int GR>
__global__ __launch_bounds__(256) void gated_group_norm_wave_k(const float* __restrict__ o, const float* __restrict__ m,
                                                               const float* __restrict__ w, const float* __restrict__ P,
                                                               int ldp, int g_off, int groups, int gs, float eps,
                                                               AT* __restrict__ out, int ldo) {
  const int t = blockIdx.x, g = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (g >= groups) return;  // (wave-uniform; no workgroup barrier below)
  const int extra = m ? 1 : 0;
  const float* x = o + ((int64_t)t * groups + g) * (gs + extra);
  float div = 1.0f;
  if (m) div = 1.0f / (fmaxf(fabsf(x[gs]), expf(-m[(int64_t)t * groups + g])) + 1e-6f);
  float v[GR];
  float ss = 0.0f;
#pragma unroll
  for (int r = 0; r < GR; ++r) {
    const int i = lane + 64 * r;
    v[r] = i < gs ? x[i] * div : 0.0f;
    ss += v[r] * v[r];
  }
  const float k = 1.0f / sqrtf(wave_sum(ss) / (float)gs + eps);
#pragma unroll
  for (int r = 0; r < GR; ++r) {
    const int i = lane + 64 * r, c = g * gs + i;
    if (i < gs) stf(out + (int64_t)t * ldo + c, v[r] * k * w[c] * sigmoidf_(P[(int64_t)t * ldp + g_off + c]));
  }
}

// ------------------------------------------------------------------ mean of two normed rows
__global__ __launch_bounds__(256) void pair_norm_mean_k(const float* __restrict__ y1, int ld1, const float* __restrict__ y2,
                                                        int ld2, const float* __restrict__ w, float eps,
                                                        float* __restrict__ out, int D) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float *a = y1 + t * ld1, *b = y2 + t * ld2;
  float sa = 0.0f, sb = 0.0f;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    sa += a[i] * a[i];
    sb += b[i] * b[i];
  }
  sa = block_sum(sa, red);
  sb = block_sum(sb, red);
  const float ka = 0.5f / sqrtf(sa / (float)D + eps), kb = 0.5f / sqrtf(sb / (float)D + eps);
  for (int i = threadIdx.x; i < D; i += blockDim.x) out[t * D + i] = a[i] * ka * w[i] + b[i] * kb * w[D + i];
}

// ------------------------------------------------------------------ host side
int grid_for(int64_t total) { return (int)std::min<int64_t>((total + 255) / 256, 65535); }

void diff_attn_out(const at::Tensor& a, const at::Tensor& P, int64_t g_off, int64_t H, int64_t G, double lam, double post,
                   double eps, at::Tensor& out) {
  f32c(a, "a");
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0) return;
  MCHECK(H > 0 && G > 0 && H % G == 0 && a.dim() == 2 && a.size(0) == T && a.size(1) % (2 * H) == 0,
         "a must be [T, 2 H dv] with H a multiple of the kv heads");
  const int64_t dv = a.size(1) / (2 * H);
  cols_ok(P, g_off, H, "gate");
  const int ldo = act_ld_min(out, T, H * dv, "out");
  const dim3 grid((unsigned)T, (unsigned)H);
  if (out.scalar_type() == at::kBFloat16)
    diff_attn_out_k<uint16_t><<<grid, 64, 0, stream()>>>(a.data_ptr<float>(), P.data_ptr<float>(), ldp, (int)g_off, (int)H,
                                                         (int)(H / G), (int)dv, (float)lam, (float)post, (float)eps,
                                                         (uint16_t*)out.data_ptr(), ldo);
  else
    diff_attn_out_k<float><<<grid, 64, 0, stream()>>>(a.data_ptr<float>(), P.data_ptr<float>(), ldp, (int)g_off, (int)H,
                                                      (int)(H / G), (int)dv, (float)lam, (float)post, (float)eps,
                                                      out.data_ptr<float>(), ldo);
}

// a [T, n]: fp32, or rows of out's dtype (also out's own rows: the gate applied in place)
void sigmoid_gate_mul(const at::Tensor& a, const at::Tensor& P, int64_t g_off, at::Tensor& out) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0) return;
  MCHECK(a.is_cuda() && a.dim() == 2 && a.size(0) == T && a.stride(1) == 1 &&
             (a.scalar_type() == at::kFloat || a.scalar_type() == out.scalar_type()),
         "a must be [T, n] rows, fp32 or of out's dtype");
  const int64_t n = a.size(1);
  const int lda = (int)a.stride(0);
  cols_ok(P, g_off, n, "gate");
  const int ldo = act_ld_min(out, T, n, "out");
  const int grid = grid_for(T * n);
  if (out.scalar_type() == at::kBFloat16 && a.scalar_type() == at::kFloat)
    sigmoid_gate_mul_k<float, uint16_t><<<grid, 256, 0, stream()>>>(a.data_ptr<float>(), lda, P.data_ptr<float>(), ldp, (int)g_off,
                                                                    (int)n, (uint16_t*)out.data_ptr(), ldo, T * n);
  else if (out.scalar_type() == at::kBFloat16)
    sigmoid_gate_mul_k<uint16_t, uint16_t><<<grid, 256, 0, stream()>>>((const uint16_t*)a.data_ptr(), lda, P.data_ptr<float>(), ldp,
                                                                       (int)g_off, (int)n, (uint16_t*)out.data_ptr(), ldo, T * n);
  else
    sigmoid_gate_mul_k<float, float><<<grid, 256, 0, stream()>>>(a.data_ptr<float>(), lda, P.data_ptr<float>(), ldp, (int)g_off,
                                                                 (int)n, out.data_ptr<float>(), ldo, T * n);
}

void silu_cols(const at::Tensor& P, int64_t off, int64_t n, at::Tensor& out) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0);
  if (T == 0 || n == 0) return;
  cols_ok(P, off, n, "columns");
  f32c(out, "out");
  MCHECK(out.numel() == T * n, "out must be [T, n]");
  silu_cols_k<<<grid_for(T * n), 256, 0, stream()>>>(P.data_ptr<float>(), ldp, (int)off, (int)n, out.data_ptr<float>(), T * n);
}

void mlstm_gates(const at::Tensor& P, int64_t i_off, int64_t f_off, const at::Tensor& gate_b, double cap, at::Tensor& mstate,
                 const at::Tensor& state_slots, const at::Tensor& cu_q, at::Tensor& decay, at::Tensor& inscale,
                 at::Tensor& mout) {
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0), B = state_slots.numel();
  if (T == 0 || B == 0) return;
  f32c(gate_b, "gate_b");
  f32c(mstate, "mstate");
  f32c(decay, "decay");
  f32c(inscale, "inscale");
  f32c(mout, "mout");
  i32c(state_slots, "state_slots");
  i32c(cu_q, "cu_q");
  MCHECK(mstate.dim() == 2, "mstate must be [slots, H]");
  const int64_t H = mstate.size(1);
  MCHECK(cap > 0.0 && gate_b.numel() == 2 * H && decay.numel() == T * H && inscale.numel() == T * H && mout.numel() == T * H &&
             cu_q.numel() == B + 1,
         "mlstm_gates: shape mismatch");
  cols_ok(P, i_off, H, "input gate");
  cols_ok(P, f_off, H, "forget gate");
  // (state slots are handed out by the slot manager: below mstate's rows)
  mlstm_gates_k<<<dim3((unsigned)B, (unsigned)H), 64, 0, stream()>>>(
      P.data_ptr<float>(), ldp, (int)i_off, (int)f_off, gate_b.data_ptr<float>(), (float)cap, mstate.data_ptr<float>(),
      state_slots.data_ptr<int>(), cu_q.data_ptr<int>(), (int)H, decay.data_ptr<float>(), inscale.data_ptr<float>(),
      mout.data_ptr<float>());
}

void gated_group_norm(const at::Tensor& o, const c10::optional<at::Tensor>& m, const at::Tensor& w, const at::Tensor& P,
                      int64_t g_off, int64_t groups, double eps, at::Tensor& out) {
  f32c(o, "o");
  f32c(w, "w");
  const int ldp = ld_of(P, "P");
  const int64_t T = P.size(0), n = w.numel();
  if (T == 0) return;
  MCHECK(groups > 0 && n % groups == 0, "the weight must hold groups * gs numbers");
  const int64_t gs = n / groups, extra = m.has_value() ? 1 : 0;
  MCHECK(o.numel() == T * groups * (gs + extra), "o must be [T, groups (gs + a normaliser channel when m is given)]");
  const float* mp = nullptr;
  if (m.has_value()) {
    f32c(*m, "m");
    MCHECK(m->numel() == T * groups, "m must be [T, groups]");
    mp = m->data_ptr<float>();
  }
  cols_ok(P, g_off, n, "gate");
  const int ldo = act_ld_min(out, T, n, "out");
#define GGN_ARGS(AT)                                                                                                      \
  o.data_ptr<float>(), mp, w.data_ptr<float>(), P.data_ptr<float>(), ldp, (int)g_off, (int)groups, (int)gs, (float)eps, \
      (AT*)out.data_ptr(), ldo
  const bool bf = out.scalar_type() == at::kBFloat16;
  if (gs <= 512 && groups > 1) {  // a wave per group
    const dim3 grid((unsigned)T, (unsigned)((groups + 3) / 4));
    if (gs <= 128) {
      if (bf) gated_group_norm_wave_k<uint16_t, 2><<<grid, 256, 0, stream()>>>(GGN_ARGS(uint16_t));
      else gated_group_norm_wave_k<float, 2><<<grid, 256, 0, stream()>>>(GGN_ARGS(float));
    } else {
      if (bf) gated_group_norm_wave_k<uint16_t, 8><<<grid, 256, 0, stream()>>>(GGN_ARGS(uint16_t));
      else gated_group_norm_wave_k<float, 8><<<grid, 256, 0, stream()>>>(GGN_ARGS(float));
    }
    return;
  }
  const dim3 grid((unsigned)T, (unsigned)groups);
  const int threads = (int)std::min<int64_t>(256, (gs + 63) / 64 * 64);
  if (bf) gated_group_norm_k<uint16_t><<<grid, threads, 0, stream()>>>(GGN_ARGS(uint16_t));
  else gated_group_norm_k<float><<<grid, threads, 0, stream()>>>(GGN_ARGS(float));
#undef GGN_ARGS
}

void pair_norm_mean(const at::Tensor& y1, const at::Tensor& y2, const at::Tensor& w, double eps, at::Tensor& out) {
  const int ld1 = ld_of(y1, "y1"), ld2 = ld_of(y2, "y2");
  f32c(w, "w");
  f32c(out, "out");
  MCHECK(out.dim() == 2, "out must be [T, D]");
  const int64_t T = out.size(0), D = out.size(1);
  if (T == 0) return;
  MCHECK(y1.size(0) == T && y2.size(0) == T && y1.size(1) >= D && y2.size(1) >= D && w.numel() == 2 * D,
         "pair_norm_mean: shape mismatch");
  pair_norm_mean_k<<<T, 256, 0, stream()>>>(y1.data_ptr<float>(), ld1, y2.data_ptr<float>(), ld2, w.data_ptr<float>(), (float)eps,
                                            out.data_ptr<float>(), (int)D);
}

}  // namespace

void bind_recurrent_gates(pybind11::module& m) {
  m.def("diff_attn_out", &diff_attn_out);
  m.def("sigmoid_gate_mul", &sigmoid_gate_mul);
  m.def("silu_cols", &silu_cols);
  m.def("mlstm_gates", &mlstm_gates);
  m.def("gated_group_norm", &gated_group_norm);
  m.def("pair_norm_mean", &pair_norm_mean);
}

}  // namespace xot
