// stack_rec.h — row-wise kernels of the layered designs whose layers run a mixer and a feed-forward side by side behind ONE norm, and whose mixers keep
// a decaying matrix state per head (Vitudra).  Same conventions as stack.h / stack_seq.h: a step's T tokens are the concatenated entries of a ragged
// batch (StepMeta), all arithmetic here is fp32, every reduction has a fixed order.
//   offset_norm_kernel      rows / sqrt(mean(row^2) + eps) * (offset + w): an RMS norm whose weight is stored as its distance from `offset`
//   token_shift_kernel      the n mixes h + (h_before - h) * mu_s of a token-shift layer, and the slot's last row
//   delta_prep_kernel       causal depth-wise convolution + silu on the q | k | v projections of a gated-delta-rule layer (tails per slot), unit q and k per
//                           head, beta = sigmoid, decay = exp(-exp(A_log) * softplus(a + dt_bias))
//   rec_scan_kernel         the recurrence over an entry's tokens with the head's matrix state in registers:
//                             REC_WKV     o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T
//                             REC_DELTA   S <- g S;  S += k (beta (v - S^T k))^T;  o = S^T q
// A sequence whose first token has position 0 starts from zero state whatever its slot held.
#pragma once
#include "stack.h"

namespace tgx {

// out[i] = x[rows ? rows[i] : i] / sqrt(mean(row^2) + eps) * (offset + w)
__global__ __launch_bounds__(256) void offset_norm_kernel(const float* x, const int* rows, const float* w, float offset, float* out, int W, float eps) {
  __shared__ float s4[4];
  const float* xr = x + (size_t)(rows ? rows[blockIdx.x] : blockIdx.x) * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) ss = fmaf(xr[c], xr[c], ss);
  ss = block_sum_256(ss, s4);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) out[(size_t)blockIdx.x * W + c] = xr[c] * r * (offset + w[c]);
}

// ---- token shift.  One workgroup per token: out[t][s] = h_t + (h_(t-1) - h_t) * mu[s] for the n mixes; h_(t-1) is the row before in the entry, the
// slot's kept row for an entry's first token, zero at position 0.  The kept row is double-buffered with the slot's step parity (the entry's last token
// writes buffer par ^ 1 while its first reads buffer par).
struct TokenShiftArgs {
  const float* h;        // [T][W]
  const float* mu;       // [n][W]
  float* out;            // [T][n][W]
  float* state;          // [2][slots][W]
  size_t state_buf;
  int W, n;
};
__global__ __launch_bounds__(256) void token_shift_kernel(StepMeta m, TokenShiftArgs a) {
  const int t = blockIdx.x, i = m.tok_idx[t], cnt = m.tok_cnt[t], pos = m.tok_pos[t], row = m.tok_row[t], par = m.tok_par[t];
  const float* cur = a.h + (size_t)t * a.W;
  const float* before = i > 0 ? cur - a.W : a.state + (size_t)par * a.state_buf + (size_t)row * a.W;
  const bool none = pos == 0;
  float* keep = i == cnt - 1 ? a.state + (size_t)(par ^ 1) * a.state_buf + (size_t)row * a.W : nullptr;
  for (int c = threadIdx.x; c < a.W; c += 256) {
    const float x = cur[c], d = (none ? 0.f : before[c]) - x;
    for (int s = 0; s < a.n; s++) a.out[((size_t)t * a.n + s) * a.W + c] = fmaf(d, a.mu[(size_t)s * a.W + c], x);
    if (keep) keep[c] = x;
  }
}

// ---- inputs of a gated-delta-rule layer.  One workgroup per token.  proj row = [.. | q (G D) | k (G D) | v (H E) | b (H) | a (H) | ..] from column col0;
// the C = 2 G D + H E convolved channels take taps weights each (last = the current token's); the taps - 1 rows before come from the step's own rows, the
// slot's tails (raw projections, double-buffered by step parity like the other per-slot rows) or are zero before the sequence's start.
// out row = [q | k | v | beta | decay]: q, k unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q times q_scale.
struct DeltaPrepArgs {
  const float* proj; long long ldp; int col0;
  const float* cw;       // [C][taps]
  const float* a_log;    // [H]
  const float* dt_bias;  // [H]
  float* out; long long ldo;
  float* state;          // [2][slots][taps - 1][C] (nullptr when taps == 1)
  size_t state_buf;
  int heads, kv_heads, dim, vdim, taps;
  float q_scale, unit_eps;
};
__global__ __launch_bounds__(256) void delta_prep_kernel(StepMeta m, DeltaPrepArgs a) {
  extern __shared__ float s_c[];      // [C] the token's convolved, activated channels
  const int t = blockIdx.x, i = m.tok_idx[t], cnt = m.tok_cnt[t], pos = m.tok_pos[t], row = m.tok_row[t], par = m.tok_par[t];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int GD = a.kv_heads * a.dim, C = 2 * GD + a.heads * a.vdim, nb = a.taps - 1;
  const float* __restrict__ pr = a.proj + (size_t)t * a.ldp + a.col0;
  const float* __restrict__ st_old = a.state ? a.state + (size_t)par * a.state_buf + (size_t)row * nb * C : nullptr;
  float* __restrict__ st_new = a.state ? a.state + (size_t)(par ^ 1) * a.state_buf + (size_t)row * nb * C : nullptr;
  float* __restrict__ o = a.out + (size_t)t * a.ldo;
  for (int c = threadIdx.x; c < C; c += 256) {
    const float x0 = pr[c];
    float acc = a.cw[(size_t)c * a.taps + nb] * x0;
    for (int d = 1; d <= nb; d++) {                        // the row d positions back
      float xv = 0.f;
      if (d <= i) xv = pr[c - (long long)d * a.ldp];
      else if (pos - d >= 0) xv = st_old[(size_t)(nb - (d - i)) * C + c];      // tail slot s holds position past - nb + s, past = pos - i
      acc = fmaf(a.cw[(size_t)c * a.taps + nb - d], xv, acc);
    }
    s_c[c] = acc / (1.0f + expf(-acc));
    if (st_new) {
      const int s = nb - (cnt - i);                        // row i of cnt lands in tail slot nb - (cnt - i) ...
      if (s >= 0) st_new[(size_t)s * C + c] = x0;
      if (i == 0)                                          // ... and an entry shorter than the tails keeps the end of the old ones
        for (int k = 0; k + cnt < nb; k++) st_new[(size_t)k * C + c] = (pos - (nb - cnt - k) >= 0) ? st_old[(size_t)(k + cnt) * C + c] : 0.f;
    }
  }
  __syncthreads();
  for (int hd = wv; hd < 2 * a.kv_heads; hd += 4) {        // q heads, then k heads: one wave each
    const float* v = s_c + (size_t)hd * a.dim;
    float ss = 0.f;
    for (int c = lane; c < a.dim; c += 64) ss = fmaf(v[c], v[c], ss);
    ss = wave_sum(ss);
    const float r = (hd < a.kv_heads ? a.q_scale : 1.0f) / sqrtf(ss + a.unit_eps);
    for (int c = lane; c < a.dim; c += 64) o[(size_t)hd * a.dim + c] = v[c] * r;
  }
  for (int c = 2 * GD + threadIdx.x; c < C; c += 256) o[c] = s_c[c];
  for (int h = threadIdx.x; h < a.heads; h += 256) {
    const float zb = pr[C + h], za = pr[C + a.heads + h] + a.dt_bias[h];
    const float sp = za > 20.f ? za : log1pf(expf(za));
    o[C + h] = 1.0f / (1.0f + expf(-zb));
    o[C + a.heads + h] = expf(-expf(a.a_log[h]) * sp);
  }
}

// ---- the recurrences.  One workgroup per (entry, head, 64 value columns) walks the entry's tokens in order, TB at a time: the block's per-key-channel
// inputs (three vectors of `dim`) and the workgroup's value columns are staged in LDS, then every lane updates its DPER rows of its column: a wave owns 16
// columns, its lanes = 4 row groups x 16 columns, 4 DPER >= dim.  Sums over the key channels cross the row groups by two lane exchanges.
enum { REC_WKV = 0, REC_DELTA = 1 };
struct RecScanArgs {
  const float* a; long long lda;     // per token and key head [dim]: the read vector (wkv: r, delta: q)
  const float* k; long long ldk;     //                               k
  const float* w; long long ldw;     //                               wkv: the decay per channel
  const float* v; long long ldv;     // per token and head [vdim]
  const float* beta; const float* g; long long ldg;      // delta: per token and head
  const float* u;                    // wkv: [heads][dim] bonus
  float* S;                          // [slots][heads][dim][vdim]
  float* out; long long ldo;         // [T][heads * vdim]
  int heads, kv_heads, dim, vdim;
};
template <int DPER, int KIND>
__global__ __launch_bounds__(256) void rec_scan_kernel(StepMeta m, RecScanArgs a) {
  constexpr int LP = DPER + 4, DP = 4 * DPER, TB = DP <= 128 ? 16 : 8;      // LP: a row group's LDS stride (the groups' reads fall into different banks)
  __shared__ __attribute__((aligned(16))) float s_a[TB][4 * LP], s_k[TB][4 * LP], s_w[KIND == REC_WKV ? TB : 1][4 * LP];
  __shared__ float s_v[TB][64], s_b[TB], s_g[TB];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, rg = lane >> 4, cl = lane & 15;
  const int jl = wv * 16 + cl, j = blockIdx.z * 64 + jl;
  const int start = m.ent_start[e], cnt = m.ent_count[e], row = m.ent_row[e];
  const bool fresh = m.tok_pos[start] == 0;
  const int kh = h / (a.heads / a.kv_heads), d0 = rg * DPER, l0 = rg * LP;
  const bool col = j < a.vdim;
  float* Sg = a.S + ((size_t)row * a.heads + h) * (size_t)a.dim * a.vdim;
  float S[DPER], ub[KIND == REC_WKV ? DPER : 1];
#pragma unroll
  for (int dd = 0; dd < DPER; dd++) {
    const int d = d0 + dd;
    S[dd] = (!fresh && d < a.dim && col) ? Sg[(size_t)d * a.vdim + j] : 0.f;
    if (KIND == REC_WKV) ub[dd] = d < a.dim ? a.u[(size_t)h * a.dim + d] : 0.f;
  }
  for (int t0 = 0; t0 < cnt; t0 += TB) {
    const int nb = min(TB, cnt - t0);
    __syncthreads();                                       // the block before has been read
    for (int i = tid; i < nb * DP; i += 256) {
      const int t = i / DP, d = i - t * DP, at = (d / DPER) * LP + d % DPER;
      const size_t tok = (size_t)(start + t0 + t);
      const bool on = d < a.dim;
      s_a[t][at] = on ? a.a[tok * a.lda + (size_t)kh * a.dim + d] : 0.f;
      s_k[t][at] = on ? a.k[tok * a.ldk + (size_t)kh * a.dim + d] : 0.f;
      if (KIND == REC_WKV) s_w[t][at] = on ? a.w[tok * a.ldw + (size_t)kh * a.dim + d] : 0.f;
    }
    for (int i = tid; i < nb * 64; i += 256) {
      const int t = i >> 6, c = i & 63;
      s_v[t][c] = blockIdx.z * 64 + c < a.vdim ? a.v[(size_t)(start + t0 + t) * a.ldv + (size_t)h * a.vdim + blockIdx.z * 64 + c] : 0.f;
    }
    if (KIND == REC_DELTA && tid < nb) { s_b[tid] = a.beta[(size_t)(start + t0 + tid) * a.ldg + h]; s_g[tid] = a.g[(size_t)(start + t0 + tid) * a.ldg + h]; }
    __syncthreads();
    for (int t = 0; t < nb; t++) {
      const float vj = s_v[t][jl];
      float po = 0.f;
      if (KIND == REC_WKV) {
#pragma unroll
        for (int dd = 0; dd < DPER; dd += 4) {
          const f32x4 r4 = *reinterpret_cast<const f32x4*>(&s_a[t][l0 + dd]), k4 = *reinterpret_cast<const f32x4*>(&s_k[t][l0 + dd]), w4 = *reinterpret_cast<const f32x4*>(&s_w[t][l0 + dd]);
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const float kv = k4[q] * vj;
            po = fmaf(r4[q], fmaf(ub[dd + q], kv, S[dd + q]), po);
            S[dd + q] = fmaf(w4[q], S[dd + q], kv);
          }
        }
      } else {
        const float g = s_g[t];
        float pk = 0.f;
#pragma unroll
        for (int dd = 0; dd < DPER; dd += 4) {
          const f32x4 k4 = *reinterpret_cast<const f32x4*>(&s_k[t][l0 + dd]);
#pragma unroll
          for (int q = 0; q < 4; q++) { S[dd + q] *= g; pk = fmaf(S[dd + q], k4[q], pk); }
        }
        pk += __shfl_xor(pk, 16, 64); pk += __shfl_xor(pk, 32, 64);
        const float uj = s_b[t] * (vj - pk);
#pragma unroll
        for (int dd = 0; dd < DPER; dd += 4) {
          const f32x4 k4 = *reinterpret_cast<const f32x4*>(&s_k[t][l0 + dd]), q4 = *reinterpret_cast<const f32x4*>(&s_a[t][l0 + dd]);
#pragma unroll
          for (int q = 0; q < 4; q++) { S[dd + q] = fmaf(k4[q], uj, S[dd + q]); po = fmaf(S[dd + q], q4[q], po); }
        }
      }
      po += __shfl_xor(po, 16, 64); po += __shfl_xor(po, 32, 64);
      if (rg == 0 && col) a.out[(size_t)(start + t0 + t) * a.ldo + (size_t)h * a.vdim + j] = po;
    }
  }
#pragma unroll
  for (int dd = 0; dd < DPER; dd++) { const int d = d0 + dd; if (d < a.dim && col) Sg[(size_t)d * a.vdim + j] = S[dd]; }
}

}  // namespace tgx
