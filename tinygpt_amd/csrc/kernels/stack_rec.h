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

// ---- token shift.  One thread per (token, channel): out[t][s] = h_t + (h_(t-1) - h_t) * mu[s] for the n mixes; h_(t-1) is the row before in the entry,
// the slot's kept row for an entry's first token, zero at position 0.  The kept row is double-buffered with the slot's step parity (the entry's last
// token writes buffer par ^ 1 while its first reads buffer par).  Grid: (tokens, width / 256).
struct TokenShiftArgs {
  const float* h;        // [T][W]
  const float* mu;       // [n][W]
  float* out;            // [T][n][W]
  float* state;          // [2][slots][W]
  size_t state_buf;
  int W, n;
};
__global__ __launch_bounds__(256) void token_shift_kernel(StepMeta m, TokenShiftArgs a) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.W) return;
  const int i = m.tok_idx[t], cnt = m.tok_cnt[t], pos = m.tok_pos[t], row = m.tok_row[t], par = m.tok_par[t];
  const float* __restrict__ cur = a.h + (size_t)t * a.W;
  const float* __restrict__ before = i > 0 ? cur - a.W : a.state + (size_t)par * a.state_buf + (size_t)row * a.W;
  float* __restrict__ outp = a.out + (size_t)t * a.n * a.W;
  const float x = cur[c], d = (pos == 0 ? 0.f : before[c]) - x;
  for (int s = 0; s < a.n; s++) outp[(size_t)s * a.W + c] = fmaf(d, a.mu[(size_t)s * a.W + c], x);
  if (i == cnt - 1) a.state[(size_t)(par ^ 1) * a.state_buf + (size_t)row * a.W + c] = x;
}

// ---- inputs of a gated-delta-rule layer.  proj row = [.. | q (G D) | k (G D) | v (H E) | b (H) | a (H) | ..] from column col0; the C = 2 G D + H E
// convolved channels take taps weights each (last = the current token's); the taps - 1 rows before come from the step's own rows, the slot's tails (raw
// projections, double-buffered by step parity like the other per-slot rows) or are zero before the sequence's start.
// out row = [q | k | v | beta | decay]: q, k unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q times q_scale.
// Grid: (tokens, 2 G + H + 1): one workgroup per q head, k head (D <= 256 channels, one per thread, and their norm), v head, and one for the H gates.
constexpr int DELTA_MAX_TAPS = 64;      // (bounds the per-slot tails, not the kernel: it loops over the taps)
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
  __shared__ float s4[4];
  const int t = blockIdx.x, u = blockIdx.y, i = m.tok_idx[t], cnt = m.tok_cnt[t], pos = m.tok_pos[t], row = m.tok_row[t], par = m.tok_par[t];
  const int G2 = 2 * a.kv_heads, GD = a.kv_heads * a.dim, C = 2 * GD + a.heads * a.vdim, nb = a.taps - 1;
  const float* __restrict__ pr = a.proj + (size_t)t * a.ldp + a.col0;
  float* __restrict__ o = a.out + (size_t)t * a.ldo;
  if (u == G2 + a.heads) {
    for (int h = threadIdx.x; h < a.heads; h += 256) {
      const float zb = pr[C + h], za = pr[C + a.heads + h] + a.dt_bias[h];
      const float sp = za > 20.f ? za : log1pf(expf(za));
      o[C + h] = 1.0f / (1.0f + expf(-zb));
      o[C + a.heads + h] = expf(-expf(a.a_log[h]) * sp);
    }
    return;
  }
  const bool qk = u < G2;
  const int n = qk ? a.dim : a.vdim, c0 = qk ? u * a.dim : 2 * GD + (u - G2) * a.vdim;
  const float* __restrict__ st_old = a.state ? a.state + (size_t)par * a.state_buf + (size_t)row * nb * C : nullptr;
  float* __restrict__ st_new = a.state ? a.state + (size_t)(par ^ 1) * a.state_buf + (size_t)row * nb * C : nullptr;
  const float* __restrict__ cw = a.cw;
  float mine = 0.f;                                        // a q / k head's channel of this thread (D <= 256)
  for (int cc = threadIdx.x; cc < n; cc += 256) {
    const int c = c0 + cc;
    const float x0 = pr[c];
    float acc = cw[(size_t)c * a.taps + nb] * x0;
    for (int d = 1; d <= nb; d++) {                        // the row d positions back
      float xv = 0.f;
      if (d <= i) xv = pr[c - (long long)d * a.ldp];
      else if (pos - d >= 0) xv = st_old[(size_t)(nb - (d - i)) * C + c];      // tail slot s holds position past - nb + s, past = pos - i
      acc = fmaf(cw[(size_t)c * a.taps + nb - d], xv, acc);
    }
    const float act = acc / (1.0f + expf(-acc));
    if (qk) mine = act; else o[c] = act;
    if (st_new) {
      const int s = nb - (cnt - i);                        // row i of cnt lands in tail slot nb - (cnt - i) ...
      if (s >= 0) st_new[(size_t)s * C + c] = x0;
      if (i == 0)                                          // ... and an entry shorter than the tails keeps the end of the old ones
        for (int k = 0; k + cnt < nb; k++) st_new[(size_t)k * C + c] = (pos - (nb - cnt - k) >= 0) ? st_old[(size_t)(k + cnt) * C + c] : 0.f;
    }
  }
  if (!qk) return;
  const float ss = block_sum_256(mine * mine, s4);
  const float r = (u < a.kv_heads ? a.q_scale : 1.0f) / sqrtf(ss + a.unit_eps);
  if ((int)threadIdx.x < n) o[c0 + threadIdx.x] = mine * r;
}

// ---- the recurrences.  One workgroup per (entry, head, 32 value columns) walks the entry's tokens in order, TB at a time: the block's per-key-channel
// inputs (up to three vectors of `dim`) and the workgroup's value columns are staged in LDS (the next block's travel in registers meanwhile), then every
// lane updates its DPER rows of its column with no barrier inside the block: a wave owns 8 columns, its lanes = 8 columns x 8 row groups (the row groups
// of a column are adjacent lanes), 8 DPER >= dim.  Sums over the key channels cross the row groups on the lane crossbar.
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
constexpr int REC_RG = 8, REC_COLS = 4 * (64 / REC_RG);      // row groups per column; columns per workgroup
template <int DPER, int KIND>
__global__ __launch_bounds__(256) void rec_scan_kernel(StepMeta m, RecScanArgs a) {
  constexpr int RG = REC_RG, CW = 64 / RG, CB = REC_COLS, LP = DPER + 4, DP = RG * DPER, TB = DP <= 128 ? 16 : 8;      // LP: a row group's LDS stride (the groups' reads fall into different banks)
  constexpr int NQ = TB * DP / 256, NV = (TB * CB + 255) / 256, NA = KIND == REC_WKV ? 3 : 2;
  __shared__ __attribute__((aligned(16))) float s_in[NA][TB][RG * LP];      // [0]: the read vector, [1]: k, [2]: the decay
  __shared__ float s_v[TB][CB], s_b[TB], s_g[TB];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, rg = lane % RG, cl = lane / RG;
  const int jl = wv * CW + cl, j = blockIdx.z * CB + jl;
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
  const float* src[3] = {a.a, a.k, a.w};
  const long long lds[3] = {a.lda, a.ldk, a.ldw};
  float rin[NA][NQ], rv[NV], rb = 0.f, rgt = 0.f;
  auto fetch = [&](int t0) {
    const int nb = min(TB, cnt - t0);
#pragma unroll
    for (int u = 0; u < NQ; u++) {
      const int i = tid + 256 * u, t = i / DP, d = i - t * DP;
      const bool on = t < nb && d < a.dim;
      const size_t tok = (size_t)(start + t0 + min(t, nb - 1));
#pragma unroll
      for (int s = 0; s < NA; s++) rin[s][u] = on ? src[s][tok * lds[s] + (size_t)kh * a.dim + d] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < NV; u++) {
      const int i = tid + 256 * u, t = i / CB, c = i - t * CB;
      rv[u] = (t < nb && blockIdx.z * CB + c < a.vdim) ? a.v[(size_t)(start + t0 + t) * a.ldv + (size_t)h * a.vdim + blockIdx.z * CB + c] : 0.f;
    }
    if (KIND == REC_DELTA && tid < nb) { rb = a.beta[(size_t)(start + t0 + tid) * a.ldg + h]; rgt = a.g[(size_t)(start + t0 + tid) * a.ldg + h]; }
  };
  fetch(0);
  for (int t0 = 0; t0 < cnt; t0 += TB) {
    const int nb = min(TB, cnt - t0);
    __syncthreads();                                       // the block before has been read
#pragma unroll
    for (int u = 0; u < NQ; u++) {
      const int i = tid + 256 * u, t = i / DP, d = i - t * DP, at = (d / DPER) * LP + d % DPER;
#pragma unroll
      for (int s = 0; s < NA; s++) s_in[s][t][at] = rin[s][u];
    }
#pragma unroll
    for (int u = 0; u < NV; u++) { const int i = tid + 256 * u; if (i < TB * CB) s_v[i / CB][i % CB] = rv[u]; }
    if (KIND == REC_DELTA && tid < TB) { s_b[tid] = rb; s_g[tid] = rgt; }
    __syncthreads();
    if (t0 + TB < cnt) fetch(t0 + TB);
    // a token's operands travel from LDS to registers one token ahead of their use (two register sets, taken in turn), so the reads' latency lies under
    // the arithmetic of the token before instead of on the recurrence's critical path
    struct Tok { f32x4 in[NA][DPER / 4]; float v, g, b; };
    auto take = [&](Tok& k, int t) {
#pragma unroll
      for (int s = 0; s < NA; s++)
#pragma unroll
        for (int dd = 0; dd < DPER; dd += 4) k.in[s][dd / 4] = *reinterpret_cast<const f32x4*>(&s_in[s][t][l0 + dd]);
      k.v = s_v[t][jl];
      if (KIND == REC_DELTA) { k.g = s_g[t]; k.b = s_b[t]; }
    };
    auto advance = [&](const Tok& k, int t) {
      float po = 0.f;
      if (KIND == REC_WKV) {
#pragma unroll
        for (int dd = 0; dd < DPER; dd++) {
          const float kv = k.in[1][dd / 4][dd & 3] * k.v;
          po = fmaf(k.in[0][dd / 4][dd & 3], fmaf(ub[dd], kv, S[dd]), po);
          S[dd] = fmaf(k.in[NA - 1][dd / 4][dd & 3], S[dd], kv);
        }
      } else {
        float pk = 0.f;
#pragma unroll
        for (int dd = 0; dd < DPER; dd++) { S[dd] *= k.g; pk = fmaf(S[dd], k.in[1][dd / 4][dd & 3], pk); }
        pk = row_group_sum<RG>(pk);
        const float uj = k.b * (k.v - pk);
#pragma unroll
        for (int dd = 0; dd < DPER; dd++) { S[dd] = fmaf(k.in[1][dd / 4][dd & 3], uj, S[dd]); po = fmaf(S[dd], k.in[0][dd / 4][dd & 3], po); }
      }
      po = row_group_sum<RG>(po);
      if (rg == 0 && col) a.out[(size_t)(start + t0 + t) * a.ldo + (size_t)h * a.vdim + j] = po;
    };
    Tok ka, kb;
    take(ka, 0);
    for (int t = 0; t < nb; t += 2) {
      take(kb, min(t + 1, TB - 1));
      advance(ka, t);
      take(ka, min(t + 2, TB - 1));
      if (t + 1 < nb) advance(kb, t + 1);
    }
  }
#pragma unroll
  for (int dd = 0; dd < DPER; dd++) { const int d = d0 + dd; if (d < a.dim && col) Sg[(size_t)d * a.vdim + j] = S[dd]; }
}

}  // namespace tgx
