// stack_seq.h — row-wise kernels of the layered designs with sandwich norms, rotary grouped-query attention over a paged key / value pool, matrix-memory
// (mLSTM) layers, PolyNorm feed-forwards and grouped-choice experts (Modepel).  Same conventions as stack.h: a step's T tokens are the concatenated
// entries of a ragged batch (StepMeta), all arithmetic here is fp32, every reduction has a fixed order.
//   embed_rows_kernel       x[t] = embed[id]
//   scalar_norm_kernel      rows / sqrt(mean(row^2) + eps) * one number
//   sandwich_kernel         x += norm_b(sublayer output) and the next sublayer's normed input, the experts' combine folded in
//   poly_norm_kernel        a N(z) + b N(z^2) + c N(z^3) + e over a token's feed-forward values
//   gqa_append_kernel       rotary positions on q (in place) and k, value mixing, store of k / v into the token's place in the pool
//   gqa_attn_kernel         one (token, head) per workgroup against the pool: softmax with a constant sink, sigmoid gate on the output
//   gqa_attn_kernel<.., SPLIT> + gqa_attn_merge_kernel   the same with a sequence's keys divided between workgroups
//   mlstm_scan_kernel       the matrix-memory recurrence over an entry's tokens, state per slot in fp32
//   head_norm_gate_kernel   per-head RMS norm, learned scale and sigmoid / silu gate of a recurrence's outputs
//   router_group_kernel     softmax scores, correction, group limit, top-k, weights = scores * scale; the shared expert's gate
#pragma once
#include "stack.h"
#include "stack_gemm.h"

namespace tgx {

template <int DT>
__global__ __launch_bounds__(256) void embed_rows_kernel(StepMeta m, const elem_t<DT>* embed, float* x, int W) {
  const int t = blockIdx.x;
  const size_t id = (size_t)m.tok_id[t];
  for (int c = threadIdx.x; c < W; c += 256) x[(size_t)t * W + c] = elem_to_f32<DT>(embed[id * W + c]);
}

// out[i] = x[rows ? rows[i] : i] / sqrt(mean(row^2) + eps) * g[0]
__global__ __launch_bounds__(256) void scalar_norm_kernel(const float* x, const int* rows, const float* g, float* out, int W, float eps) {
  __shared__ float s4[4];
  const float* xr = x + (size_t)(rows ? rows[blockIdx.x] : blockIdx.x) * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) ss = fmaf(xr[c], xr[c], ss);
  ss = block_sum_256(ss, s4);
  const float r = g[0] / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) out[(size_t)blockIdx.x * W + c] = xr[c] * r;
}

// ---- the seam between two sublayers.  y_t = the sublayer's output for token t: one row, or the sum over the token's `top` expert rows (router weights
// already applied; a pair whose choice is an identity output contributes weight * h_t instead of a row) plus the shared expert's row.
// x_t <- x_t + g_post * y_t / rms(y_t);  out_t = g_next * x_t / rms(x_t) (the next sublayer's input; skipped without g_next).  One workgroup per token;
// a thread keeps its channels between the passes, so only the two sums cross threads.
struct SandwichArgs {
  float* x;                  // [T][W]
  const float* y;            // [T * top][W]
  int top;
  const int* sel;            // [T * top] chosen router outputs (nullptr: plain rows)
  const float* selw;         // [T * top]
  int n_real;                // router outputs below this have a row in y
  const float* h;            // [T][W] the sublayer's input (identity outputs); never the same buffer as out
  const float* ysh;          // [T][W] (nullptr: no shared expert)
  float* ytmp;               // [T][W] scratch
  const float* g_post;
  const float* g_next;
  float* out;                // [T][W]
  int W; float eps;
};
__global__ __launch_bounds__(256) void sandwich_kernel(SandwichArgs a) {
  __shared__ float s4[4];
  const size_t t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.W; c += 256) {
    float v = 0.f;
    for (int k = 0; k < a.top; k++) {
      const size_t p = t * a.top + k;
      if (a.sel && a.sel[p] >= a.n_real) v = fmaf(a.selw[p], a.h[t * a.W + c], v);
      else v += a.y[p * a.W + c];
    }
    if (a.ysh) v += a.ysh[t * a.W + c];
    a.ytmp[t * a.W + c] = v;
    ss = fmaf(v, v, ss);
  }
  ss = block_sum_256(ss, s4);
  const float r1 = a.g_post[0] / sqrtf(ss / (float)a.W + a.eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < a.W; c += 256) {
    const float v = fmaf(a.ytmp[t * a.W + c], r1, a.x[t * a.W + c]);
    a.x[t * a.W + c] = v;
    s2 = fmaf(v, v, s2);
  }
  if (!a.g_next) return;
  s2 = block_sum_256(s2, s4);
  const float r2 = a.g_next[0] / sqrtf(s2 / (float)a.W + a.eps);
  for (int c = threadIdx.x; c < a.W; c += 256) a.out[t * a.W + c] = a.x[t * a.W + c] * r2;
}

// ---- PolyNorm in place on z [T][F]: coef = (a, b, c, e)
__global__ __launch_bounds__(256) void poly_norm_kernel(float* z, const float* coef, int F, float eps) {
  __shared__ float s4[4];
  float* zr = z + (size_t)blockIdx.x * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = zr[c], v2 = v * v, v3 = v2 * v;
    s1 = fmaf(v, v, s1); s2 = fmaf(v2, v2, s2); s3 = fmaf(v3, v3, s3);
  }
  s1 = block_sum_256(s1, s4); s2 = block_sum_256(s2, s4); s3 = block_sum_256(s3, s4);
  const float r1 = coef[0] / sqrtf(s1 / (float)F + eps), r2 = coef[1] / sqrtf(s2 / (float)F + eps), r3 = coef[2] / sqrtf(s3 / (float)F + eps), e = coef[3];
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = zr[c], v2 = v * v;
    zr[c] = fmaf(v, r1, fmaf(v2, r2, fmaf(v2 * v, r3, e)));
  }
}

// ---- rotary positions, query temperature, value mixing and the pool append of one attention layer.  One workgroup per token.
// proj row = [q (heads * dim) | k (kv_heads * dim) | v (kv_heads * vdim) | ...]; a pair of channels of every q and k head turns by the angle of
// (position, i), whose cosine and sine come from a host-made table: the pair is (i, i + rot_dims / 2), or the neighbours (2i, 2i + 1) with rot_pairs.
// q is rotated in place (and multiplied by 1 + q_temp_coef * ln(floor((position + 1) / q_temp_every) + 1) where the design has a query temperature);
// k and v go to the pool in the storage dtype.  A layer that reads another layer's keys and values has q alone in its row and no pool of its own.
struct GqaAppendArgs {
  float* proj; long long ldp;
  int heads, kv_heads, dim, vdim, rot_dims;
  const float* cs;           // [positions][rot_dims / 2][2]
  void* poolK;               // [pages][page_tokens][kv_heads * dim] (nullptr: nothing is appended, the row holds no k / v)
  void* poolV;               // [pages][page_tokens][kv_heads * vdim]
  void* poolVT;              // [pages][kv_heads * vdim][page_tokens]: the same values, token-contiguous per channel (nullptr: not kept)
  float* vfirst;             // [T][kv_heads * vdim] values of the first mixing layer for the step's tokens
  int vmode;                 // 0: no mixing; 1: this layer's values become vfirst; 2: v <- (1 - lam) v + lam vfirst
  const float* lam;
  int rot_pairs;             // 1: neighbours turn together
  float q_temp_coef; int q_temp_every;      // coef 0: no query temperature
  float qk_unit_eps;         // > 0: every q and k head is first divided by sqrt(mean(head^2) + qk_unit_eps) (no weight)
  unsigned short *q_hi, *q_lo;      // [T][heads * dim] (nullptr: not kept): the finished queries as two 16-bit terms, the A operand of a matrix-core score product
};
template <int DT>
__global__ __launch_bounds__(256) void gqa_append_kernel(StepMeta m, GqaAppendArgs a) {
  const int t = blockIdx.x, pos = m.tok_pos[t];
  float* row = a.proj + (size_t)t * a.ldp;
  const int half = a.rot_dims >> 1, nh = a.heads + (a.poolK ? a.kv_heads : 0);      // q heads and k heads are adjacent in the row: head index hd, offset hd * dim
  if (a.qk_unit_eps > 0.f) {      // a wave per head
    const int lane = threadIdx.x & 63;
    for (int hd = threadIdx.x >> 6; hd < nh; hd += 4) {
      float* u = row + (size_t)hd * a.dim;
      float ss = 0.f;
      for (int c = lane; c < a.dim; c += 64) ss = fmaf(u[c], u[c], ss);
      ss = wave_sum(ss);
      const float r = 1.0f / sqrtf(ss / (float)a.dim + a.qk_unit_eps);
      for (int c = lane; c < a.dim; c += 64) u[c] *= r;
    }
    __syncthreads();
  }
  for (int i = threadIdx.x; i < nh * half; i += 256) {
    const int hd = i / half, p = i - hd * half;
    const float c = a.cs[((size_t)pos * half + p) * 2], s = a.cs[((size_t)pos * half + p) * 2 + 1];
    float* u = row + (size_t)hd * a.dim + (a.rot_pairs ? 2 * p : p);
    const int other = a.rot_pairs ? 1 : half;
    const float x0 = u[0], x1 = u[other];
    u[0] = __fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, s));
    u[other] = __fadd_rn(__fmul_rn(x1, c), __fmul_rn(x0, s));
  }
  if (a.q_temp_coef != 0.f) {
    __syncthreads();
    const float f = fmaf(a.q_temp_coef, logf((float)((pos + 1) / a.q_temp_every) + 1.0f), 1.0f);
    for (int c = threadIdx.x; c < a.heads * a.dim; c += 256) row[c] *= f;
  }
  if constexpr (DT != DT_F32) {
    if (a.q_hi) {
      __syncthreads();
      const size_t qd = (size_t)a.heads * a.dim;
      for (int c = threadIdx.x; c < (int)qd; c += 256) split16<DT>(row[c], a.q_hi[(size_t)t * qd + c], a.q_lo[(size_t)t * qd + c]);
    }
  }
  if (!a.poolK) return;
  __syncthreads();
  const int page = m.tbl[(size_t)m.tok_row[t] * m.tbl_stride + (pos >> m.page_shift)];
  const size_t slot = ((size_t)page << m.page_shift) + (size_t)(pos & ((1 << m.page_shift) - 1));
  const int kd = a.kv_heads * a.dim, vd = a.kv_heads * a.vdim;
  elem_t<DT>* kdst = reinterpret_cast<elem_t<DT>*>(a.poolK) + slot * kd;
  elem_t<DT>* vdst = reinterpret_cast<elem_t<DT>*>(a.poolV) + slot * vd;
  const float* ksrc = row + (size_t)a.heads * a.dim;
  const float* vsrc = ksrc + kd;
  for (int c = threadIdx.x; c < kd; c += 256) kdst[c] = f32_to_elem<DT>(ksrc[c]);
  const float lam = a.vmode == 2 ? a.lam[0] : 0.f;
  for (int c = threadIdx.x; c < vd; c += 256) {
    float v = vsrc[c];
    if (a.vmode == 1) a.vfirst[(size_t)t * vd + c] = v;
    if (a.vmode == 2) v = fmaf(lam, a.vfirst[(size_t)t * vd + c], __fmul_rn(1.0f - lam, v));
    const elem_t<DT> sv = f32_to_elem<DT>(v);
    vdst[c] = sv;
    if (a.poolVT) reinterpret_cast<elem_t<DT>*>(a.poolVT)[((((size_t)page * vd) + c) << m.page_shift) + (size_t)(pos & ((1 << m.page_shift) - 1))] = sv;
  }
}

// ---- attention of one (token, head) per workgroup: the four waves take every fourth key, lanes hold dim / 64 key and vdim / 64 value channels.
// Scores, softmax and the weighted value sum are fp32; the denominator also holds exp(sink) for a sink without a value (has_sink).  Every key, also
// those of the step's own tokens, is read from the pool.  The output is multiplied by sigmoid(gate) where a gate is given.
// The query at position i sees the keys [first_key(i), i]: all before it, a sliding window of mask_size positions, or its own block of mask_size
// positions (blocks counted from position 0 of the sequence).  score = q . k * scale, then softcap * tanh(score / softcap), then minus
// slope_h * (i - j), slope_h = 2^(-8 (h + 1) / heads), each where the layer has it.
// (first_key and distance_slope: stack_meta.h)
struct GqaAttnArgs {
  const float* q; long long ldq;       // head h of token t at q + t * ldq + h * dim
  const void* poolK; const void* poolV;
  const float* gate; long long ldg;    // gate pre-activation of (t, h, c) at gate + t * ldg + h * vdim + c (nullptr: none)
  float* out; long long ldo;           // [T][heads * vdim]
  int heads, kv_heads, dim, vdim;
  float scale, sink; int has_sink;
  float* part; int nsplit, keys_per;   // split form: records (m, l, acc[vdim]) per (token, head, split); split z takes keys_per keys from first_key on
  int mask_kind, mask_size;            // MASK_*
  float softcap; int dist_bias;        // softcap <= 0: none
};
constexpr int GQA_MAX_RPL = 4;          // channels per lane: dim, vdim <= 256
template <int DT, int RPL, bool SPLIT>
__global__ __launch_bounds__(256) void gqa_attn_kernel(StepMeta m, GqaAttnArgs a) {
  __shared__ float s_m[4], s_l[4];
  extern __shared__ float s_acc[];      // [4][vdim]
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int row = m.tok_row[t], nkeys = m.tok_pos[t] + 1;
  const int kvh = h / (a.heads / a.kv_heads), kd = a.kv_heads * a.dim, vd = a.kv_heads * a.vdim;
  int k0 = first_key(nkeys - 1, a.mask_kind, a.mask_size), k1 = nkeys;
  if (SPLIT) { k0 = min(nkeys, k0 + (int)blockIdx.z * a.keys_per); k1 = min(nkeys, k0 + a.keys_per); }
  const float slope = a.dist_bias ? distance_slope(h, a.heads) : 0.f;
  const float* q = a.q + (size_t)t * a.ldq + (size_t)h * a.dim;
  float qv[RPL], acc[RPL];
#pragma unroll
  for (int k = 0; k < RPL; k++) { const int c = lane + 64 * k; qv[k] = c < a.dim ? q[c] : 0.f; acc[k] = 0.f; }
  const bool sink_here = a.has_sink && wv == 0 && (!SPLIT || blockIdx.z == 0);      // the sink enters once
  float mx = sink_here ? a.sink : -INFINITY, l = sink_here ? 1.f : 0.f;
  const elem_t<DT>* pk = reinterpret_cast<const elem_t<DT>*>(a.poolK) + (size_t)kvh * a.dim;
  const elem_t<DT>* pv = reinterpret_cast<const elem_t<DT>*>(a.poolV) + (size_t)kvh * a.vdim;
  const int pmask = (1 << m.page_shift) - 1;
  for (int j = k0 + wv; j < k1; j += 4) {
    const int page = m.tbl[(size_t)row * m.tbl_stride + (j >> m.page_shift)];
    const size_t slot = ((size_t)page << m.page_shift) + (size_t)(j & pmask);
    const elem_t<DT>* kr = pk + slot * kd;
    const elem_t<DT>* vr = pv + slot * vd;
    float vv[RPL], s = 0.f;
#pragma unroll
    for (int k = 0; k < RPL; k++) {
      const int c = lane + 64 * k;
      s = fmaf(qv[k], c < a.dim ? elem_to_f32<DT>(kr[c]) : 0.f, s);
      vv[k] = c < a.vdim ? elem_to_f32<DT>(vr[c]) : 0.f;
    }
    s = wave_sum(s) * a.scale;
    if (a.softcap > 0.f) s = a.softcap * tanhf(s / a.softcap);
    s = fmaf(-slope, (float)(nkeys - 1 - j), s);
    const float mn = fmaxf(mx, s);
    const float corr = expf(mx - mn), p = expf(s - mn);      // mx = -inf on a wave's first key: corr = 0
    l = fmaf(l, corr, p);
#pragma unroll
    for (int k = 0; k < RPL; k++) acc[k] = fmaf(acc[k], corr, p * vv[k]);
    mx = mn;
  }
  if (lane == 0) { s_m[wv] = mx; s_l[wv] = l; }
#pragma unroll
  for (int k = 0; k < RPL; k++) { const int c = lane + 64 * k; if (c < a.vdim) s_acc[wv * a.vdim + c] = acc[k]; }
  __syncthreads();
  const float M = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
  float f[4], L = 0.f;
#pragma unroll
  for (int w = 0; w < 4; w++) { f[w] = s_m[w] == -INFINITY ? 0.f : expf(s_m[w] - M); L = fmaf(s_l[w], f[w], L); }
  if (SPLIT) {
    float* rec = a.part + (((size_t)t * a.heads + h) * a.nsplit + blockIdx.z) * (size_t)(a.vdim + 2);
    if (threadIdx.x == 0) { rec[0] = M; rec[1] = L; }
    for (int c = threadIdx.x; c < a.vdim; c += 256) rec[2 + c] = s_acc[c] * f[0] + s_acc[a.vdim + c] * f[1] + s_acc[2 * a.vdim + c] * f[2] + s_acc[3 * a.vdim + c] * f[3];
  } else {
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    float* o = a.out + (size_t)t * a.ldo + (size_t)h * a.vdim;
    for (int c = threadIdx.x; c < a.vdim; c += 256) {
      float v = (s_acc[c] * f[0] + s_acc[a.vdim + c] * f[1] + s_acc[2 * a.vdim + c] * f[2] + s_acc[3 * a.vdim + c] * f[3]) * inv;
      if (a.gate) v = v / (1.0f + expf(-a.gate[(size_t)t * a.ldg + (size_t)h * a.vdim + c]));
      o[c] = v;
    }
  }
}
// merges the split records of one (token, head) in split order
__global__ __launch_bounds__(256) void gqa_attn_merge_kernel(GqaAttnArgs a) {
  __shared__ float s_f[64];
  __shared__ float s_inv;
  const int t = blockIdx.x, h = blockIdx.y;
  const size_t rs = (size_t)(a.vdim + 2);
  const float* rec = a.part + ((size_t)t * a.heads + h) * a.nsplit * rs;
  if (threadIdx.x < 64) {
    const int s = threadIdx.x;
    const float ms = s < a.nsplit ? rec[(size_t)s * rs] : -INFINITY;
    const float M = group_max<64>(ms);
    const float f = ms == -INFINITY ? 0.f : expf(ms - M);
    float lf = s < a.nsplit ? rec[(size_t)s * rs + 1] * f : 0.f;
    for (int o = 1; o < 64; o <<= 1) { const float other = __shfl_up(lf, o, 64); if (s >= o) lf += other; }
    s_f[s] = f;
    if (s == 63) s_inv = lf > 0.f ? 1.0f / lf : 0.f;
  }
  __syncthreads();
  const float inv = s_inv;
  float* o = a.out + (size_t)t * a.ldo + (size_t)h * a.vdim;
  for (int c = threadIdx.x; c < a.vdim; c += 256) {
    float v = 0.f;
    for (int s = 0; s < a.nsplit; s++) v = fmaf(rec[(size_t)s * rs + 2 + c], s_f[s], v);
    v *= inv;
    if (a.gate) v = v / (1.0f + expf(-a.gate[(size_t)t * a.ldg + (size_t)h * a.vdim + c]));
    o[c] = v;
  }
}

// ---- matrix memory (mLSTM).  Per head: a [dim][vdim] matrix S, a [dim] vector n and a running maximum mx (log scale), all fp32, all zero (mx too) at a
// sequence's start.  For every token, with log gates i = cap tanh(zi / cap), f = logsigmoid(cap tanh(zf / cap)) (applied by the input product's epilogue):
//   mx' = max(f + mx, i);  S' = exp(f + mx - mx') S + exp(i - mx') k v^T;  n' likewise with k;  o = S'^T q / (max(|n' . q|, exp(-mx')) + 1e-6)
// One workgroup per (entry, head, 4 CW value columns; CW = 16, or 8 when the step has few entries and heads) walks the entry's tokens in order, a block of
// 8 .. 32 at a time:
//   stage   q (scaled), k, the workgroup's v columns and the gate pre-activations of the block's tokens into LDS (coalesced)
//   gates   one lane per token: mx' and the three factors exp(f + mx - mx'), exp(i - mx'), exp(-mx') from prefix sums and maxima over the block
//           (mx'_t = B_t + max(mx_before, max_{s<=t} (i_s - B_s)), B_t = f_0 + .. + f_t: the recurrence unrolled); i and f arrive activated
//   scan    no barrier and no lane exchange inside: a wave owns CW columns, its lanes = 64 / CW row groups x CW columns, each lane keeps DPER rows of its
//           column in registers and leaves its partial sums of S^T q and n . q (every wave computes the latter) per token in LDS
//   out     the partial sums of the block's tokens are added up (over the row groups; over the wave for n . q) and divided
// n and mx are double-buffered per slot (buffer `par` is read, `par ^ 1` written), because the workgroups of a head's other columns read them too.
// The outputs leave un-normed (head_norm_gate_kernel follows).
struct MlstmArgs {
  const float* proj; long long ldp;     // [T][q | k | v | g | i | f]: q, k per head [dim]; v, g per head [vdim]; i, f per head: the log gates (the input product's epilogue has applied cap and log sigmoid)
  int heads, dim, vdim;
  float qscale;
  float* S;                             // [slots][heads][dim][vdim]
  float* n;                             // [2][slots][heads][dim]
  float* mx;                            // [2][slots][heads]
  size_t n_buf, mx_buf;                 // elements between the two buffers
  float* hs; long long ldh;             // [T][heads * vdim]
};
template <int DPER, int CW>      // rows per lane and columns per wave: (64 / CW) DPER >= dim
__global__ __launch_bounds__(256) void mlstm_scan_kernel(StepMeta m, MlstmArgs a) {
  constexpr int RG = 64 / CW, NPL = (DPER + CW - 1) / CW, DP = RG * DPER, LP = DPER + 4, CB = 4 * CW;      // LP: a row group's LDS stride (the groups' reads fall into different banks)
  // tokens per block: the eight-column form runs alone on its compute unit (few workgroups) and takes long blocks; the sixteen-column form keeps its
  // LDS (staged q and k, the partial sums) near 50 KB so that several workgroups share a compute unit
  constexpr int TB = CW == 8 ? (DP <= 128 ? 32 : 16) : (DP <= 256 ? 16 : 8);
  constexpr int NQ = TB * DP / 256, NV = (TB * CB + 255) / 256;
  __shared__ __attribute__((aligned(16))) float s_q[TB][RG * LP], s_k[TB][RG * LP];
  __shared__ float s_v[TB][CB], s_zi[TB], s_zf[TB], s_keep[TB], s_take[TB], s_emn[TB], s_mx[2];
  __shared__ float s_po[TB][4][64], s_pn[TB][4][64];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, rg = lane / CW, cl = lane % CW;
  const int jl = wv * CW + cl, j = blockIdx.z * CB + jl;
  const int start = m.ent_start[e], cnt = m.ent_count[e], row = m.ent_row[e], par = m.ent_par[e];
  const bool fresh = m.tok_pos[start] == 0;
  const int d0 = rg * DPER, l0 = rg * LP;
  const int oq = h * a.dim, ok = a.heads * a.dim + h * a.dim, ov = 2 * a.heads * a.dim + h * a.vdim + blockIdx.z * CB;
  const int oi = 2 * a.heads * a.dim + 2 * a.heads * a.vdim + h, of = oi + a.heads;
  float* Sg = a.S + ((size_t)row * a.heads + h) * (size_t)a.dim * a.vdim;
  const float* n_old = a.n + (size_t)par * a.n_buf + ((size_t)row * a.heads + h) * a.dim;
  float* n_new = a.n + (size_t)(par ^ 1) * a.n_buf + ((size_t)row * a.heads + h) * a.dim;
  float S[DPER], nn[NPL];
#pragma unroll
  for (int dd = 0; dd < DPER; dd++) { const int d = d0 + dd; S[dd] = (!fresh && d < a.dim && j < a.vdim) ? Sg[(size_t)d * a.vdim + j] : 0.f; }
#pragma unroll
  for (int k = 0; k < NPL; k++) { const int dl = cl + CW * k, d = d0 + dl; nn[k] = (!fresh && dl < DPER && d < a.dim) ? n_old[d] : 0.f; }
  if (tid == 0) s_mx[0] = fresh ? 0.f : a.mx[(size_t)par * a.mx_buf + (size_t)row * a.heads + h];
  // the next block's inputs travel in registers while the current block is scanned
  float rq[NQ], rk[NQ], rv[NV], rzi = 0.f, rzf = 0.f;
  auto fetch = [&](int t0) {
    const int nb = min(TB, cnt - t0);
#pragma unroll
    for (int u = 0; u < NQ; u++) {
      const int i = tid + 256 * u, t = i / DP, d = i - t * DP;
      const bool on = t < nb && d < a.dim;
      const float* r = a.proj + (size_t)(start + t0 + min(t, nb - 1)) * a.ldp;
      rq[u] = on ? r[oq + d] : 0.f; rk[u] = on ? r[ok + d] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < NV; u++) {
      const int i = tid + 256 * u, t = i / CB, c = i - t * CB;
      rv[u] = (t < nb && blockIdx.z * CB + c < a.vdim) ? a.proj[(size_t)(start + t0 + t) * a.ldp + ov + c] : 0.f;
    }
    if (tid < nb) { const float* r = a.proj + (size_t)(start + t0 + tid) * a.ldp; rzi = r[oi]; rzf = r[of]; }
  };
  fetch(0);
  for (int t0 = 0, blk = 0; t0 < cnt; t0 += TB, blk++) {
    const int nb = min(TB, cnt - t0);
    __syncthreads();                                       // the previous block's rows and partial sums have been read
#pragma unroll
    for (int u = 0; u < NQ; u++) {
      const int i = tid + 256 * u, t = i / DP, d = i - t * DP, at = (d / DPER) * LP + d % DPER;
      s_q[t][at] = rq[u] * a.qscale; s_k[t][at] = rk[u];
    }
#pragma unroll
    for (int u = 0; u < NV; u++) { const int i = tid + 256 * u; if (i < TB * CB) s_v[i / CB][i % CB] = rv[u]; }
    if (tid < TB) { s_zi[tid] = tid < nb ? rzi : -INFINITY; s_zf[tid] = tid < nb ? rzf : 0.f; }
    __syncthreads();
    if (t0 + TB < cnt) fetch(t0 + TB);
    if (wv == 0) {      // one lane per token: prefix sums of the log forget gates, prefix maxima of i - B, both by lane exchanges
      const float fl = lane < TB ? s_zf[lane] : 0.f, ig = lane < TB ? s_zi[lane] : -INFINITY, mprev = s_mx[blk & 1];
      float bs = fl;
#pragma unroll
      for (int o = 1; o < TB; o <<= 1) { const float v = __shfl_up(bs, o, 64); if (lane >= o) bs += v; }
      float c = ig - bs;
#pragma unroll
      for (int o = 1; o < TB; o <<= 1) { const float v = __shfl_up(c, o, 64); if (lane >= o) c = fmaxf(c, v); }
      const float mn = bs + fmaxf(mprev, c);
      const float up = __shfl_up(mn, 1, 64), mbefore = lane == 0 ? mprev : up;      // the maximum after the token before
      if (lane < nb) {
        s_keep[lane] = expf(fl + mbefore - mn); s_take[lane] = expf(ig - mn); s_emn[lane] = expf(-mn);
        if (lane == nb - 1) s_mx[(blk + 1) & 1] = mn;
      }
    }
    __syncthreads();
    for (int t = 0; t < nb; t++) {
      const float keep = s_keep[t], tv = s_take[t] * s_v[t][jl];
      float po = 0.f;
#pragma unroll
      for (int dd = 0; dd < DPER; dd += 4) {
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(&s_k[t][l0 + dd]), q4 = *reinterpret_cast<const f32x4*>(&s_q[t][l0 + dd]);
#pragma unroll
        for (int u = 0; u < 4; u++) { S[dd + u] = fmaf(keep, S[dd + u], k4[u] * tv); po = fmaf(S[dd + u], q4[u], po); }
      }
      float pn = 0.f;
#pragma unroll
      for (int k = 0; k < NPL; k++) {
        const int dl = cl + CW * k;
        if (dl < DPER) { nn[k] = fmaf(keep, nn[k], s_take[t] * s_k[t][l0 + dl]); pn = fmaf(nn[k], s_q[t][l0 + dl], pn); }
      }
      s_po[t][wv][lane] = po; s_pn[t][wv][lane] = pn;      // partial sums over this lane's rows: reduced after the block, off the recurrence's critical path
    }
    __syncthreads();
    // the block's outputs: row group rg of a wave takes tokens rg, rg + RG, ...; its CW lanes are the wave's columns
    for (int t = rg; t < nb; t += RG) {
      float o = 0.f, nq = 0.f;
#pragma unroll
      for (int g = 0; g < RG; g++) o += s_po[t][wv][g * CW + cl];
#pragma unroll
      for (int g = 0; g < RG; g++) nq += s_pn[t][wv][RG * cl + g];
      nq = row_group_sum<CW>(nq);
      if (j < a.vdim) a.hs[(size_t)(start + t0 + t) * a.ldh + (size_t)h * a.vdim + j] = o / (fmaxf(fabsf(nq), s_emn[t]) + 1e-6f);
    }
  }
  __syncthreads();
#pragma unroll
  for (int dd = 0; dd < DPER; dd++) { const int d = d0 + dd; if (d < a.dim && j < a.vdim) Sg[(size_t)d * a.vdim + j] = S[dd]; }
  if (blockIdx.z == 0 && wv == 0) {
#pragma unroll
    for (int k = 0; k < NPL; k++) { const int dl = cl + CW * k, d = d0 + dl; if (dl < DPER && d < a.dim) n_new[d] = nn[k]; }
    if (tid == 0) a.mx[(size_t)(par ^ 1) * a.mx_buf + (size_t)row * a.heads + h] = s_mx[((cnt + TB - 1) / TB) & 1];
  }
}

// out[t][h][c] = hs / sqrt(mean_c(hs^2) + eps) * w[h * w_hstride + c] * gate, gate = sigmoid(z) or silu(z) of the pre-activation z (w_hstride 0: one
// weight vector for all heads).  One wave per (token, head): the seam behind every recurrent mixer (mLSTM, wkv, gated delta rule).
struct HeadNormGateArgs { const float* hs; long long ldh; const float* w; int w_hstride; const float* gate; long long ldg; int silu_gate; float* out; long long ldo; int vdim; float eps; };
__global__ __launch_bounds__(64) void head_norm_gate_kernel(HeadNormGateArgs a) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* r = a.hs + (size_t)t * a.ldh + (size_t)h * a.vdim;
  float ss = 0.f;
  for (int c = lane; c < a.vdim; c += 64) ss = fmaf(r[c], r[c], ss);
  ss = wave_sum(ss);
  const float rinv = 1.0f / sqrtf(ss / (float)a.vdim + a.eps);
  for (int c = lane; c < a.vdim; c += 64) {
    const float g = a.gate[(size_t)t * a.ldg + (size_t)h * a.vdim + c], sg = 1.0f / (1.0f + expf(-g));
    a.out[(size_t)t * a.ldo + (size_t)h * a.vdim + c] = r[c] * rinv * a.w[(size_t)h * a.w_hstride + c] * (a.silu_gate ? g * sg : sg);
  }
}

// ---- grouped-choice router.  z [T][ldz]: the E router products of a token (fp32 product of fp32 weights), then the shared expert's gate product where
// there is one.  Scores s = softmax(z) over all E; choice scores c = s + corr; the E outputs form `groups` equal groups of neighbours, a group counts as
// its largest choice score, members of the `keep` best groups stay eligible; the `top` largest eligible choice scores are chosen (ties: the lower index);
// weights = s * scale.  One wave per token.
// Variants: sigmoid_scores: s = sigmoid(z) instead of the softmax (corr may be nullptr: no correction); group_top2: a group counts as the sum of its two
// largest choice scores; normalise: the chosen weights are divided by their sum + 1e-20 (before the scale).
struct RouterGroupArgs {
  const float* z; int ldz;
  const float* corr;         // [E]
  int* sel; float* selw;     // [T][top]
  float* sgw;                // [T] sigmoid of the product in column E (nullptr: none)
  int E, top, groups, keep;
  float scale;
  int sigmoid_scores, group_top2, normalise;
};
__global__ __launch_bounds__(64) void router_group_kernel(RouterGroupArgs a) {
  __shared__ float s_s[ROUTER_MAX_E], s_c[ROUTER_MAX_E], s_g[ROUTER_MAX_E];
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* z = a.z + (size_t)t * a.ldz;
  if (a.sigmoid_scores) {
    for (int e = lane; e < a.E; e += 64) { s_s[e] = 1.0f / (1.0f + expf(-z[e])); s_c[e] = a.corr ? s_s[e] + a.corr[e] : s_s[e]; }
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < a.E; e += 64) mx = fmaxf(mx, z[e]);
    mx = group_max<64>(mx);
    float den = 0.f;
    for (int e = lane; e < a.E; e += 64) { const float p = expf(z[e] - mx); s_s[e] = p; den += p; }
    den = wave_sum(den);
    for (int e = lane; e < a.E; e += 64) { s_s[e] = s_s[e] / den; s_c[e] = a.corr ? s_s[e] + a.corr[e] : s_s[e]; }
  }
  __syncthreads();
  if (a.groups > 1) {
    const int per = a.E / a.groups;
    for (int g = lane; g < a.groups; g += 64) {
      float b = -INFINITY, b2 = -INFINITY;      // the largest and the second largest
      for (int e = g * per; e < (g + 1) * per; e++) { const float v = s_c[e]; if (v > b) { b2 = b; b = v; } else b2 = fmaxf(b2, v); }
      s_g[g] = a.group_top2 && per > 1 ? b + b2 : b;
    }
    __syncthreads();
    // the `keep` best groups, one pick per round; a kept group is marked by +inf, the others end as dropped
    for (int k = 0; k < a.keep; k++) {
      float bv = -INFINITY; int bi = 0x7fffffff;
      for (int g = lane; g < a.groups; g += 64) { const float v = s_g[g]; if (v != INFINITY && v > bv) { bv = v; bi = g; } }
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64); const int oi = __shfl_xor(bi, o, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
      }
      if (bi < a.groups && (bi & 63) == lane) s_g[bi] = INFINITY;
    }
    __syncthreads();
    for (int e = lane; e < a.E; e += 64) if (s_g[e / per] != INFINITY) s_c[e] = -INFINITY;
    __syncthreads();
  }
  for (int k = 0; k < a.top; k++) {
    float bv = -INFINITY; int bi = 0x7fffffff;
    for (int e = lane; e < a.E; e += 64) { const float v = s_c[e]; if (v > bv) { bv = v; bi = e; } }
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64); const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi < a.E && (bi & 63) == lane) s_c[bi] = -INFINITY;
    if (lane == 0) {
      const int pick = bi < a.E ? bi : 0;
      a.sel[(size_t)t * a.top + k] = pick;
      a.selw[(size_t)t * a.top + k] = bi < a.E ? s_s[pick] * a.scale : 0.f;
    }
  }
  if (a.normalise && lane == 0) {      // in choice order
    float sum = 0.f;
    for (int k = 0; k < a.top; k++) sum += a.selw[(size_t)t * a.top + k];
    const float inv = a.scale / (sum + 1e-20f * a.scale);
    for (int k = 0; k < a.top; k++) a.selw[(size_t)t * a.top + k] *= inv;
  }
  if (a.sgw && lane == 0) a.sgw[t] = 1.0f / (1.0f + expf(-z[a.E]));
}

}  // namespace tgx
