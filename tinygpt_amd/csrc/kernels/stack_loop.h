// stack_loop.h — row-wise kernels of the layered designs with layer norms (weight and bias) before and after every sublayer, a looped span of layers and
// un-normalised sigmoid attention whose weights are mixed across heads (Zaluvik).  Same conventions as stack.h / stack_seq.h: a step's T tokens are the
// concatenated entries of a ragged batch (StepMeta), all arithmetic here is fp32, every reduction has a fixed order.
//   embed_scale_rows_kernel    x[t] = embed[id] * scale, and a second copy for the loop's re-injection
//   copy_rows_kernel           rows of one width between buffers of different strides
//   layer_norm_rows_kernel     (row - mean) / sqrt(var + eps) * w + b
//   affine_seam_kernel         x += mult * LN_b(sublayer output) and the next sublayer's LN_a input, the experts' combine folded in
//   sigmoid_mix_attn_kernel    a token against the window of its keys in the pool: sigmoid(score + bias) per head, weights mixed across heads, value sums
//   sigmoid_mix_merge_kernel   adds up the partial sums of a window divided between workgroups, applies the output gate
//   (kernels/stack_mix_mfma.h holds the same attention for portions of prompts on the matrix cores)
#pragma once
#include "stack.h"

namespace tgx {

template <int DT>
__global__ __launch_bounds__(256) void embed_scale_rows_kernel(StepMeta m, const elem_t<DT>* embed, float scale, float* x, float* x0, long long ldx0, int W) {
  const int t = blockIdx.x;
  const size_t id = (size_t)m.tok_id[t];
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = elem_to_f32<DT>(embed[id * W + c]) * scale;
    x[(size_t)t * W + c] = v;
    if (x0) x0[(size_t)t * ldx0 + c] = v;
  }
}

__global__ __launch_bounds__(256) void copy_rows_kernel(const float* src, long long lds, float* dst, long long ldd, int W) {
  const size_t t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) dst[t * ldd + c] = src[t * lds + c];
}

// mean and 1 / sqrt(variance + eps) of one row, the variance as the mean of the squared deviations (second pass over the row)
__device__ __forceinline__ void row_moments_256(const float* r, int W, float eps, float* s4, float& mean, float& rstd) {
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) s += r[c];
  mean = block_sum_256(s, s4) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) { const float d = r[c] - mean; q = fmaf(d, d, q); }
  rstd = 1.0f / sqrtf(block_sum_256(q, s4) / (float)W + eps);
}

// out[i] = LN(x[rows ? rows[i] : i]) * w + b
__global__ __launch_bounds__(256) void layer_norm_rows_kernel(const float* x, const int* rows, const float* w, const float* b, float* out, int W, float eps) {
  __shared__ float s4[4];
  const float* xr = x + (size_t)(rows ? rows[blockIdx.x] : blockIdx.x) * W;
  float mean, rstd;
  row_moments_256(xr, W, eps, s4, mean, rstd);
  for (int c = threadIdx.x; c < W; c += 256) out[(size_t)blockIdx.x * W + c] = fmaf((xr[c] - mean) * rstd, w[c], b[c]);
}

// ---- the seam between two sublayers of a layer-norm design.  y_t = the sublayer's output for token t: one row, or the sum over the token's `top` expert
// rows (router weights already applied) plus the shared expert's row.  x_t <- x_t + mult * (LN(y_t) * w_post + b_post);  out_t = LN(x_t) * w_next + b_next
// (the next sublayer's input; skipped without w_next: the stream is changed before the next norm, or the model ends).  One workgroup per token.
struct AffineSeamArgs {
  float* x;                  // [T][W]
  const float* y;            // [T * top][W]
  int top;
  const float* ysh;          // [T][W] (nullptr: no shared expert)
  float* ytmp;               // [T][W] scratch
  const float *w_post, *b_post;
  float mult;
  const float *w_next, *b_next;
  float* out;                // [T][W]
  int W; float eps;
};
constexpr int SEAM_REG = 16;      // widths up to 256 * SEAM_REG keep a token's row in registers between the passes (same sums in the same order as the scratch form)
__global__ __launch_bounds__(256) void affine_seam_kernel(AffineSeamArgs a) {
  __shared__ float s4[4];
  const size_t t = blockIdx.x;
  float* xt = a.x + t * a.W;
  if (a.W <= 256 * SEAM_REG) {
    float v[SEAM_REG], s = 0.f;
#pragma unroll
    for (int k = 0; k < SEAM_REG; k++) {
      const int c = threadIdx.x + 256 * k;
      float y = 0.f;
      if (c < a.W) {
        for (int j = 0; j < a.top; j++) y += a.y[(t * a.top + j) * a.W + c];
        if (a.ysh) y += a.ysh[t * a.W + c];
        s += y;
      }
      v[k] = y;
    }
    float mean = block_sum_256(s, s4) / (float)a.W, q = 0.f;
#pragma unroll
    for (int k = 0; k < SEAM_REG; k++) if (threadIdx.x + 256 * k < a.W) { const float d = v[k] - mean; q = fmaf(d, d, q); }
    float rstd = 1.0f / sqrtf(block_sum_256(q, s4) / (float)a.W + a.eps);
    s = 0.f;
#pragma unroll
    for (int k = 0; k < SEAM_REG; k++) {
      const int c = threadIdx.x + 256 * k;
      if (c < a.W) { v[k] = fmaf(a.mult, fmaf((v[k] - mean) * rstd, a.w_post[c], a.b_post[c]), xt[c]); xt[c] = v[k]; s += v[k]; }
    }
    if (!a.w_next) return;
    mean = block_sum_256(s, s4) / (float)a.W; q = 0.f;
#pragma unroll
    for (int k = 0; k < SEAM_REG; k++) if (threadIdx.x + 256 * k < a.W) { const float d = v[k] - mean; q = fmaf(d, d, q); }
    rstd = 1.0f / sqrtf(block_sum_256(q, s4) / (float)a.W + a.eps);
#pragma unroll
    for (int k = 0; k < SEAM_REG; k++) {
      const int c = threadIdx.x + 256 * k;
      if (c < a.W) a.out[t * a.W + c] = fmaf((v[k] - mean) * rstd, a.w_next[c], a.b_next[c]);
    }
    return;
  }
  float* yt = a.ytmp + t * a.W;
  for (int c = threadIdx.x; c < a.W; c += 256) {
    float v = 0.f;
    for (int k = 0; k < a.top; k++) v += a.y[(t * a.top + k) * a.W + c];
    if (a.ysh) v += a.ysh[t * a.W + c];
    yt[c] = v;
  }
  float mean, rstd;
  row_moments_256(yt, a.W, a.eps, s4, mean, rstd);      // (a thread reads back only what it wrote)
  for (int c = threadIdx.x; c < a.W; c += 256) xt[c] = fmaf(a.mult, fmaf((yt[c] - mean) * rstd, a.w_post[c], a.b_post[c]), xt[c]);
  if (!a.w_next) return;
  row_moments_256(xt, a.W, a.eps, s4, mean, rstd);
  for (int c = threadIdx.x; c < a.W; c += 256) a.out[t * a.W + c] = fmaf((xt[c] - mean) * rstd, a.w_next[c], a.b_next[c]);
}

// ---- sigmoid attention with mixed heads.  For the query token i and every key j it sees (a sliding window, a chunk, or all before it: stack_meta.h):
//   w_g(i, j) = sigmoid(q_g(i) . k_kv(g)(j) * scale + pb[g])          per query head g, not normalised over the keys
//   w'_h(i, j) = sum_g talk[h][g] w_g(i, j)                            the heads' weights mixed (talk nullptr: w' = w)
//   out_h(i) = sum_j w'_h(i, j) v_kv(h)(j)                             head h keeps its own key / value head
// and out_h is multiplied by sigmoid(gate) per channel where a gate is given.  Every key, also those of the step's own tokens, is read from the pool.
// One workgroup per token (and per share of its keys in the split form).  Keys are taken KT at a time:
//   scores   the tile's (key, head) pairs are dealt to the threads: a key row against the head's query (queries in LDS, read as broadcasts), sigmoid
//   mix      the pairs again: a pair's mixed weight from its key's `heads` weights in LDS
//   values   a thread owns NPT output channels (head, c), or NPT slices of eight channels where rows are 16-byte aligned (VEC): it walks the tile's keys,
//            reading weights from LDS and value rows coalesced from the pool
// Nothing is normalised, so the shares of a divided window are simply added (sigmoid_mix_merge_kernel, in split order).
struct MixAttnArgs {
  const float* q; long long ldq;        // head h of token t at q + t * ldq + h * dim
  const void* poolK; const void* poolV; // [pages][page_tokens][kv_heads * dim], [pages][page_tokens][kv_heads * vdim]
  const float* pb;                      // [heads] (nullptr: no bias)
  const float* talk;                    // [heads][heads] (nullptr: heads are not mixed)
  const float* gate; long long ldg;     // gate pre-activation of (t, h, c) at gate + t * ldg + h * vdim + c (nullptr: none)
  float* out; long long ldo;            // [T][heads * vdim]
  int heads, kv_heads, dim, vdim, kt;   // kt: keys per tile (<= 256)
  float scale;
  int mask_kind, mask_size;
  float* part; int nsplit, keys_per;    // split form: part [T][nsplit][heads * vdim]; split z takes keys_per keys from the first visible key on
};
inline size_t mix_attn_lds_bytes(int heads, int dim, int kt) { return ((size_t)heads * dim + 2 * (size_t)heads * kt + (size_t)heads * heads) * 4 + (size_t)kt * 4; }
template <int DT, int NPT, bool VEC, bool SPLIT>
__global__ __launch_bounds__(256) void sigmoid_mix_attn_kernel(StepMeta m, MixAttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) float s_mix[];
  const int H = a.heads, G = a.kv_heads, qpg = H / G, KT = a.kt, tid = threadIdx.x;
  float* s_q = s_mix;                        // [H][dim]
  float* s_w = s_q + (size_t)H * a.dim;      // [H][KT] sigmoid weights
  float* s_w2 = s_w + (size_t)H * KT;        // [H][KT] mixed weights
  float* s_t = s_w2 + (size_t)H * KT;        // [H][H]
  int* s_slot = reinterpret_cast<int*>(s_t + (size_t)H * H);      // [KT] pool row of the tile's keys
  const int t = blockIdx.x, row = m.tok_row[t], pos = m.tok_pos[t];
  int k0 = first_key(pos, a.mask_kind, a.mask_size), k1 = pos + 1;
  if (SPLIT) { k0 = min(k1, k0 + (int)blockIdx.y * a.keys_per); k1 = min(k1, k0 + a.keys_per); }
  const float* q = a.q + (size_t)t * a.ldq;
  for (int i = tid; i < H * a.dim; i += 256) s_q[i] = q[i];
  if (a.talk) for (int i = tid; i < H * H; i += 256) s_t[i] = a.talk[i];
  const int kd = G * a.dim, vd = G * a.vdim, O = H * a.vdim, pmask = (1 << m.page_shift) - 1;
  const elem_t<DT>* pk = reinterpret_cast<const elem_t<DT>*>(a.poolK);
  const elem_t<DT>* pv = reinterpret_cast<const elem_t<DT>*>(a.poolV);
  // a thread's outputs: NPT channels (tid + 256 n), or with VEC NPT slices of eight neighbouring channels of one head (slice tid + 256 n)
  constexpr int CW = VEC ? 8 : 1;
  float acc[NPT][CW];
  int oh[NPT], ov[NPT];      // the output's head and its (first) column in a value row
#pragma unroll
  for (int n = 0; n < NPT; n++) {
    const int o = (tid + 256 * n) * CW, h = o < O ? o / a.vdim : 0;
#pragma unroll
    for (int e = 0; e < CW; e++) acc[n][e] = 0.f;
    oh[n] = h; ov[n] = (h / qpg) * a.vdim + (o < O ? o - h * a.vdim : 0);
  }
  for (int kb = k0; kb < k1; kb += KT) {
    const int nk = min(KT, k1 - kb);
    __syncthreads();                         // queries staged; the previous tile's weights and rows have been read
    if (tid < nk) {
      const int j = kb + tid;
      const int page = m.tbl[(size_t)row * m.tbl_stride + (j >> m.page_shift)];
      s_slot[tid] = (page << m.page_shift) + (j & pmask);
    }
    __syncthreads();
    for (int i = tid; i < nk * H; i += 256) {      // scores: one (key, head) pair per thread and round; neighbours take neighbouring keys of one head
      const int g = i / nk, jj = i - g * nk;
      const elem_t<DT>* kc = pk + (size_t)s_slot[jj] * kd + (size_t)(g / qpg) * a.dim;
      const float* qg = s_q + (size_t)g * a.dim;
      float s = 0.f;
      if (VEC) {
#pragma unroll 4
        for (int d = 0; d < a.dim; d += 8) {      // (several slices in flight: a step of few tokens is bound by the latency of these loads)
          float f[8];
          slice_unpack<DT>(load_slice<DT>(kc, (size_t)(d >> 3)), f);
          const f32x4 qa = *reinterpret_cast<const f32x4*>(qg + d), qb = *reinterpret_cast<const f32x4*>(qg + d + 4);
#pragma unroll
          for (int e = 0; e < 4; e++) s = fmaf(qa[e], f[e], s);
#pragma unroll
          for (int e = 0; e < 4; e++) s = fmaf(qb[e], f[4 + e], s);
        }
      } else {
        for (int d = 0; d < a.dim; d++) s = fmaf(qg[d], elem_to_f32<DT>(kc[d]), s);
      }
      s = fmaf(s, a.scale, a.pb ? a.pb[g] : 0.f);
      s_w[(size_t)g * KT + jj] = 1.0f / (1.0f + expf(-s));
    }
    __syncthreads();
    if (a.talk) {
      for (int i = tid; i < nk * H; i += 256) {    // mix: every (key, head) pair reads its key's weights of all heads
        const int h = i / nk, jj = i - h * nk;
        float v = 0.f;
        for (int g = 0; g < H; g++) v = fmaf(s_t[h * H + g], s_w[(size_t)g * KT + jj], v);
        s_w2[(size_t)h * KT + jj] = v;
      }
      __syncthreads();
    }
    const float* sw = a.talk ? s_w2 : s_w;
#pragma unroll 4
    for (int jj = 0; jj < nk; jj++) {
      const elem_t<DT>* vr = pv + (size_t)s_slot[jj] * vd;
#pragma unroll
      for (int n = 0; n < NPT; n++) {
        if ((tid + 256 * n) * CW >= O) continue;
        const float wt = sw[(size_t)oh[n] * KT + jj];
        if constexpr (VEC) {
          float f[8];
          slice_unpack<DT>(load_slice<DT>(vr + ov[n], 0), f);
#pragma unroll
          for (int e = 0; e < 8; e++) acc[n][e] = fmaf(wt, f[e], acc[n][e]);
        } else acc[n][0] = fmaf(wt, elem_to_f32<DT>(vr[ov[n]]), acc[n][0]);
      }
    }
  }
#pragma unroll
  for (int n = 0; n < NPT; n++)
#pragma unroll
    for (int e = 0; e < CW; e++) {
      const int o = (tid + 256 * n) * CW + e;
      if (o >= O) continue;
      if (SPLIT) a.part[((size_t)t * a.nsplit + blockIdx.y) * O + o] = acc[n][e];
      else a.out[(size_t)t * a.ldo + o] = a.gate ? acc[n][e] / (1.0f + expf(-a.gate[(size_t)t * a.ldg + o])) : acc[n][e];
    }
}
__global__ __launch_bounds__(256) void sigmoid_mix_merge_kernel(MixAttnArgs a) {
  const size_t t = blockIdx.x;
  const int O = a.heads * a.vdim;
  for (int o = threadIdx.x + 256 * blockIdx.y; o < O; o += 256 * gridDim.y) {
    float v = 0.f;
#pragma unroll 8
    for (int s = 0; s < a.nsplit; s++) v += a.part[(t * a.nsplit + s) * O + o];
    a.out[t * a.ldo + o] = a.gate ? v / (1.0f + expf(-a.gate[t * a.ldg + o])) : v;
  }
}

}  // namespace tgx
