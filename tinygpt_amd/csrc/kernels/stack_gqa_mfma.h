// stack_gqa_mfma.h — grouped-query attention over the paged key / value pool on the matrix cores (16-bit storage; dim a multiple of 64 up to 256, vdim a
// multiple of 32 up to 256).
//
// The query heads of one key / value head read the same cached rows, so a workgroup owns 32 ROWS = consecutive (token, query head of the group) pairs of
// one entry of the step and one key / value head — eight tokens x four heads of a prompt portion, or the group's heads of one decoded token — and walks the
// keys its rows see in tiles of 64 (the scheme of latent_attn_mfma_kernel, with separate key and value operands and two of its key tiles per barrier pair):
//   1. S = Q K^T: the four waves split the head's dim channels (the contraction), each leaves a partial 32 x 64 tile in LDS
//   2. softmax bookkeeping in fp32, eight rows per wave: sum of the partials, causal mask per row, running maximum / denominator (the denominator
//      starts at exp(sink) where the design has a sink: a term without key or value), P as two 16-bit terms and the rows' rescale factors back to LDS
//   3. O += P V: every wave owns 32 NT of the vdim output columns; its B operand comes from a TRANSPOSED copy of the value page ([channel][token]: eight
//      consecutive keys of a channel are one 16-byte load) that the append kernel writes
// Q (score scale and log2 e folded in: the softmax runs in base 2 on the hardware exponential, as in the other families' prompt attention) enters as two 16-bit
// terms (one with option act.round16).  Key tiles never straddle a page (pages hold a multiple of 64
// tokens).  The output is multiplied by sigmoid(gate) where a gate is given.  SPLIT: blockIdx.z takes a range of the keys and leaves (m, l, O) records
// for gqa_attn_merge_kernel.
#pragma once
#include "prefill.h"
#include "stack_meta.h"

namespace tgx {

struct GqaMfmaArgs {
  const float* q; long long ldq;       // head h of token t at q + t * ldq + h * dim
  const void* poolK;                   // [pages][page][kv_heads * dim]
  const void* poolVT;                  // [pages][kv_heads * vdim][page]
  const float* gate; long long ldg;    // gate pre-activation of (t, h, c) at gate + t * ldg + h * vdim + c (nullptr: none)
  float* out; long long ldo;           // [T][heads * vdim]
  float* part; int nsplit, keys_per;   // keys_per: a multiple of 64
  int heads, kv_heads, dim, vdim, terms;
  float scale, sink; int has_sink;
  int mask_kind, mask_size;            // MASK_* (stack_meta.h): a row sees the keys [first_key(position), position]
  float softcap; int dist_bias;        // score shaping as in gqa_attn_kernel (softcap <= 0: none)
};

template <int DT, int ND, int NT, bool SPLIT>      // ND = dim / 64: 16-channel steps of a wave's share of the contraction; NT = ceil(vdim / 128): 32-column output tiles per wave
__global__ __launch_bounds__(256) void gqa_attn_mfma_kernel(StepMeta m, GqaMfmaArgs a) {
  constexpr int RQ = 16 * ND, KS = ND;
  constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;
  const bool capped = a.softcap > 0.f;
  const float qscale = capped ? a.scale : a.scale * LOG2E;      // a capped score is needed in natural units first
  __shared__ float s_part[4][32][65];
  __shared__ __attribute__((aligned(16))) bf16_t s_ph[32][72], s_pl[32][72];
  __shared__ float s_corr[32], s_l[32];
  const int e = blockIdx.y / a.kv_heads, kvh = blockIdx.y - e * a.kv_heads, Gq = a.heads / a.kv_heads;
  const int cnt = m.ent_count[e], start = m.ent_start[e], slot = m.ent_row[e];
  const int nrows = cnt * Gq, r0 = blockIdx.x * 32;
  if (r0 >= nrows) return;
  const int past = m.tok_pos[start];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, half = lane >> 5, l31 = lane & 31;
  const int kmax = past + min(r0 + 31, nrows - 1) / Gq + 1;      // keys of the tile's last row
  const int klo = first_key(past + r0 / Gq, a.mask_kind, a.mask_size) & ~63;      // the tile's first row sees the oldest key; whole key tiles
  int k0 = klo, k1 = kmax;
  if (SPLIT) { k0 = min(kmax, klo + (int)blockIdx.z * a.keys_per); k1 = min(kmax, k0 + a.keys_per); }
  const int page = 1 << m.page_shift, kd = a.kv_heads * a.dim, vd = a.kv_heads * a.vdim;
  const bf16_t* poolK = reinterpret_cast<const bf16_t*>(a.poolK) + (size_t)kvh * a.dim;
  const bf16_t* poolVT = reinterpret_cast<const bf16_t*>(a.poolVT);

  // this lane's query row as the A operand of step 1: channels wv * RQ + 16 kk + 8 half .. + 7, as hi / lo terms
  bf16x8 qh[KS], ql[KS];
  {
    const int r = r0 + l31, rc = min(r, nrows - 1);
    const float* qp = a.q + (size_t)(start + rc / Gq) * a.ldq + (size_t)(kvh * Gq + rc % Gq) * a.dim + wv * RQ + 8 * half;
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(qp + 16 * kk), v1 = *reinterpret_cast<const f32x4*>(qp + 16 * kk + 4);
      bf16_t h[8], l[8];
#pragma unroll
      for (int i = 0; i < 4; i++) { split16<DT>(r < nrows ? v0[i] * qscale : 0.f, h[i], l[i]); split16<DT>(r < nrows ? v1[i] * qscale : 0.f, h[4 + i], l[4 + i]); }
      u32x4 uh, ul;
#pragma unroll
      for (int i = 0; i < 4; i++) { uh[i] = (unsigned int)h[2 * i] | ((unsigned int)h[2 * i + 1] << 16); ul[i] = (unsigned int)l[2 * i] | ((unsigned int)l[2 * i + 1] << 16); }
      qh[kk] = __builtin_bit_cast(bf16x8, uh); ql[kk] = __builtin_bit_cast(bf16x8, ul);
    }
  }
  f32x16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[t][r] = 0.f;

  // softmax bookkeeping: wave wv keeps rows 8 wv .. 8 wv + 7, eight lanes a row, eight keys a lane
  const int srow = 8 * wv + (lane >> 3), kq = 8 * (lane & 7);
  const int sr = r0 + srow;
  const bool svalid = sr < nrows;
  const int skeys = svalid ? past + sr / Gq + 1 : 0;
  const int slo = first_key(skeys - 1, a.mask_kind, a.mask_size);
  const float slope2 = a.dist_bias && svalid ? distance_slope(kvh * Gq + sr % Gq, a.heads) * LOG2E : 0.f;
  const bool sinked = a.has_sink && svalid && (!SPLIT || blockIdx.z == 0);
  float m_s = sinked ? a.sink * LOG2E : -INFINITY, l_s = sinked ? 1.f : 0.f;      // the running maximum in base-2 units

  auto key_rows = [&](int kt) -> const bf16_t* {
    const size_t pg = (size_t)m.tbl[(size_t)slot * m.tbl_stride + (kt >> m.page_shift)];
    return poolK + ((pg << m.page_shift) + (kt & (page - 1)) + l31) * (size_t)kd + wv * RQ + 8 * half;
  };
  u32x4 bq[2][KS];
  if (k0 < k1) {
    const bf16_t* cp = key_rows(k0);
#pragma unroll
    for (int kk = 0; kk < KS; kk++) { bq[0][kk] = *reinterpret_cast<const u32x4*>(cp + 16 * kk); bq[1][kk] = *reinterpret_cast<const u32x4*>(cp + 32 * (size_t)kd + 16 * kk); }
  }
  for (int kt = k0; kt < k1; kt += 64) {
    const size_t pg = (size_t)m.tbl[(size_t)slot * m.tbl_stride + (kt >> m.page_shift)];
    const int off = kt & (page - 1);
    u32x4 bt[NT][4];
#pragma unroll
    for (int t = 0; t < NT; t++) {
      const int col = min(wv * 32 * NT + 32 * t + l31, a.vdim - 1);
      const bf16_t* tp = poolVT + ((pg * vd + (size_t)(kvh * a.vdim + col)) << m.page_shift) + off + 8 * half;
#pragma unroll
      for (int kk = 0; kk < 4; kk++) bt[t][kk] = *reinterpret_cast<const u32x4*>(tp + 16 * kk);
    }
    // 1. partial scores over this wave's channels, keys kt .. kt + 31 and kt + 32 .. kt + 63
    f32x16 s[2];
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) {
#pragma unroll
      for (int r = 0; r < 16; r++) s[h2][r] = 0.f;
#pragma unroll
      for (int kk = 0; kk < KS; kk++) {
        const bf16x8 b = __builtin_bit_cast(bf16x8, bq[h2][kk]);
        s[h2] = mfma16<DT>(qh[kk], b, s[h2]);
        if (a.terms > 1) s[h2] = mfma16<DT>(ql[kk], b, s[h2]);
      }
    }
    if (kt + 64 < k1) {
      const bf16_t* cp = key_rows(kt + 64);
#pragma unroll
      for (int kk = 0; kk < KS; kk++) { bq[0][kk] = *reinterpret_cast<const u32x4*>(cp + 16 * kk); bq[1][kk] = *reinterpret_cast<const u32x4*>(cp + 32 * (size_t)kd + 16 * kk); }
    }
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
      for (int r = 0; r < 16; r++) s_part[wv][(r & 3) + 8 * (r >> 2) + 4 * half][32 * h2 + l31] = s[h2][r];
    __syncthreads();
    // 2. the rows' softmax state
    {
      float sv[8], tmax = -INFINITY;
#pragma unroll
      for (int c = 0; c < 8; c++) {
        float v = s_part[0][srow][kq + c] + s_part[1][srow][kq + c] + s_part[2][srow][kq + c] + s_part[3][srow][kq + c];
        const int key = kt + kq + c;
        if (capped) v = a.softcap * tanhf(v / a.softcap) * LOG2E;
        v = fmaf(-slope2, (float)(skeys - 1 - key), v);
        sv[c] = (key >= slo && key < min(skeys, k1)) ? v : -INFINITY;
        tmax = fmaxf(tmax, sv[c]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 1, 64)); tmax = fmaxf(tmax, __shfl_xor(tmax, 2, 64)); tmax = fmaxf(tmax, __shfl_xor(tmax, 4, 64));
      const float mn = fmaxf(m_s, tmax);
      const bool dead = mn == -INFINITY;                  // nothing seen yet (a row of another split, or a padding row)
      const float corr = dead ? 1.f : __builtin_amdgcn_exp2f(m_s - mn);
      float psum = 0.f;
      bf16_t ph[8], pl[8];
#pragma unroll
      for (int c = 0; c < 8; c++) { const float p = dead ? 0.f : __builtin_amdgcn_exp2f(sv[c] - mn); psum += p; split16<DT>(p, ph[c], pl[c]); }
      psum += __shfl_xor(psum, 1, 64); psum += __shfl_xor(psum, 2, 64); psum += __shfl_xor(psum, 4, 64);
      l_s = fmaf(l_s, corr, psum);
      m_s = mn;
      u32x4 uh, ul;
#pragma unroll
      for (int i = 0; i < 4; i++) { uh[i] = (unsigned int)ph[2 * i] | ((unsigned int)ph[2 * i + 1] << 16); ul[i] = (unsigned int)pl[2 * i] | ((unsigned int)pl[2 * i + 1] << 16); }
      *reinterpret_cast<u32x4*>(&s_ph[srow][kq]) = uh;
      *reinterpret_cast<u32x4*>(&s_pl[srow][kq]) = ul;
      if ((lane & 7) == 0) s_corr[srow] = corr;
    }
    __syncthreads();
    // 3. O = O * corr + P V on this wave's columns
    float cr[16];
#pragma unroll
    for (int r = 0; r < 16; r++) cr[r] = s_corr[(r & 3) + 8 * (r >> 2) + 4 * half];
    bf16x8 pa[4], pb[4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
      pa[kk] = *reinterpret_cast<const bf16x8*>(&s_ph[l31][16 * kk + 8 * half]);
      pb[kk] = *reinterpret_cast<const bf16x8*>(&s_pl[l31][16 * kk + 8 * half]);
    }
#pragma unroll
    for (int t = 0; t < NT; t++) {
      if (wv * 32 * NT + 32 * t >= a.vdim) continue;      // (wave-uniform: this wave has no columns in the tile)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[t][r] *= cr[r];
#pragma unroll
      for (int kk = 0; kk < 4; kk++) {
        const bf16x8 b = __builtin_bit_cast(bf16x8, bt[t][kk]);
        acc[t] = mfma16<DT>(pa[kk], b, acc[t]);
        if (a.terms > 1) acc[t] = mfma16<DT>(pb[kk], b, acc[t]);
      }
    }
  }
  auto rec_of = [&](int gr) -> float* {      // the split record of row gr: indexed by (token, head) like the lane kernel's
    return a.part + (((size_t)(start + gr / Gq) * a.heads + (size_t)(kvh * Gq + gr % Gq)) * a.nsplit + blockIdx.z) * (size_t)(a.vdim + 2);
  };
  if ((lane & 7) == 0) {
    s_l[srow] = l_s;
    if (SPLIT && svalid) { float* rec = rec_of(sr); rec[0] = m_s * LN2; rec[1] = l_s; }      // the merge kernel works in natural units
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int ri = (r & 3) + 8 * (r >> 2) + 4 * half, gr = r0 + ri, col = wv * 32 * NT + 32 * t + l31;
      if (gr >= nrows || col >= a.vdim) continue;
      if (SPLIT) rec_of(gr)[2 + col] = acc[t][r];
      else {
        const size_t tok = (size_t)(start + gr / Gq), hc = (size_t)(kvh * Gq + gr % Gq) * a.vdim + col;
        float v = s_l[ri] > 0.f ? acc[t][r] / s_l[ri] : 0.f;
        if (a.gate) v = v / (1.0f + expf(-a.gate[tok * a.ldg + hc]));
        a.out[tok * a.ldo + hc] = v;
      }
    }
}

}  // namespace tgx
