// stack_attn_mfma.h — latent attention on the matrix cores (16-bit storage; kv_rank a multiple of 128 up to 512).
//
// All heads of a token share one cached latent c_j, so in latent space attention is multi-query attention with head size kv_rank: scores
// s = q' . c_j (q' = the head's query multiplied into latent space, score scale folded in) and output o' = sum_j p_j c_j, which the value
// up-projection turns into the head's values afterwards.  A workgroup owns 32 ROWS = consecutive (token, head) pairs of one entry of the step — two
// tokens x 16 heads of a prompt portion, or the heads of one decoded token — and walks the keys its rows see in tiles of 32:
//   1. S = Q' C^T: the four waves split the latent channels (the contraction), each leaves a partial 32 x 32 tile in LDS
//   2. softmax bookkeeping in fp32, eight rows per wave: sum of the partials, causal mask per row, running maximum / denominator (the denominator
//      starts at exp(sink[head]): a term without key or value), P as two 16-bit terms and the rows' rescale factors back to LDS
//   3. O' += P C: every wave owns kv_rank / 4 output columns; its B operand comes from a second, TRANSPOSED copy of the page ([channel][token]: eight
//      consecutive keys of a channel are one 16-byte load) that the append kernel writes beside the row-major one
// Q' enters as two 16-bit terms (one with option act.round16), like every activation of the matrix-core products.  Key tiles never straddle a page
// (pages hold a multiple of 32 tokens).  SPLIT: blockIdx.z takes a range of the keys and leaves (m, l, O') records for latent_attn_merge_kernel.
#pragma once
#include "prefill.h"
#include "stack.h"

namespace tgx {

struct LatentMfmaArgs {
  const float* q;        // [T * heads][rank]
  const void* pool;      // [pages][page][rank]
  const void* poolT;     // [pages][rank][page]
  const float* sink;     // [heads] (nullptr: the softmax has no sink)
  float* out;            // [T * heads][rank]
  float* part; int nsplit, keys_per;      // keys_per: a multiple of 32
  int rank, heads, terms;
  int mask_kind, mask_size;      // MASK_*: a row at position i sees the keys [first_key(i), i] (stack_meta.h); the walk starts at the key tile that holds the first row's first key
};

template <int DT, int NT, bool SPLIT>      // NT = rank / 128: 32-column output tiles per wave
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(StepMeta m, LatentMfmaArgs a) {
  constexpr int RQ = 32 * NT, KS = 2 * NT;      // latent channels per wave; 16-channel steps of its share of the contraction
  __shared__ float s_part[4][32][33];
  __shared__ __attribute__((aligned(16))) bf16_t s_ph[32][40], s_pl[32][40];
  __shared__ float s_corr[32], s_l[32];
  const int e = blockIdx.y, H = a.heads;
  const int cnt = m.ent_count[e], start = m.ent_start[e], slot = m.ent_row[e];
  const int nrows = cnt * H, r0 = blockIdx.x * 32;
  if (r0 >= nrows) return;
  const int past = m.tok_pos[start];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, half = lane >> 5, l31 = lane & 31;
  const int kmax = past + min(r0 + 31, nrows - 1) / H + 1;      // keys of the tile's last row
  int k0 = first_key(past + r0 / H, a.mask_kind, a.mask_size) & ~31, k1 = kmax;
  if (SPLIT) { k0 = min(kmax, k0 + (int)blockIdx.z * a.keys_per); k1 = min(kmax, k0 + a.keys_per); }
  const size_t row_base = (size_t)start * H;
  const int page = 1 << m.page_shift;
  const bf16_t* pool = reinterpret_cast<const bf16_t*>(a.pool);
  const bf16_t* poolT = reinterpret_cast<const bf16_t*>(a.poolT);

  // this lane's query row as the A operand of step 1: channels wv * RQ + 16 kk + 8 half .. + 7, as hi / lo terms
  bf16x8 qh[KS], ql[KS];
  {
    const int r = r0 + l31;
    const float* qp = a.q + (row_base + (size_t)min(r, nrows - 1)) * a.rank + wv * RQ + 8 * half;
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(qp + 16 * kk), v1 = *reinterpret_cast<const f32x4*>(qp + 16 * kk + 4);
      bf16_t h[8], l[8];
#pragma unroll
      for (int i = 0; i < 4; i++) { split16<DT>(r < nrows ? v0[i] : 0.f, h[i], l[i]); split16<DT>(r < nrows ? v1[i] : 0.f, h[4 + i], l[4 + i]); }
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

  // softmax bookkeeping: wave wv keeps rows 8 wv .. 8 wv + 7, eight lanes a row, four keys a lane
  const int srow = 8 * wv + (lane >> 3), kq = 4 * (lane & 7);
  const int sr = r0 + srow;
  const bool svalid = sr < nrows;
  const int skeys = svalid ? past + sr / H + 1 : 0;
  const int sfirst = svalid ? first_key(skeys - 1, a.mask_kind, a.mask_size) : 0;
  const bool sinked = a.sink && svalid && (!SPLIT || blockIdx.z == 0);
  float m_s = sinked ? a.sink[sr % H] : -INFINITY, l_s = sinked ? 1.f : 0.f;

  // operand fetches run one phase ahead: the score operands of the NEXT key tile are requested while this tile's softmax and P C run, the P C operands
  // (transposed page) at the top of the tile, ahead of its score products
  auto key_rows = [&](int kt) -> const bf16_t* {
    const size_t pg = (size_t)m.tbl[(size_t)slot * m.tbl_stride + (kt >> m.page_shift)];
    return pool + ((pg << m.page_shift) + (kt & (page - 1)) + l31) * (size_t)a.rank + wv * RQ + 8 * half;
  };
  u32x4 bq[KS];
  if (k0 < k1) {
    const bf16_t* cp = key_rows(k0);
#pragma unroll
    for (int kk = 0; kk < KS; kk++) bq[kk] = *reinterpret_cast<const u32x4*>(cp + 16 * kk);
  }
  for (int kt = k0; kt < k1; kt += 32) {
    const size_t pg = (size_t)m.tbl[(size_t)slot * m.tbl_stride + (kt >> m.page_shift)];
    const int off = kt & (page - 1);
    u32x4 bt[NT][2];
#pragma unroll
    for (int t = 0; t < NT; t++) {
      const bf16_t* tp = poolT + ((pg * a.rank + (size_t)(wv * RQ + 32 * t + l31)) << m.page_shift) + off + 8 * half;
      bt[t][0] = *reinterpret_cast<const u32x4*>(tp); bt[t][1] = *reinterpret_cast<const u32x4*>(tp + 16);
    }
    // 1. partial scores over this wave's channels
    f32x16 s;
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
      const bf16x8 b = __builtin_bit_cast(bf16x8, bq[kk]);
      s = mfma16<DT>(qh[kk], b, s);
      if (a.terms > 1) s = mfma16<DT>(ql[kk], b, s);
    }
    if (kt + 32 < k1) {
      const bf16_t* cp = key_rows(kt + 32);
#pragma unroll
      for (int kk = 0; kk < KS; kk++) bq[kk] = *reinterpret_cast<const u32x4*>(cp + 16 * kk);
    }
#pragma unroll
    for (int r = 0; r < 16; r++) s_part[wv][(r & 3) + 8 * (r >> 2) + 4 * half][l31] = s[r];
    __syncthreads();
    // 2. the rows' softmax state
    {
      float sv[4], tmax = -INFINITY;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float v = s_part[0][srow][kq + c] + s_part[1][srow][kq + c] + s_part[2][srow][kq + c] + s_part[3][srow][kq + c];
        sv[c] = (kt + kq + c < min(skeys, k1) && kt + kq + c >= sfirst) ? v : -INFINITY;
        tmax = fmaxf(tmax, sv[c]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 1, 64)); tmax = fmaxf(tmax, __shfl_xor(tmax, 2, 64)); tmax = fmaxf(tmax, __shfl_xor(tmax, 4, 64));
      const float mn = fmaxf(m_s, tmax);
      const bool dead = mn == -INFINITY;                  // nothing seen yet (a row of another split, or a padding row)
      const float corr = dead ? 1.f : expf(m_s - mn);
      float psum = 0.f;
      bf16_t ph[4], pl[4];
#pragma unroll
      for (int c = 0; c < 4; c++) { const float p = dead ? 0.f : expf(sv[c] - mn); psum += p; split16<DT>(p, ph[c], pl[c]); }
      psum += __shfl_xor(psum, 1, 64); psum += __shfl_xor(psum, 2, 64); psum += __shfl_xor(psum, 4, 64);
      l_s = fmaf(l_s, corr, psum);
      m_s = mn;
      *reinterpret_cast<u32x2*>(&s_ph[srow][kq]) = u32x2{(unsigned int)ph[0] | ((unsigned int)ph[1] << 16), (unsigned int)ph[2] | ((unsigned int)ph[3] << 16)};
      *reinterpret_cast<u32x2*>(&s_pl[srow][kq]) = u32x2{(unsigned int)pl[0] | ((unsigned int)pl[1] << 16), (unsigned int)pl[2] | ((unsigned int)pl[3] << 16)};
      if ((lane & 7) == 0) s_corr[srow] = corr;
    }
    __syncthreads();
    // 3. O' = O' * corr + P C on this wave's columns
    float cr[16];
#pragma unroll
    for (int r = 0; r < 16; r++) cr[r] = s_corr[(r & 3) + 8 * (r >> 2) + 4 * half];
    bf16x8 pa[2], pb[2];
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      pa[kk] = *reinterpret_cast<const bf16x8*>(&s_ph[l31][16 * kk + 8 * half]);
      pb[kk] = *reinterpret_cast<const bf16x8*>(&s_pl[l31][16 * kk + 8 * half]);
    }
#pragma unroll
    for (int t = 0; t < NT; t++) {
#pragma unroll
      for (int r = 0; r < 16; r++) acc[t][r] *= cr[r];
#pragma unroll
      for (int kk = 0; kk < 2; kk++) {
        const bf16x8 b = __builtin_bit_cast(bf16x8, bt[t][kk]);
        acc[t] = mfma16<DT>(pa[kk], b, acc[t]);
        if (a.terms > 1) acc[t] = mfma16<DT>(pb[kk], b, acc[t]);
      }
    }
  }
  if ((lane & 7) == 0) {
    s_l[srow] = l_s;
    if (SPLIT && svalid) {
      float* rec = a.part + ((row_base + sr) * a.nsplit + blockIdx.z) * (size_t)(a.rank + 2);
      rec[0] = m_s; rec[1] = l_s;
    }
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int ri = (r & 3) + 8 * (r >> 2) + 4 * half, gr = r0 + ri, col = wv * RQ + 32 * t + l31;
      if (gr >= nrows) continue;
      if (SPLIT) a.part[((row_base + gr) * a.nsplit + blockIdx.z) * (size_t)(a.rank + 2) + 2 + col] = acc[t][r];
      else a.out[(row_base + gr) * a.rank + col] = s_l[ri] > 0.f ? acc[t][r] / s_l[ri] : 0.f;
    }
}

}  // namespace tgx
