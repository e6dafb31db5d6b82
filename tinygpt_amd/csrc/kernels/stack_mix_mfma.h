// stack_mix_mfma.h — un-normalised sigmoid attention with mixed heads (kernels/stack_loop.h states the mechanism) on the matrix cores, for portions of
// prompts: 16-bit storage; dim a multiple of 16, vdim a multiple of 32 up to 128, 1 / 2 / 4 / 8 query heads per key / value head.
//
// A workgroup owns 32 consecutive tokens of one entry and ONE key / value head c (two, NG, where their accumulators fit the registers and the halved
// grid still fills the chip), and walks the keys its tokens see in tiles of 32:
//   1. S_g = Q_g K_kv(g)^T for EVERY query head g (the mix needs them all), the heads dealt to the four waves; mask and sigmoid (base 2, hardware
//      exponential and reciprocal) in registers, the weights to LDS in fp32.  The queries come as two 16-bit terms (one with option act.round16) from
//      planes the append kernel writes; where a wave's heads fit (HPW heads of KS 16-channel steps, HPW * KS <= 32) they stay in its registers for the
//      whole walk, so a key tile costs the key rows only; otherwise they are streamed per key tile.
//   2. the mixed weights of the group's own heads, w'_h = sum_g talk[h][g] w_g: every thread takes four keys of one token, reads the tile of every head
//      once and keeps the group's sums; they go back to LDS as two 16-bit terms
//   3. O_h += w'_h V_c: every wave owns 32 value columns; its B operand comes from the transposed copy of the value page, shared by the group's heads
// Step 1 is done once per workgroup (the workgroups of a token tile do not exchange anything): kv_heads / NG times the score arithmetic, in exchange
// for accumulators that fit the register file.  Key tiles never straddle a page (pages hold a multiple of 32 tokens).
#pragma once
#include "prefill.h"
#include "stack_meta.h"

namespace tgx {

struct MixMfmaArgs {
  const bf16_t* qh; const bf16_t* ql;   // [T][heads * dim]: the unit queries as 16-bit terms
  const void* poolK;                    // [pages][page][kv_heads * dim]
  const void* poolVT;                   // [pages][kv_heads * vdim][page]
  const float* pb;                      // [heads] score bias (nullptr: none)
  const float* talk;                    // [heads][heads] (nullptr: heads are not mixed)
  const float* gate; long long ldg;     // gate pre-activation of (t, h, c) at gate + t * ldg + h * vdim + c (nullptr: none)
  float* out; long long ldo;            // [T][heads * vdim]
  int heads, kv_heads, dim, vdim, terms;
  float scale;
  int mask_kind, mask_size;
};
constexpr int MIXM_LDW = 32;            // floats per row of a weight tile in LDS
// qpg: the query heads a workgroup sums values for (NG * QPG)
inline size_t mix_mfma_lds_bytes(int heads, int qpg) { return (size_t)heads * 32 * MIXM_LDW * 4 + (size_t)qpg * 2 * 32 * 40 * 2 + (size_t)qpg * heads * 4 + (size_t)heads * 4; }

template <int DT, int QPG, int KS, int HPW, int NG>      // KS = dim / 16 and HPW >= ceil(heads / 4): the wave's queries stay in registers; KS = 0: any shape, queries streamed; NG: key / value heads per workgroup
__global__ __launch_bounds__(256) void sigmoid_mix_mfma_kernel(StepMeta m, MixMfmaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char s_raw[];
  constexpr float LOG2E = 1.4426950408889634f;
  constexpr bool RES = KS > 0;
  constexpr int NH = NG * QPG;      // the query heads whose values this workgroup sums
  const int H = a.heads;
  float* s_w = reinterpret_cast<float*>(s_raw);                                  // [H][32][MIXM_LDW]
  bf16_t* s_ph = reinterpret_cast<bf16_t*>(s_w + (size_t)H * 32 * MIXM_LDW);    // [NH][32][40]
  bf16_t* s_pl = s_ph + NH * 32 * 40;
  float* s_t = reinterpret_cast<float*>(s_pl + NH * 32 * 40);                    // [NH][H]: the rows of the mixing matrix for this workgroup's heads
  float* s_pb = s_t + NH * H;                                                   // [H], in units of log 2 like the scores
  const int e = blockIdx.y, c0 = blockIdx.z * NG;      // key / value heads c0 .. c0 + NG - 1 (those that exist)
  const int cnt = m.ent_count[e], start = m.ent_start[e], slot = m.ent_row[e];
  const int t0 = blockIdx.x * 32;
  if (t0 >= cnt) return;
  const int past = m.tok_pos[start];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, half = lane >> 5, l31 = lane & 31;
  const int kmax = past + min(t0 + 31, cnt - 1) + 1;
  const int k0 = first_key(past + t0, a.mask_kind, a.mask_size) & ~31;
  const int page = 1 << m.page_shift, kd = a.kv_heads * a.dim, vd = a.kv_heads * a.vdim, qd = H * a.dim;
  const bf16_t* poolK = reinterpret_cast<const bf16_t*>(a.poolK);
  const bf16_t* poolVT = reinterpret_cast<const bf16_t*>(a.poolVT);
  for (int i = tid; i < NH * H; i += 256) {
    const int hq = i / H, g = i - hq * H, hd = c0 * QPG + hq;
    s_t[i] = hd >= H ? 0.f : a.talk ? a.talk[(size_t)hd * H + g] : (g == hd ? 1.f : 0.f);
  }
  for (int i = tid; i < H; i += 256) s_pb[i] = a.pb ? a.pb[i] * LOG2E : 0.f;
  const float qscale = a.scale * LOG2E;
  // this lane's token as the A operand's row of step 1
  const size_t qrow = ((size_t)start + (size_t)min(t0 + l31, cnt - 1)) * qd + 8 * half;
  constexpr int RH = RES ? HPW : 1, RK = RES ? KS : 1;
  u32x4 rqh[RH][RK], rql[RH][RK];
  if constexpr (RES) {
#pragma unroll
    for (int i = 0; i < HPW; i++) {
      const int g = min(wv + 4 * i, H - 1);
#pragma unroll
      for (int kk = 0; kk < KS; kk++) {
        rqh[i][kk] = *reinterpret_cast<const u32x4*>(a.qh + qrow + (size_t)g * a.dim + 16 * kk);
        rql[i][kk] = a.terms > 1 ? *reinterpret_cast<const u32x4*>(a.ql + qrow + (size_t)g * a.dim + 16 * kk) : u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
  // the keys each of this lane's 16 accumulator rows (tokens) may see: [lo, hi]; a padding row sees none
  int vlo[16], vhi[16];
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int ri = (r & 3) + 8 * (r >> 2) + 4 * half, p = past + t0 + ri;
    vlo[r] = first_key(p, a.mask_kind, a.mask_size); vhi[r] = t0 + ri < cnt ? p : -1;
  }
  // step 2's share: token srow, keys kq .. kq + 3 of the tile
  const int srow = tid >> 3, kq = 4 * (tid & 7);
  const bool wave_cols = 32 * wv < a.vdim;      // this wave has value columns
  f32x16 acc[NH];
#pragma unroll
  for (int hq = 0; hq < NH; hq++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[hq][r] = 0.f;
  const int ksteps = a.dim >> 4;
  for (int kt = k0; kt < kmax; kt += 32) {
    const size_t pg = (size_t)m.tbl[(size_t)slot * m.tbl_stride + (kt >> m.page_shift)];
    const int off = kt & (page - 1);
    const int key = kt + l31;
    // the value operands of step 3 travel while the scores are made
    u32x4 vb[NG][2];
#pragma unroll
    for (int gi = 0; gi < NG; gi++) {
      vb[gi][0] = u32x4{0u, 0u, 0u, 0u}; vb[gi][1] = u32x4{0u, 0u, 0u, 0u};
      if (wave_cols && c0 + gi < a.kv_heads) {
        const bf16_t* tp = poolVT + ((pg * vd + (size_t)((c0 + gi) * a.vdim + 32 * wv + l31)) << m.page_shift) + off + 8 * half;
        vb[gi][0] = *reinterpret_cast<const u32x4*>(tp); vb[gi][1] = *reinterpret_cast<const u32x4*>(tp + 16);
      }
    }
    const bf16_t* krow = poolK + ((pg << m.page_shift) + off + l31) * (size_t)kd + 8 * half;
    auto finish = [&](const f32x16& s, int g) {      // mask, sigmoid, store
      const float bias = s_pb[g];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ri = (r & 3) + 8 * (r >> 2) + 4 * half;
        const float w = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-fmaf(s[r], qscale, bias)));
        s_w[((size_t)g * 32 + ri) * MIXM_LDW + l31] = (key >= vlo[r] && key <= vhi[r]) ? w : 0.f;
      }
    };
    // 1. scores, mask and sigmoid of this wave's heads
    if constexpr (RES) {
      u32x4 kb[2][KS];      // the key operands of one head travel while the head before is finished
#pragma unroll
      for (int kk = 0; kk < KS; kk++) kb[0][kk] = *reinterpret_cast<const u32x4*>(krow + (size_t)(min(wv, H - 1) / QPG) * a.dim + 16 * kk);
#pragma unroll
      for (int i = 0; i < HPW; i++) {
        const int g = wv + 4 * i;
        if (i + 1 < HPW && g + 4 < H) {
#pragma unroll
          for (int kk = 0; kk < KS; kk++) kb[(i + 1) & 1][kk] = *reinterpret_cast<const u32x4*>(krow + (size_t)((g + 4) / QPG) * a.dim + 16 * kk);
        }
        if (g < H) {
          f32x16 s;
#pragma unroll
          for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
          for (int kk = 0; kk < KS; kk++) {
            const bf16x8 b = __builtin_bit_cast(bf16x8, kb[i & 1][kk]);
            s = mfma16<DT>(__builtin_bit_cast(bf16x8, rqh[i][kk]), b, s);
            if (a.terms > 1) s = mfma16<DT>(__builtin_bit_cast(bf16x8, rql[i][kk]), b, s);
          }
          finish(s, g);
        }
      }
    } else {
      for (int g = wv; g < H; g += 4) {
        const bf16_t* kp = krow + (size_t)(g / QPG) * a.dim;
        const bf16_t* qhp = a.qh + qrow + (size_t)g * a.dim;
        const bf16_t* qlp = a.ql + qrow + (size_t)g * a.dim;
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f;
        for (int kk = 0; kk < ksteps; kk++) {
          const bf16x8 b = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(kp + 16 * kk));
          s = mfma16<DT>(__builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qhp + 16 * kk)), b, s);
          if (a.terms > 1) s = mfma16<DT>(__builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qlp + 16 * kk)), b, s);
        }
        finish(s, g);
      }
    }
    __syncthreads();
    // 2. the group's mixed weights
    {
      float mx[NH][4];
#pragma unroll
      for (int hq = 0; hq < NH; hq++)
#pragma unroll
        for (int k = 0; k < 4; k++) mx[hq][k] = 0.f;
      for (int g = 0; g < H; g++) {
        const f32x4 w4 = *reinterpret_cast<const f32x4*>(&s_w[((size_t)g * 32 + srow) * MIXM_LDW + kq]);
#pragma unroll
        for (int hq = 0; hq < NH; hq++) {
          const float tw = s_t[hq * H + g];
#pragma unroll
          for (int k = 0; k < 4; k++) mx[hq][k] = fmaf(tw, w4[k], mx[hq][k]);
        }
      }
#pragma unroll
      for (int hq = 0; hq < NH; hq++) {
        bf16_t ph[4], pl[4];
#pragma unroll
        for (int k = 0; k < 4; k++) split16<DT>(mx[hq][k], ph[k], pl[k]);
        *reinterpret_cast<u32x2*>(&s_ph[(hq * 32 + srow) * 40 + kq]) = u32x2{(unsigned int)ph[0] | ((unsigned int)ph[1] << 16), (unsigned int)ph[2] | ((unsigned int)ph[3] << 16)};
        *reinterpret_cast<u32x2*>(&s_pl[(hq * 32 + srow) * 40 + kq]) = u32x2{(unsigned int)pl[0] | ((unsigned int)pl[1] << 16), (unsigned int)pl[2] | ((unsigned int)pl[3] << 16)};
      }
    }
    __syncthreads();
    // 3. O_h += w'_h V_c on this wave's 32 value columns
    if (wave_cols) {
#pragma unroll
      for (int hq = 0; hq < NH; hq++) {
        const bf16x8 b0 = __builtin_bit_cast(bf16x8, vb[hq / QPG][0]), b1 = __builtin_bit_cast(bf16x8, vb[hq / QPG][1]);
        const bf16_t* pa = &s_ph[(hq * 32 + l31) * 40 + 8 * half];
        const bf16_t* pl = &s_pl[(hq * 32 + l31) * 40 + 8 * half];
        acc[hq] = mfma16<DT>(*reinterpret_cast<const bf16x8*>(pa), b0, acc[hq]);
        acc[hq] = mfma16<DT>(*reinterpret_cast<const bf16x8*>(pa + 16), b1, acc[hq]);
        if (a.terms > 1) {
          acc[hq] = mfma16<DT>(*reinterpret_cast<const bf16x8*>(pl), b0, acc[hq]);
          acc[hq] = mfma16<DT>(*reinterpret_cast<const bf16x8*>(pl + 16), b1, acc[hq]);
        }
      }
    }
  }
  if (!wave_cols) return;
#pragma unroll
  for (int hq = 0; hq < NH; hq++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int ri = (r & 3) + 8 * (r >> 2) + 4 * half;
      if (t0 + ri >= cnt || c0 * QPG + hq >= H) continue;
      const size_t tk = (size_t)start + t0 + ri, o = (size_t)(c0 * QPG + hq) * a.vdim + 32 * wv + l31;
      a.out[tk * a.ldo + o] = a.gate ? acc[hq][r] / (1.0f + expf(-a.gate[tk * a.ldg + o])) : acc[hq][r];
    }
}

}  // namespace tgx
