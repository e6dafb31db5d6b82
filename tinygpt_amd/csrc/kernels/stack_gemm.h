// stack_gemm.h — the matrix products of layered models: C = epilogue(A · Bᵀ) with fp32 activations A [M][K] and stored weights B [N][K].
//   16-bit storage: v_mfma_f32_32x32x16 on the activation's two 16-bit terms (x = hi + lo, 16 significant bits) — or its rounded first term alone
//   (option act.round16) — against the stored weight, fp32 accumulation; fp32 storage: v_mfma_f32_32x32x2_f32, nothing rounded.
// One kernel serves plain, batched and grouped products:
//   batched (blockIdx.z = head):   B advances by b_zstride, the A / C columns by a_zoff / c_zoff per z — per-head products on slices of wide rows
//   grouped (experts):             blockIdx.y walks a tile list (expert, first row) built on the device (moe_plan_kernel); rows are gathered through
//                                  a_rows and scattered through c_rows
//   dual:                          two weight matrices against the same activation tile (an expert's gate and up projections), combined in the epilogue
// Workgroup = 4 waves as 2 x 2, each WT x WT tiles of 32 x 32: 64 WT x 64 WT outputs per workgroup, K in steps of 64 (32 for fp32 storage) staged through LDS with the
// next step's global loads in flight under the MFMAs.  Any M, N, K: rows, columns and the K tail are masked; shapes that break the 16-byte
// alignment of the vector loads take element loads (VEC = false).
#pragma once
#include "prefill.h"

namespace tgx {

enum { SG_ACT_NONE = 0, SG_ACT_TANH = 1, SG_ACT_DECAY = 2, SG_ACT_GELU = 3 };
enum { SG_STORE = 0, SG_ADD = 1, SG_GATE = 2, SG_EXPERT_ACT = 3, SG_ROWSCALE = 4, SG_SILU_MUL = 5 };
constexpr bool sg_dual(int epi) { return epi == SG_EXPERT_ACT || epi == SG_SILU_MUL; }
struct StackGemmArgs {
  const float* A; long long lda; int a_zoff;
  const int* a_rows;
  const void* B; const void* B2; long long ldb; long long b_zstride;
  float* C; long long ldc; int c_zoff;
  const int* c_rows;
  const int* z_off; const int* tile_z; const int* tile_m0; const int* n_tiles;      // grouped
  int M, N, K;
  float scale;                 // SG_STORE: C = act(acc * scale + bias); SG_ADD: C += acc * scale
  int act;                     // SG_STORE: SG_ACT_NONE, SG_ACT_TANH, SG_ACT_DECAY = exp(-exp(v)) (a decay in (0, 1) from a log-log pre-activation), or
                               //           SG_ACT_GELU = v (1 + erf(v / sqrt 2)) / 2
  const float* bias;           // SG_STORE: [N] per z (column z * c_zoff + n), nullptr: none
  int gate_col0, gate_heads;   // SG_STORE: columns [gate_col0, + gate_heads) leave as log input gates cap tanh(v / cap), the next gate_heads columns as log forget gates
  float gate_cap;              //           logsigmoid(cap tanh(v / cap)) (the two gate rows of a matrix-memory layer's input product); gate_heads 0: none
  float limit;                 // SG_EXPERT_ACT
  const float* G; long long ldg; int g_col0;     // SG_GATE: C = acc * sigmoid(G[row][g_col0 + z * c_zoff + n]), or with g_per_z
  int g_per_z;                                   //          one gate per batch member z (a head): sigmoid(G[row][g_col0 + z])
  const float* rw;             // SG_ROWSCALE: C = acc * rw[c row]
  int terms;                   // 16-bit storage: 2 = hi + lo, 1 = hi only
};

// an expert's activation: g = min(gate, limit), u = clamp(up, -limit, limit); g * sigmoid(1.702 g) * (u + 1)
__device__ __forceinline__ float expert_act(float gate, float up, float limit) {
  const float g = fminf(gate, limit), u = fminf(fmaxf(up, -limit), limit);
  return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
}
// log-space gates of a matrix-memory layer: soft cap, and log sigmoid in the form that loses nothing for large |z|
__device__ __forceinline__ float soft_cap(float z, float cap) { return cap * tanhf(z / cap); }
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float store_value(const StackGemmArgs& a, float v, size_t bias_at, int n) {
  float o = a.bias ? fmaf(v, a.scale, a.bias[bias_at]) : v * a.scale;
  if (a.gate_heads > 0 && n >= a.gate_col0) { o = soft_cap(o, a.gate_cap); if (n >= a.gate_col0 + a.gate_heads) o = log_sigmoid(o); }
  if (a.act == SG_ACT_TANH) o = tanhf(o);
  else if (a.act == SG_ACT_DECAY) o = expf(-expf(o));
  else if (a.act == SG_ACT_GELU) o = 0.5f * o * (1.0f + erff(o * 0.70710678118654752f));
  return o;
}
// the plain gated expert: silu(gate) * up
__device__ __forceinline__ float silu_mul(float gate, float up) { return gate / (1.0f + expf(-gate)) * up; }

template <int DT, int EPI, bool DUAL, int WT, bool VEC>
__global__ __launch_bounds__(256) void stack_gemm_kernel(const StackGemmArgs a) {
  constexpr bool F32 = DT == DT_F32;
  constexpr int BM = 64 * WT, BN = 64 * WT, BK = F32 ? 32 : 64;      // 16-bit tiles take 64 k per step: half the barriers, twice the bytes in flight
  constexpr int ACH = BK / 4, BCH = F32 ? BK / 4 : BK / 8;            // 16-byte chunks per staged row
  constexpr int LDK = BK + 8;                       // 16-bit tiles: row-major, k contiguous, 16 bytes of padding
  constexpr int LDA = BM + 1, LDB = BN + 1;         // fp32 tiles: k-major
  constexpr int NB = DUAL ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16_t* sAh = reinterpret_cast<bf16_t*>(smem);
  bf16_t* sAl = sAh + BM * LDK;
  bf16_t* sB = sAl + BM * LDK;                      // [NB][BN][LDK]
  float* fA = reinterpret_cast<float*>(smem);       // [BK][LDA]
  float* fB = fA + BK * LDA;                        // [NB][BK][LDB]

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, wm = wv >> 1, wn = wv & 1;
  int z, mbase, mend;
  if (a.z_off) {
    if ((int)blockIdx.y >= *a.n_tiles) return;
    z = a.tile_z[blockIdx.y]; mbase = a.tile_m0[blockIdx.y]; mend = a.z_off[z + 1];
  } else { z = blockIdx.z; mbase = blockIdx.y * BM; mend = a.M; }
  const int n0 = blockIdx.x * BN;
  const float* Ab = a.A + (size_t)z * a.a_zoff;
  const elem_t<DT>* Bz[NB];
  Bz[0] = reinterpret_cast<const elem_t<DT>*>(a.B) + (size_t)z * a.b_zstride;
  if constexpr (DUAL) Bz[1] = reinterpret_cast<const elem_t<DT>*>(a.B2) + (size_t)z * a.b_zstride;

  f32x16 acc[NB][WT][WT];
#pragma unroll
  for (int b = 0; b < NB; b++)
#pragma unroll
    for (int i = 0; i < WT; i++)
#pragma unroll
      for (int j = 0; j < WT; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[b][i][j][r] = 0.f;

  // ---- staging maps.  A: chunks of 4 k (fp32) -> chunk c: row c / ACH, k 4 (c % ACH).  B: 16-bit chunks of 8 k -> row c / BCH, k 8 (c % BCH); fp32 as A.
  constexpr int AI = BM * (BK / 4) / 256;
  constexpr int BI = F32 ? BN * (BK / 4) / 256 : BN * (BK / 8) / 256;
  f32x4 ra[AI];
  f32x4 rbf[F32 ? NB * BI : 1];
  u32x4 rbh[F32 ? 1 : NB * BI];
  size_t arow[AI];
#pragma unroll
  for (int i = 0; i < AI; i++) {
    const int m = mbase + (tid + 256 * i) / ACH;
    const int mc = min(m, mend - 1);
    arow[i] = (size_t)(a.a_rows ? a.a_rows[mc] : mc) * a.lda;
  }
  auto load_tiles = [&](int k0) {
#pragma unroll
    for (int i = 0; i < AI; i++) {
      const int k = k0 + 4 * ((tid + 256 * i) % ACH);
      const float* p = Ab + arow[i] + k;
      if (VEC) ra[i] = k < a.K ? *reinterpret_cast<const f32x4*>(p) : f32x4{0.f, 0.f, 0.f, 0.f};
      else
#pragma unroll
        for (int e = 0; e < 4; e++) ra[i][e] = k + e < a.K ? p[e] : 0.f;
    }
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
      for (int i = 0; i < BI; i++) {
        const int c = tid + 256 * i;
        if constexpr (F32) {
          const int n = min(n0 + c / BCH, a.N - 1), k = k0 + 4 * (c % BCH);
          const float* p = reinterpret_cast<const float*>(Bz[b]) + (size_t)n * a.ldb + k;
          if (VEC) rbf[b * BI + i] = k < a.K ? *reinterpret_cast<const f32x4*>(p) : f32x4{0.f, 0.f, 0.f, 0.f};
          else
#pragma unroll
            for (int e = 0; e < 4; e++) rbf[b * BI + i][e] = k + e < a.K ? p[e] : 0.f;
        } else {
          const int n = min(n0 + c / BCH, a.N - 1), k = k0 + 8 * (c % BCH);
          const bf16_t* p = reinterpret_cast<const bf16_t*>(Bz[b]) + (size_t)n * a.ldb + k;
          if (VEC) rbh[b * BI + i] = k < a.K ? *reinterpret_cast<const u32x4*>(p) : u32x4{0u, 0u, 0u, 0u};
          else {
            u32x4 v = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int e = 0; e < 8; e++) if (k + e < a.K) v[e >> 1] |= (unsigned int)p[e] << (16 * (e & 1));
            rbh[b * BI + i] = v;
          }
        }
      }
  };
  auto store_tiles = [&]() {
#pragma unroll
    for (int i = 0; i < AI; i++) {
      const int c = tid + 256 * i, row = c / ACH, kc = c % ACH;
      if constexpr (F32) {
#pragma unroll
        for (int e = 0; e < 4; e++) fA[(4 * kc + e) * LDA + row] = ra[i][e];
      } else {
        bf16_t h[4], l[4];
#pragma unroll
        for (int e = 0; e < 4; e++) split16<DT>(ra[i][e], h[e], l[e]);
        *reinterpret_cast<u32x2*>(sAh + row * LDK + 4 * kc) = u32x2{(unsigned int)h[0] | ((unsigned int)h[1] << 16), (unsigned int)h[2] | ((unsigned int)h[3] << 16)};
        *reinterpret_cast<u32x2*>(sAl + row * LDK + 4 * kc) = u32x2{(unsigned int)l[0] | ((unsigned int)l[1] << 16), (unsigned int)l[2] | ((unsigned int)l[3] << 16)};
      }
    }
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
      for (int i = 0; i < BI; i++) {
        const int c = tid + 256 * i;
        if constexpr (F32) {
          const int row = c / BCH, kc = c % BCH;
#pragma unroll
          for (int e = 0; e < 4; e++) fB[(b * BK + 4 * kc + e) * LDB + row] = rbf[b * BI + i][e];
        } else {
          const int row = c / BCH, kc = c % BCH;
          *reinterpret_cast<u32x4*>(sB + ((size_t)b * BN + row) * LDK + 8 * kc) = rbh[b * BI + i];
        }
      }
  };

  load_tiles(0);
  for (int k0 = 0; k0 < a.K; k0 += BK) {
    __syncthreads();
    store_tiles();
    __syncthreads();
    if (k0 + BK < a.K) load_tiles(k0 + BK);
    if constexpr (F32) {
#pragma unroll
      for (int kk = 0; kk < BK / 2; kk++) {
        const int krow = 2 * kk + (lane >> 5);
        float fa[WT], fb[NB][WT];
#pragma unroll
        for (int i = 0; i < WT; i++) fa[i] = fA[krow * LDA + wm * (32 * WT) + i * 32 + (lane & 31)];
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
          for (int j = 0; j < WT; j++) fb[b][j] = fB[(b * BK + krow) * LDB + wn * (32 * WT) + j * 32 + (lane & 31)];
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
          for (int i = 0; i < WT; i++)
#pragma unroll
            for (int j = 0; j < WT; j++) acc[b][i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[b][j], acc[b][i][j], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < BK / 16; kk++) {
        const int kof = 16 * kk + 8 * (lane >> 5);
        bf16x8 ah[WT], al[WT], bb[NB][WT];
#pragma unroll
        for (int i = 0; i < WT; i++) {
          const int row = wm * (32 * WT) + i * 32 + (lane & 31);
          ah[i] = *reinterpret_cast<const bf16x8*>(sAh + row * LDK + kof);
          al[i] = *reinterpret_cast<const bf16x8*>(sAl + row * LDK + kof);
        }
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
          for (int j = 0; j < WT; j++) bb[b][j] = *reinterpret_cast<const bf16x8*>(sB + ((size_t)b * BN + wn * (32 * WT) + j * 32 + (lane & 31)) * LDK + kof);
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
          for (int i = 0; i < WT; i++)
#pragma unroll
            for (int j = 0; j < WT; j++) {
              acc[b][i][j] = mfma16<DT>(ah[i], bb[b][j], acc[b][i][j]);
              if (a.terms > 1) acc[b][i][j] = mfma16<DT>(al[i], bb[b][j], acc[b][i][j]);
            }
      }
    }
  }

  // ---- epilogue.  C / D layout of the 32 x 32 product: column = lane & 31, row = (r & 3) + 8 (r >> 2) + 4 (lane >> 5)
#pragma unroll
  for (int i = 0; i < WT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int m = mbase + wm * (32 * WT) + i * 32 + (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5);
      if (m >= mend) continue;
      const size_t crow = a.c_rows ? (size_t)a.c_rows[m] : (size_t)m;
      float* cp = a.C + crow * a.ldc + (size_t)z * a.c_zoff;
#pragma unroll
      for (int j = 0; j < WT; j++) {
        const int n = n0 + wn * (32 * WT) + j * 32 + (lane & 31);
        if (n >= a.N) continue;
        const float v = acc[0][i][j][r];
        if constexpr (EPI == SG_STORE) cp[n] = store_value(a, v, (size_t)z * a.c_zoff + n, n);
        else if constexpr (EPI == SG_ADD) cp[n] = fmaf(v, a.scale, cp[n]);
        else if constexpr (EPI == SG_GATE) cp[n] = v / (1.0f + expf(-a.G[crow * a.ldg + a.g_col0 + (a.g_per_z ? (size_t)z : (size_t)z * a.c_zoff + n)]));
        else if constexpr (EPI == SG_EXPERT_ACT) cp[n] = expert_act(v, acc[NB - 1][i][j][r], a.limit);
        else if constexpr (EPI == SG_SILU_MUL) cp[n] = silu_mul(v, acc[NB - 1][i][j][r]);
        else cp[n] = v * a.rw[crow];
      }
    }
}

template <int DT, bool DUAL, int WT>
constexpr size_t stack_gemm_lds() {
  constexpr int BM = 64 * WT, BN = 64 * WT, BK = DT == DT_F32 ? 32 : 64, NB = DUAL ? 2 : 1;
  return DT == DT_F32 ? (size_t)(BK * (BM + 1) + NB * BK * (BN + 1)) * 4 : (size_t)(2 * BM + NB * BN) * (BK + 8) * 2;
}

}  // namespace tgx

namespace tgx {

// output columns per wave of the few-row kernel (four for eight-row tiles was measured slower: 16 rows x 8 layers at width 2048 6.6k -> 6.2k tokens/s)
constexpr int stack_gemv_cols(int, bool) { return 2; }

// ---- the same products for a FEW rows (decode steps): a weight-streaming kernel.  One wave per pair of output columns: every lane takes 8 weights of each
// column per pass (one 16-byte load for the 16-bit dtypes) against the 8 activations of up to MR rows, fp32 FMA chains, one cross-lane sum per (row, column)
// at the end.  Same argument block, batching (blockIdx.z), grouping (tile list with tiles of MR rows) and epilogues as stack_gemm_kernel; the activations
// enter in fp32 (rounded to the storage dtype first under option act.round16).  Needs the vector-load alignment (K a multiple of 8).
template <int DT, int EPI, bool DUAL, int MR>
__global__ __launch_bounds__(256) void stack_gemv_kernel(const StackGemmArgs a) {
  constexpr int NC = stack_gemv_cols(MR, DUAL), NB = DUAL ? 2 : 1;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  int z, mbase, mend;
  if (a.z_off) {
    if ((int)blockIdx.y >= *a.n_tiles) return;
    z = a.tile_z[blockIdx.y]; mbase = a.tile_m0[blockIdx.y]; mend = min(a.z_off[z + 1], mbase + MR);
  } else { z = blockIdx.z; mbase = blockIdx.y * MR; mend = min(a.M, mbase + MR); }
  const int n0 = (blockIdx.x * 4 + wv) * NC;
  if (n0 >= a.N) return;
  const float* Ab = a.A + (size_t)z * a.a_zoff;
  const float* arow[MR];
#pragma unroll
  for (int r = 0; r < MR; r++) { const int mc = min(mbase + r, mend - 1); arow[r] = Ab + (size_t)(a.a_rows ? a.a_rows[mc] : mc) * a.lda; }
  const elem_t<DT>* wrow[NB][NC];
#pragma unroll
  for (int b = 0; b < NB; b++)
#pragma unroll
    for (int j = 0; j < NC; j++)
      wrow[b][j] = reinterpret_cast<const elem_t<DT>*>(b ? a.B2 : a.B) + (size_t)z * a.b_zstride + (size_t)min(n0 + j, a.N - 1) * a.ldb;
  float acc[NB][NC][MR];
#pragma unroll
  for (int b = 0; b < NB; b++)
#pragma unroll
    for (int j = 0; j < NC; j++)
#pragma unroll
      for (int r = 0; r < MR; r++) acc[b][j][r] = 0.f;
  const int round16 = a.terms == 1;
  const int nsl = a.K >> 3;                               // 8-element slices of a row
  for (int s0 = lane; s0 < nsl; s0 += 128) {              // two slices per lane and pass: twice the loads in flight
    const int s1 = s0 + 64;
    const bool two = s1 < nsl;
    Slice8<DT> w0[NB][NC], w1[NB][NC];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
      for (int j = 0; j < NC; j++) { w0[b][j] = load_slice_nt<DT>(wrow[b][j], (size_t)s0); w1[b][j] = load_slice_nt<DT>(wrow[b][j], (size_t)(two ? s1 : s0)); }
#pragma unroll
    for (int r = 0; r < MR; r++) {
      const f32x4* xp = reinterpret_cast<const f32x4*>(arow[r]);
      f32x4 xa = xp[2 * s0], xb = xp[2 * s0 + 1], ya = xp[2 * (two ? s1 : s0)], yb = xp[2 * (two ? s1 : s0) + 1];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        xa[i] = round_storage_if<DT>(xa[i], round16); xb[i] = round_storage_if<DT>(xb[i], round16);
        ya[i] = two ? round_storage_if<DT>(ya[i], round16) : 0.f; yb[i] = two ? round_storage_if<DT>(yb[i], round16) : 0.f;
      }
#pragma unroll
      for (int b = 0; b < NB; b++)
#pragma unroll
        for (int j = 0; j < NC; j++) { acc[b][j][r] = dot8<DT>(acc[b][j][r], w0[b][j], xa, xb); acc[b][j][r] = dot8<DT>(acc[b][j][r], w1[b][j], ya, yb); }
    }
  }
#pragma unroll
  for (int b = 0; b < NB; b++)
#pragma unroll
    for (int j = 0; j < NC; j++)
#pragma unroll
      for (int r = 0; r < MR; r++) acc[b][j][r] = wave_sum(acc[b][j][r]);
  if (lane != 0) return;
#pragma unroll
  for (int r = 0; r < MR; r++) {
    const int m = mbase + r;
    if (m >= mend) break;
    const size_t crow = a.c_rows ? (size_t)a.c_rows[m] : (size_t)m;
    float* cp = a.C + crow * a.ldc + (size_t)z * a.c_zoff;
#pragma unroll
    for (int j = 0; j < NC; j++) {
      const int n = n0 + j;
      if (n >= a.N) break;
      const float v = acc[0][j][r];
      if constexpr (EPI == SG_STORE) cp[n] = store_value(a, v, (size_t)z * a.c_zoff + n, n);
      else if constexpr (EPI == SG_ADD) cp[n] = fmaf(v, a.scale, cp[n]);
      else if constexpr (EPI == SG_GATE) cp[n] = v / (1.0f + expf(-a.G[crow * a.ldg + a.g_col0 + (a.g_per_z ? (size_t)z : (size_t)z * a.c_zoff + n)]));
      else if constexpr (EPI == SG_EXPERT_ACT) cp[n] = expert_act(v, acc[NB - 1][j][r], a.limit);
      else if constexpr (EPI == SG_SILU_MUL) cp[n] = silu_mul(v, acc[NB - 1][j][r]);
      else cp[n] = v * a.rw[crow];
    }
  }
}

}  // namespace tgx
