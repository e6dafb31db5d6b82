// stack_gqa.hip — launches of the matrix-core grouped-query attention (kernels/stack_gqa_mfma.h) and of the matrix-core sigmoid attention with mixed heads
// (kernels/stack_mix_mfma.h) of layered models; a translation unit of its own so that
// its template instances compile beside stack.hip.
#include "stack.h"

#include "kernels/stack_gqa_mfma.h"
#include "kernels/stack_mix_mfma.h"

namespace {
template <int DT, int ND, bool SPLIT>
void launch_nt(tgx_ctx* c, const tgx::StepMeta& m, const tgx::GqaMfmaArgs& a, dim3 grid) {
  if (a.vdim <= 128) hipLaunchKernelGGL((tgx::gqa_attn_mfma_kernel<DT, ND, 1, SPLIT>), grid, dim3(256), 0, c->stream, m, a);
  else hipLaunchKernelGGL((tgx::gqa_attn_mfma_kernel<DT, ND, 2, SPLIT>), grid, dim3(256), 0, c->stream, m, a);
}
template <int DT, bool SPLIT>
void launch_nd(tgx_ctx* c, const tgx::StepMeta& m, const tgx::GqaMfmaArgs& a, dim3 grid) {
  switch (a.dim / 64) {
    case 1: launch_nt<DT, 1, SPLIT>(c, m, a, grid); break;
    case 2: launch_nt<DT, 2, SPLIT>(c, m, a, grid); break;
    default: launch_nt<DT, 4, SPLIT>(c, m, a, grid); break;
  }
}
}  // namespace

bool gqa_mfma_shapes_ok(int dt, int dim, int vdim, int page_shift, long long ldq) {
  return dt != tgx::DT_F32 && (dim == 64 || dim == 128 || dim == 256) && vdim % 32 == 0 && vdim >= 32 && vdim <= 256 && page_shift >= 6 && ldq % 4 == 0;
}

void launch_gqa_mfma(tgx_ctx* c, const tgx::StepMeta& m, const tgx::GqaMfmaArgs& a, dim3 grid, bool split) {
  if (!gqa_mfma_shapes_ok(c->dt, a.dim, a.vdim, m.page_shift, a.ldq)) { c->launch_fault = "matrix-core attention: head sizes or storage dtype it does not take"; return; }
  TGX_DT16_SWITCH(c->dt, if (split) launch_nd<DT, true>(c, m, a, grid); else launch_nd<DT, false>(c, m, a, grid);)
}

// ---- sigmoid attention with mixed heads
namespace {
// key / value heads per workgroup: two (half the score products) where the accumulators of their query heads, 16 registers each, still fit beside the
// resident queries: not 8 accumulators beside 16 heads of 128 (they spill)
bool mix_queries_resident(int heads, int dim, int acc_heads) {
  const int hpw = (heads + 3) / 4;
  return (dim == 64 || dim == 128) && hpw <= 4 && !(dim == 128 && hpw > 2 && acc_heads >= 8);
}
int mix_groups_per_wg(int heads, int kv_heads, int dim, int forced) {
  const int qpg = heads / kv_heads;
  if (kv_heads < 2 || qpg > 4) return 1;
  if (forced == 1) return 1;
  const bool res1 = mix_queries_resident(heads, dim, qpg), res2 = mix_queries_resident(heads, dim, 2 * qpg);
  return res1 && !res2 ? 1 : 2;      // resident queries are worth more than shared scores
}
template <int DT, int QPG, int NG>
void launch_mix_q(tgx_ctx* c, const tgx::StepMeta& m, const tgx::MixMfmaArgs& a, dim3 grid) {
  const size_t lds = tgx::mix_mfma_lds_bytes(a.heads, QPG * NG);
  auto go = [&](auto K, auto P) {
    constexpr int KS = decltype(K)::value, HPW = decltype(P)::value;
    auto* fn = &tgx::sigmoid_mix_mfma_kernel<DT, QPG, KS, HPW, NG>;
    if (lds > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(fn, grid, dim3(256), lds, c->stream, m, a);
  };
  // a wave's heads stay in its registers where they fit: key sizes 64 / 128, at most 16 heads
  const int hpw = (a.heads + 3) / 4;
  const bool res = mix_queries_resident(a.heads, a.dim, QPG * NG);
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>; using I2 = std::integral_constant<int, 2>; using I4 = std::integral_constant<int, 4>; using I8 = std::integral_constant<int, 8>;
  if (res && a.dim == 128 && hpw <= 2) go(I8{}, I2{});
  else if (res && a.dim == 128) go(I8{}, I4{});
  else if (res && a.dim == 64 && hpw <= 2) go(I4{}, I2{});
  else if (res && a.dim == 64) go(I4{}, I4{});
  else go(I0{}, I1{});
}
}  // namespace

size_t mix_mfma_wg_lds(int heads, int kv_heads) { return tgx::mix_mfma_lds_bytes(heads, heads / kv_heads * (kv_heads >= 2 && heads / kv_heads <= 4 ? 2 : 1)); }      // (the larger of its forms)

void launch_mix_mfma(tgx_ctx* c, const tgx::StepMeta& m, const tgx::MixMfmaArgs& a, dim3 grid) {
  const int qpg = a.heads / a.kv_heads;
  int ng = mix_groups_per_wg(a.heads, a.kv_heads, a.dim, c->stack->mix_groups);
  if (ng == 2 && c->stack->mix_groups != 2 && (long long)grid.x * grid.y * ((a.kv_heads + 1) / 2) < c->num_cus) ng = 1;      // sharing the scores halves the workgroups: only while they still fill the chip
  grid.z = (a.kv_heads + ng - 1) / ng;
  TGX_DT16_SWITCH(c->dt,
    if (qpg == 1) { if (ng == 2) launch_mix_q<DT, 1, 2>(c, m, a, grid); else launch_mix_q<DT, 1, 1>(c, m, a, grid); }
    else if (qpg == 2) { if (ng == 2) launch_mix_q<DT, 2, 2>(c, m, a, grid); else launch_mix_q<DT, 2, 1>(c, m, a, grid); }
    else if (qpg == 4) { if (ng == 2) launch_mix_q<DT, 4, 2>(c, m, a, grid); else launch_mix_q<DT, 4, 1>(c, m, a, grid); }
    else launch_mix_q<DT, 8, 1>(c, m, a, grid);)
}
