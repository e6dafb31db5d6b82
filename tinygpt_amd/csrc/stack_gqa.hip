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
template <int DT, int QPG>
void launch_mix_q(tgx_ctx* c, const tgx::StepMeta& m, const tgx::MixMfmaArgs& a, dim3 grid) {
  const size_t lds = tgx::mix_mfma_lds_bytes(a.heads, QPG);
  auto go = [&](auto K, auto P) {
    constexpr int KS = decltype(K)::value, HPW = decltype(P)::value;
    auto* fn = &tgx::sigmoid_mix_mfma_kernel<DT, QPG, KS, HPW>;
    if (lds > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(fn, grid, dim3(256), lds, c->stream, m, a);
  };
  // a wave's heads stay in its registers where they fit: key sizes 64 / 128, at most 16 heads (8 at key size 128 ... 32 steps in all)
  const int hpw = (a.heads + 3) / 4;
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>; using I2 = std::integral_constant<int, 2>; using I4 = std::integral_constant<int, 4>; using I8 = std::integral_constant<int, 8>;
  if (a.dim == 128 && hpw <= 2) go(I8{}, I2{});
  else if (a.dim == 128 && hpw <= 4) go(I8{}, I4{});
  else if (a.dim == 64 && hpw <= 2) go(I4{}, I2{});
  else if (a.dim == 64 && hpw <= 4) go(I4{}, I4{});
  else go(I0{}, I1{});
}
}  // namespace

void launch_mix_mfma(tgx_ctx* c, const tgx::StepMeta& m, const tgx::MixMfmaArgs& a, dim3 grid) {
  const int qpg = a.heads / a.kv_heads;
  TGX_DT16_SWITCH(c->dt,
    if (qpg == 1) launch_mix_q<DT, 1>(c, m, a, grid);
    else if (qpg == 2) launch_mix_q<DT, 2>(c, m, a, grid);
    else if (qpg == 4) launch_mix_q<DT, 4>(c, m, a, grid);
    else launch_mix_q<DT, 8>(c, m, a, grid);)
}
