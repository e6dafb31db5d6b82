// stack.hip — layered models behind the C ABI (include/tgx.h tgx_create_stack / tgx_step_ragged): creation from a per-layer description, weight upload by
// checkpoint name, the paged latent pool and the slots' convolution state, the ragged engine step, and the decode loop on top of the shared sampler.
//
// One step = T tokens of S entries (a portion of a prompt, or one decoded token, per sequence slot).  Per layer:
//   norm_conv (norm1, canon1) -> one product for [queries | latent | gate] -> latent norm + pool append -> queries into latent space (per head)
//   -> latent attention over the pool -> value up-projection with the sigmoid gate in its epilogue -> output product added to the stream
//   -> norm_conv (norm2, canon2) -> router top-k -> grouped expert products (gate / up with the activation, down with the router weight)
//   -> combine + depth average.
// Attention reads every key from the pool — also the keys of the step's own tokens, appended before it runs — so a position's result does not depend
// on how its sequence was cut into steps.  The residual stream, norms, scores and the router are fp32; the matrices and the pool are in the storage dtype.
#include "stack.h"

#include "kernels/stack.h"
#include "kernels/stack_gemm.h"
#include "kernels/stack_attn_mfma.h"
#include "kernels/stack_seq.h"
#include "kernels/stack_gqa_mfma.h"
#include "kernels/stack_rec.h"
#include "kernels/stack_loop.h"
#include "kernels/stack_mix_mfma.h"

int upload_param_ext(tgx_ctx* c, ebyte* dst, const void* host, int64_t n, int src_dtype);      // abi.hip

namespace {

float half_bits_to_f32(uint16_t h) {
  const uint32_t s = (h >> 15) & 1, e = (h >> 10) & 0x1f, m = h & 0x3ff;
  float v = e == 0 ? ldexpf((float)m, -24) : e == 31 ? (m ? NAN : INFINITY) : ldexpf((float)(m | 0x400), (int)e - 25);
  return s ? -v : v;
}
std::vector<float> to_f32(const void* host, int64_t n, int src_dtype) {
  std::vector<float> out((size_t)n);
  for (int64_t i = 0; i < n; i++) {
    if (src_dtype == TGX_F32) out[(size_t)i] = ((const float*)host)[i];
    else if (src_dtype == TGX_BF16) { const uint32_t u = (uint32_t)((const uint16_t*)host)[i] << 16; memcpy(&out[(size_t)i], &u, 4); }
    else out[(size_t)i] = half_bits_to_f32(((const uint16_t*)host)[i]);
  }
  return out;
}
int upload_f32(tgx_ctx* c, float* dst, const void* host, int64_t n, int src_dtype) {
  const std::vector<float> v = to_f32(host, n, src_dtype);
  HIP_OK(c, hipMemcpy(dst, v.data(), (size_t)n * 4, hipMemcpyHostToDevice));
  return TGX_OK;
}
size_t esize(int src_dtype) { return src_dtype == TGX_F32 ? 4 : 2; }

struct MetaPtrs { int *tok_id, *tok_pos, *tok_ent, *tok_row, *tok_idx, *tok_cnt, *tok_par, *ent_row, *ent_start, *ent_count, *ent_par, *want, *want_row; size_t n; };
MetaPtrs meta_layout(int* base, int T, int S, int NW) {
  MetaPtrs p;
  p.tok_id = base; p.tok_pos = p.tok_id + T; p.tok_ent = p.tok_pos + T; p.tok_row = p.tok_ent + T; p.tok_idx = p.tok_row + T; p.tok_cnt = p.tok_idx + T; p.tok_par = p.tok_cnt + T;
  p.ent_row = p.tok_par + T; p.ent_start = p.ent_row + S; p.ent_count = p.ent_start + S; p.ent_par = p.ent_count + S;
  p.want = p.ent_par + S; p.want_row = p.want + NW;
  p.n = (size_t)7 * T + (size_t)4 * S + (size_t)2 * NW;
  return p;
}
tgx::StepMeta step_meta(const StackModel* sm, const MetaPtrs& p, int T, int S) {
  tgx::StepMeta m{};
  m.tok_id = p.tok_id; m.tok_pos = p.tok_pos; m.tok_ent = p.tok_ent; m.tok_row = p.tok_row; m.tok_idx = p.tok_idx; m.tok_cnt = p.tok_cnt; m.tok_par = p.tok_par; m.ent_row = p.ent_row; m.ent_start = p.ent_start; m.ent_count = p.ent_count; m.ent_par = p.ent_par;
  m.tbl = sm->tbl_dev; m.tbl_stride = sm->tbl_stride; m.page_shift = sm->page_shift; m.T = T; m.S = S;
  return m;
}

// ---- the products --------------------------------------------------------------------------------------------------------------------------
template <int DT, int EPI, bool DUAL>
void launch_gemm_t(tgx_ctx* c, const tgx::StackGemmArgs& a, dim3 grid1, dim3 grid2, int wt, bool vec) {
  auto go = [&](auto WTc, auto VECc) {
    constexpr int WT = decltype(WTc)::value; constexpr bool VEC = decltype(VECc)::value;
    const size_t lds = tgx::stack_gemm_lds<DT, DUAL, WT>();
    hipLaunchKernelGGL((tgx::stack_gemm_kernel<DT, EPI, DUAL, WT, VEC>), WT == 1 ? grid1 : grid2, dim3(256), lds, c->stream, a);
  };
  if (wt == 1) { if (vec) go(std::integral_constant<int, 1>{}, std::true_type{}); else go(std::integral_constant<int, 1>{}, std::false_type{}); }
  else { if (vec) go(std::integral_constant<int, 2>{}, std::true_type{}); else go(std::integral_constant<int, 2>{}, std::false_type{}); }
}
template <int DT, int EPI, bool DUAL>
void launch_gemv_t(tgx_ctx* c, const tgx::StackGemmArgs& a, dim3 grid, int mr) {
  switch (mr) {
    case 1: hipLaunchKernelGGL((tgx::stack_gemv_kernel<DT, EPI, DUAL, 1>), grid, dim3(256), 0, c->stream, a); break;
    case 2: hipLaunchKernelGGL((tgx::stack_gemv_kernel<DT, EPI, DUAL, 2>), grid, dim3(256), 0, c->stream, a); break;
    case 4: hipLaunchKernelGGL((tgx::stack_gemv_kernel<DT, EPI, DUAL, 4>), grid, dim3(256), 0, c->stream, a); break;
    default: hipLaunchKernelGGL((tgx::stack_gemv_kernel<DT, EPI, DUAL, 8>), grid, dim3(256), 0, c->stream, a); break;
  }
}
// rows per tile of a grouped product's plan (moe_plan_kernel tile_m): steps of few (token, expert) pairs stream the experts through the few-row kernel
constexpr int GROUPED_FEW_PAIRS = 128, GROUPED_FEW_ROWS = 4, FEW_ROWS_MAX = 16;
constexpr int FEW_COLS_ANY_ROWS = 64;      // a matrix of so few rows (the router's) is streamed per eight-row tile whatever the step's size: the 64-wide matrix-core tiles would stand mostly empty
// (both products of the layer must be able to take it: their contraction lengths, the width and the expert width, in whole 8-element slices)
int grouped_tile_rows(const tgx_ctx* c, int pairs, int width, int ff) {
  return c->stack->gemv && pairs <= GROUPED_FEW_PAIRS && width % 8 == 0 && ff % 8 == 0 ? GROUPED_FEW_ROWS : 64;
}

// nz: batched products (blockIdx.z); grouped products pass the number of their rows and groups (the device-side tile list says how many tiles are real)
void launch_gemm(tgx_ctx* c, tgx::StackGemmArgs a, int epi, int nz, int grouped_rows = 0, int groups = 0, int grouped_tile = 64, int dt = -1) {
  const StackModel* sm = c->stack;
  if (dt < 0) dt = c->dt;      // (the router's weights are fp32 whatever the storage dtype)
  if (a.M <= 0 && !a.z_off) return;
  if (a.N <= 0 || a.K <= 0) return;
  a.terms = c->act16 ? 1 : 2;
  const int kq = dt == tgx::DT_F32 ? 4 : 8;
  const bool vec = a.K % kq == 0 && a.ldb % kq == 0 && a.b_zstride % kq == 0 && a.lda % 4 == 0 && a.a_zoff % 4 == 0 && ((uintptr_t)a.A % 16 == 0) && ((uintptr_t)a.B % 16 == 0) &&
                   (!a.B2 || (uintptr_t)a.B2 % 16 == 0);
  const bool dual = tgx::sg_dual(epi);
  // few rows: the weight-streaming kernel (its loads take whole 8-element slices)
  const bool few = sm->gemv && vec && a.K % 8 == 0 && a.ldb % 8 == 0 && a.b_zstride % 8 == 0 && (a.z_off ? grouped_tile == GROUPED_FEW_ROWS : (a.M <= FEW_ROWS_MAX || a.N <= FEW_COLS_ANY_ROWS));
  if (a.z_off && grouped_tile == GROUPED_FEW_ROWS && !few) { c->launch_fault = "grouped product: the plan was made for the few-row kernel, which these operands cannot take"; return; }
  if (few) {
    const int mr = a.z_off ? GROUPED_FEW_ROWS : (a.M <= 1 ? 1 : a.M <= 2 ? 2 : a.M <= 4 ? 4 : 8);
    const int cols = 4 * tgx::stack_gemv_cols(mr, dual);      // per workgroup
    const dim3 grid((a.N + cols - 1) / cols, a.z_off ? grouped_rows / mr + groups : (a.M + mr - 1) / mr, a.z_off ? 1 : nz);
    TGX_DT_SWITCH(dt,
      switch (epi) {
        case tgx::SG_STORE: launch_gemv_t<DT, tgx::SG_STORE, false>(c, a, grid, mr); break;
        case tgx::SG_ADD: launch_gemv_t<DT, tgx::SG_ADD, false>(c, a, grid, mr); break;
        case tgx::SG_GATE: launch_gemv_t<DT, tgx::SG_GATE, false>(c, a, grid, mr); break;
        case tgx::SG_ROWSCALE: launch_gemv_t<DT, tgx::SG_ROWSCALE, false>(c, a, grid, mr); break;
        case tgx::SG_SILU_MUL: launch_gemv_t<DT, tgx::SG_SILU_MUL, true>(c, a, grid, mr); break;
        default: if (dual) launch_gemv_t<DT, tgx::SG_EXPERT_ACT, true>(c, a, grid, mr); break;
      })
    return;
  }
  int wt;
  dim3 g1, g2;
  if (a.z_off) {      // grouped: the tile list is built for 64-row tiles
    wt = 1;
    g1 = dim3((a.N + 63) / 64, grouped_rows / 64 + groups, 1);
  } else {
    g1 = dim3((a.N + 63) / 64, (a.M + 63) / 64, nz);
    g2 = dim3((a.N + 127) / 128, (a.M + 127) / 128, nz);
    wt = (size_t)g2.x * g2.y * g2.z >= 2 * (size_t)c->num_cus ? 2 : 1;      // the wide tile once it fills the chip twice over: fewer, larger tiles hide less latency
    if (sm->gemm_wt) wt = sm->gemm_wt;
  }
  TGX_DT_SWITCH(dt,
    switch (epi) {
      case tgx::SG_STORE: launch_gemm_t<DT, tgx::SG_STORE, false>(c, a, g1, g2, wt, vec); break;
      case tgx::SG_ADD: launch_gemm_t<DT, tgx::SG_ADD, false>(c, a, g1, g2, wt, vec); break;
      case tgx::SG_GATE: launch_gemm_t<DT, tgx::SG_GATE, false>(c, a, g1, g2, wt, vec); break;
      case tgx::SG_ROWSCALE: launch_gemm_t<DT, tgx::SG_ROWSCALE, false>(c, a, g1, g2, wt, vec); break;
      case tgx::SG_SILU_MUL: launch_gemm_t<DT, tgx::SG_SILU_MUL, true>(c, a, g1, g2, wt, vec); break;
      default: if (dual) launch_gemm_t<DT, tgx::SG_EXPERT_ACT, true>(c, a, g1, g2, wt, vec); break;
    })
}

template <int DT, bool SPLIT>
void launch_attn_t(tgx_ctx* c, const tgx::StepMeta& m, const tgx::LatentAttnArgs& a, dim3 grid) {
  const size_t lds = (size_t)4 * a.rank * 4;
  const int rpl = (a.rank + 63) / 64;
  if (rpl <= 1) hipLaunchKernelGGL((tgx::latent_attn_kernel<DT, 1, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
  else if (rpl <= 2) hipLaunchKernelGGL((tgx::latent_attn_kernel<DT, 2, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
  else if (rpl <= 4) hipLaunchKernelGGL((tgx::latent_attn_kernel<DT, 4, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
  else if (rpl <= 8) hipLaunchKernelGGL((tgx::latent_attn_kernel<DT, 8, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
  else if (rpl <= 16) hipLaunchKernelGGL((tgx::latent_attn_kernel<DT, 16, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
  else hipLaunchKernelGGL((tgx::latent_attn_kernel<DT, 32, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
}

// the matrix-core attention serves 16-bit storage, latent widths of 128 .. 512 in steps of 128, pages of a multiple of 32 tokens
bool layer_attn_mfma(const tgx_ctx* c, const tgx_layer_desc& l) {
  return c->dt != tgx::DT_F32 && l.kv_rank % 128 == 0 && l.kv_rank <= 512 && c->stack->page_shift >= 5;
}

template <int DT, bool SPLIT>
void launch_attn_mfma_t(tgx_ctx* c, const tgx::StepMeta& m, const tgx::LatentMfmaArgs& a, dim3 grid) {
  switch (a.rank / 128) {
    case 1: hipLaunchKernelGGL((tgx::latent_attn_mfma_kernel<DT, 1, SPLIT>), grid, dim3(256), 0, c->stream, m, a); break;
    case 2: hipLaunchKernelGGL((tgx::latent_attn_mfma_kernel<DT, 2, SPLIT>), grid, dim3(256), 0, c->stream, m, a); break;
    case 3: hipLaunchKernelGGL((tgx::latent_attn_mfma_kernel<DT, 3, SPLIT>), grid, dim3(256), 0, c->stream, m, a); break;
    default: hipLaunchKernelGGL((tgx::latent_attn_mfma_kernel<DT, 4, SPLIT>), grid, dim3(256), 0, c->stream, m, a); break;
  }
}

int ensure_ws(tgx_ctx* c, int T) {
  StackModel* sm = c->stack;
  if (T <= sm->cap_tokens) return TGX_OK;
  HIP_OK(c, hipStreamSynchronize(c->stream));
  auto fr = [](auto*& p) { if (p) (void)hipFree(p); p = nullptr; };
  fr(sm->x); fr(sm->xs); fr(sm->a); fr(sm->proj); fr(sm->ql); fr(sm->lat); fr(sm->o); fr(sm->selw); fr(sm->yh); fr(sm->yd); fr(sm->xn); fr(sm->lg);
  fr(sm->sel); fr(sm->perm); fr(sm->ptok); fr(sm->tile_e); fr(sm->tile_m0); fr(sm->meta_dev); fr(sm->zr);
  fr(sm->a2); fr(sm->ytmp); fr(sm->ysh); fr(sm->sgw); fr(sm->vfirst); fr(sm->hs); fr(sm->mixed); fr(sm->lora); fr(sm->rec_in); fr(sm->xcat); fr(sm->qplanes);
  if (sm->meta_host) { (void)hipHostFree(sm->meta_host); sm->meta_host = nullptr; }
  const int cap = std::max(T, 64);
  const size_t W = (size_t)sm->d.width, n = (size_t)cap;
  int rc;
  if (sm->sandwich) {      // no layer results are kept; the seams need a second normed stream, a scratch row and the mixers' side buffers
    if ((rc = dev_alloc(c, &sm->a2, n * W)) || (rc = dev_alloc(c, &sm->ytmp, n * W)) || (rc = dev_alloc(c, &sm->ysh, n * W)) || (rc = dev_alloc(c, &sm->sgw, n)) ||
        (rc = dev_alloc(c, &sm->vfirst, n * (size_t)std::max(1, sm->max_kvv))) || (rc = dev_alloc(c, &sm->hs, n * (size_t)std::max(1, sm->max_hv)))) return rc;
  } else if (sm->affine) {   // the seam's scratch row, the shared expert's row, the stream beside the embedding output
    if ((rc = dev_alloc(c, &sm->ytmp, n * W)) || (rc = dev_alloc(c, &sm->ysh, n * W)) || (rc = dev_alloc(c, &sm->xcat, 2 * n * W)) ||
        (rc = dev_alloc(c, &sm->qplanes, 2 * n * (size_t)std::max(1, sm->max_qd) + 8))) return rc;
  } else if (sm->joint) {    // the recurrent mixers' side buffers: un-normed outputs, token-shift mixes, the decay's inner product, the delta rule's inputs
    if ((rc = dev_alloc(c, &sm->hs, n * (size_t)std::max(1, sm->max_hv))) || (rc = dev_alloc(c, &sm->mixed, n * (size_t)std::max(1, sm->max_shift))) ||
        (rc = dev_alloc(c, &sm->lora, n * (size_t)std::max(1, sm->max_lora))) || (rc = dev_alloc(c, &sm->rec_in, n * (size_t)std::max(1, sm->max_rec)))) return rc;
  } else if ((rc = dev_alloc(c, &sm->xs, (size_t)(sm->d.layers + 1) * n * W))) return rc;
  if ((rc = dev_alloc(c, &sm->x, n * W)) || (rc = dev_alloc(c, &sm->a, n * W)) ||
      (rc = dev_alloc(c, &sm->proj, n * (size_t)sm->max_in)) || (rc = dev_alloc(c, &sm->ql, n * (size_t)sm->max_hr)) || (rc = dev_alloc(c, &sm->lat, n * (size_t)sm->max_hr)) ||
      (rc = dev_alloc(c, &sm->o, n * (size_t)sm->max_hv)) || (rc = dev_alloc(c, &sm->xn, n * W)) || (rc = dev_alloc(c, &sm->lg, n * (size_t)sm->d.vocab))) return rc;
  if (sm->max_top > 0) {
    const size_t np = n * (size_t)sm->max_top;
    if ((rc = dev_alloc(c, &sm->zr, n * (size_t)(sm->max_E + 1))) || (rc = dev_alloc(c, &sm->selw, np)) || (rc = dev_alloc(c, &sm->sel, np)) || (rc = dev_alloc(c, &sm->perm, np)) || (rc = dev_alloc(c, &sm->ptok, np)) ||
        (rc = dev_alloc(c, &sm->yh, np * (size_t)sm->max_ff + n * (size_t)sm->max_sff)) || (rc = dev_alloc(c, &sm->yd, np * W)) ||
        (rc = dev_alloc(c, &sm->tile_e, std::max<size_t>(np / 64, GROUPED_FEW_PAIRS / GROUPED_FEW_ROWS) + (size_t)sm->max_E + 1)) ||
        (rc = dev_alloc(c, &sm->tile_m0, std::max<size_t>(np / 64, GROUPED_FEW_PAIRS / GROUPED_FEW_ROWS) + (size_t)sm->max_E + 1))) return rc;
  }
  sm->meta_cap = (size_t)9 * n + (size_t)4 * sm->d.max_seqs;
  if ((rc = dev_alloc(c, &sm->meta_dev, sm->meta_cap))) return rc;
  HIP_OK(c, hipHostMalloc((void**)&sm->meta_host, sm->meta_cap * 4, hipHostMallocDefault));
  sm->cap_tokens = cap;
  return TGX_OK;
}

int ensure_part(tgx_ctx* c, size_t elems) {
  StackModel* sm = c->stack;
  if (elems <= sm->part_elems) return TGX_OK;
  HIP_OK(c, hipStreamSynchronize(c->stream));
  if (sm->part) (void)hipFree(sm->part);
  sm->part = nullptr; sm->part_elems = 0;
  int rc = dev_alloc(c, &sm->part, elems);
  if (rc) return rc;
  sm->part_elems = elems;
  return TGX_OK;
}

// the layers of one step; meta is on the device.  max_keys: the longest context any token of the step attends (host knowledge; picks the attention form)
int run_layers_latent(tgx_ctx* c, const MetaPtrs& mp, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx::StepMeta m = step_meta(sm, mp, T, S);
  const int W = sm->d.width, nslots = sm->d.max_seqs, nb = sm->d.canon_taps - 1;
  const size_t slot_stride = (size_t)sm->cap_tokens * W;
  TGX_DT_SWITCH(c->dt, hipLaunchKernelGGL(tgx::sinusoid_embed_kernel<DT>, dim3(T), dim3(256), 0, c->stream, m, reinterpret_cast<const tgx::elem_t<DT>*>(c->embed), sm->freq, sm->x, sm->xs, W))
  for (int li = 0; li < sm->d.layers; li++) {
    StackLayerW& w = sm->L[(size_t)li];
    const tgx_layer_desc& ld = w.d;
    const int H = ld.heads, qd = H * ld.dim, R = ld.kv_rank, vd = H * ld.vdim, nin = qd + R + vd;
    const size_t st_buf = (size_t)nslots * nb * W;
    tgx::NormConvArgs nc{};
    nc.x = sm->x; nc.nw = w.norm1; nc.cw = w.canon1; nc.out = sm->a; nc.state = nb > 0 ? w.conv_state : nullptr; nc.state_buf = st_buf;
    nc.W = W; nc.groups = sm->d.norm_groups; nc.taps = sm->d.canon_taps; nc.eps = sm->d.norm_eps;
    hipLaunchKernelGGL(tgx::norm_conv_kernel, dim3(T), dim3(256), 0, c->stream, m, nc);
    // [q | latent | gate] = a . w_in^T
    tgx::StackGemmArgs g{};
    g.A = sm->a; g.lda = W; g.B = w.w_in; g.ldb = W; g.C = sm->proj; g.ldc = nin; g.M = T; g.N = nin; g.K = W; g.scale = 1.f;
    launch_gemm(c, g, tgx::SG_STORE, 1);
    tgx::LatentAppendArgs la{};
    la.src = sm->proj; la.lds = nin; la.col0 = qd; la.nw = w.lat_norm; la.pool = w.pool; la.poolT = w.poolT; la.rank = R; la.eps = sm->d.norm_eps;
    TGX_DT_SWITCH(c->dt, hipLaunchKernelGGL(tgx::latent_append_kernel<DT>, dim3(T), dim3(64), 0, c->stream, m, la))
    // queries into latent space, head by head: ql[t][h] = scale * q[t][h] . ukT[h]^T
    g = tgx::StackGemmArgs{};
    g.A = sm->proj; g.lda = nin; g.a_zoff = ld.dim; g.B = w.w_ukT; g.ldb = ld.dim; g.b_zstride = (long long)R * ld.dim; g.C = sm->ql; g.ldc = (long long)H * R; g.c_zoff = R;
    g.M = T; g.N = R; g.K = ld.dim; g.scale = ld.scale;
    launch_gemm(c, g, tgx::SG_STORE, H);
    tgx::LatentAttnArgs aa{};
    aa.q = sm->ql; aa.ldq = (long long)H * R; aa.pool = w.pool; aa.sink = w.sink; aa.out = sm->lat; aa.ldo = (long long)H * R; aa.rank = R; aa.heads = H;
    if (w.poolT && sm->attn_mfma) {
      // rows = (token, head) pairs of an entry in tiles of 32; few tiles and a long context: the keys are divided between workgroups
      tgx::LatentMfmaArgs ma{};
      ma.q = sm->ql; ma.pool = w.pool; ma.poolT = w.poolT; ma.sink = w.sink; ma.out = sm->lat; ma.rank = R; ma.heads = H; ma.terms = c->act16 ? 1 : 2;
      const int tiles = (max_count * H + 31) / 32;
      int nsplit = 1;
      if (max_keys >= sm->attn_split_min_keys && (long long)tiles * S < c->num_cus) {
        nsplit = (int)std::min<long long>(64, (2LL * c->num_cus) / ((long long)tiles * S));
        const int per = std::max(64, ((max_keys + nsplit - 1) / nsplit + 31) / 32 * 32);      // two key tiles per workgroup at least
        nsplit = (max_keys + per - 1) / per;
        ma.keys_per = per;
      }
      if (nsplit > 1) {
        int rc = ensure_part(c, (size_t)T * H * nsplit * (size_t)(R + 2));
        if (rc) return rc;
        ma.part = sm->part; ma.nsplit = nsplit;
        aa.part = sm->part; aa.nsplit = nsplit;
        if (c->dt == tgx::DT_F16) launch_attn_mfma_t<tgx::DT_F16, true>(c, m, ma, dim3(tiles, S, nsplit)); else launch_attn_mfma_t<tgx::DT_BF16, true>(c, m, ma, dim3(tiles, S, nsplit));
        hipLaunchKernelGGL(tgx::latent_attn_merge_kernel, dim3(T, H), dim3(256), 0, c->stream, aa);
      } else {
        if (c->dt == tgx::DT_F16) launch_attn_mfma_t<tgx::DT_F16, false>(c, m, ma, dim3(tiles, S)); else launch_attn_mfma_t<tgx::DT_BF16, false>(c, m, ma, dim3(tiles, S));
      }
    } else {
    int nsplit = 1;
    if (max_keys >= sm->attn_split_min_keys && (long long)T * H < 2LL * c->num_cus) {
      nsplit = (int)std::min<long long>(64, (4LL * c->num_cus) / ((long long)T * H));
      const int per = std::max(256, ((max_keys + nsplit - 1) / nsplit + 63) / 64 * 64);
      nsplit = (max_keys + per - 1) / per;
      aa.keys_per = per;
    }
    if (nsplit > 1) {
      int rc = ensure_part(c, (size_t)T * H * nsplit * (size_t)(R + 2));
      if (rc) return rc;
      aa.part = sm->part; aa.nsplit = nsplit;
      TGX_DT_SWITCH(c->dt, (launch_attn_t<DT, true>(c, m, aa, dim3(T, H, nsplit))))
      hipLaunchKernelGGL(tgx::latent_attn_merge_kernel, dim3(T, H), dim3(256), 0, c->stream, aa);
    } else {
      TGX_DT_SWITCH(c->dt, (launch_attn_t<DT, false>(c, m, aa, dim3(T, H))))
    }
    }
    // o[t][h] = (lat[t][h] . uv[h]^T) * sigmoid(gate)
    g = tgx::StackGemmArgs{};
    g.A = sm->lat; g.lda = (long long)H * R; g.a_zoff = R; g.B = w.w_uv; g.ldb = R; g.b_zstride = (long long)ld.vdim * R; g.C = sm->o; g.ldc = vd; g.c_zoff = ld.vdim;
    g.M = T; g.N = ld.vdim; g.K = R; g.G = sm->proj; g.ldg = nin; g.g_col0 = qd + R;
    launch_gemm(c, g, tgx::SG_GATE, H);
    // x += o . w_o^T
    g = tgx::StackGemmArgs{};
    g.A = sm->o; g.lda = vd; g.B = w.w_o; g.ldb = vd; g.C = sm->x; g.ldc = W; g.M = T; g.N = W; g.K = vd; g.scale = 1.f;
    launch_gemm(c, g, tgx::SG_ADD, 1);
    int top = 0;
    if (ld.mlp == TGX_MLP_MOE) {
      top = ld.top;
      nc.nw = w.norm2; nc.cw = w.canon2; nc.state = nb > 0 ? w.conv_state + 2 * st_buf : nullptr;
      hipLaunchKernelGGL(tgx::norm_conv_kernel, dim3(T), dim3(256), 0, c->stream, m, nc);
      // router: fp32 weights, fp32 products (nothing is rounded), then bias, top-k and the softmax over the chosen
      g = tgx::StackGemmArgs{};
      g.A = sm->a; g.lda = W; g.B = w.w_router; g.ldb = W; g.C = sm->zr; g.ldc = ld.experts; g.M = T; g.N = ld.experts; g.K = W; g.scale = 1.f;
      launch_gemm(c, g, tgx::SG_STORE, 1, 0, 0, 64, tgx::DT_F32);
      tgx::RouterArgs ra{};
      ra.z = sm->zr; ra.br = w.b_router; ra.sel = sm->sel; ra.selw = sm->selw; ra.E = ld.experts; ra.top = top;
      hipLaunchKernelGGL(tgx::router_topk_kernel, dim3(T), dim3(64), 0, c->stream, ra);
      const int np = T * top;
      tgx::MoePlanArgs pa{};
      pa.sel = sm->sel; pa.n_pairs = np; pa.E = ld.experts; pa.top = top; pa.tile_m = grouped_tile_rows(c, np, W, ld.ff);
      pa.off = sm->moe_off; pa.perm = sm->perm; pa.tok = sm->ptok; pa.tile_e = sm->tile_e; pa.tile_m0 = sm->tile_m0; pa.n_tiles = sm->n_tiles;
      hipLaunchKernelGGL(tgx::moe_plan_kernel, dim3(1), dim3(1024), 0, c->stream, pa);
      // yh[n] = act(gate_e . a[tok(n)], up_e . a[tok(n)]) over the pairs grouped by expert
      g = tgx::StackGemmArgs{};
      g.A = sm->a; g.lda = W; g.a_rows = sm->ptok; g.B = w.w_gate; g.B2 = w.w_up; g.ldb = W; g.b_zstride = (long long)ld.ff * W; g.C = sm->yh; g.ldc = ld.ff;
      g.z_off = sm->moe_off; g.tile_z = sm->tile_e; g.tile_m0 = sm->tile_m0; g.n_tiles = sm->n_tiles; g.M = np; g.N = ld.ff; g.K = W; g.limit = ld.limit;
      launch_gemm(c, g, tgx::SG_EXPERT_ACT, 1, np, ld.experts, pa.tile_m);
      // yd[pair] = router weight * (down_e . yh[n])
      g = tgx::StackGemmArgs{};
      g.A = sm->yh; g.lda = ld.ff; g.B = w.w_down; g.ldb = ld.ff; g.b_zstride = (long long)W * ld.ff; g.C = sm->yd; g.ldc = W; g.c_rows = sm->perm;
      g.z_off = sm->moe_off; g.tile_z = sm->tile_e; g.tile_m0 = sm->tile_m0; g.n_tiles = sm->n_tiles; g.M = np; g.N = W; g.K = ld.ff; g.rw = sm->selw;
      launch_gemm(c, g, tgx::SG_ROWSCALE, 1, np, ld.experts, pa.tile_m);
    }
    tgx::CombineDepthArgs cd{};
    cd.x = sm->x; cd.y = sm->yd; cd.xs = sm->xs; cd.slot_stride = slot_stride; cd.dw = w.dwa; cd.W = W; cd.top = top; cd.n_res = li + 2;
    hipLaunchKernelGGL(tgx::combine_depth_kernel, dim3(T), dim3(256), 0, c->stream, cd);
  }
  return TGX_OK;
}

// ---- sandwich-norm designs (Modepel): per layer  norm -> mixer -> norm, add  and  norm -> feed-forward -> norm, add.  The seam kernel between two sublayers
// applies the norm behind one, the residual add and the norm in front of the next, so the stream is read and written once per sublayer.
template <int DT, bool SPLIT>
void launch_gqa_t(tgx_ctx* c, const tgx::StepMeta& m, const tgx::GqaAttnArgs& a, dim3 grid) {
  const size_t lds = (size_t)4 * a.vdim * 4;
  const int rpl = (std::max(a.dim, a.vdim) + 63) / 64;
  if (rpl <= 1) hipLaunchKernelGGL((tgx::gqa_attn_kernel<DT, 1, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
  else if (rpl <= 2) hipLaunchKernelGGL((tgx::gqa_attn_kernel<DT, 2, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
  else hipLaunchKernelGGL((tgx::gqa_attn_kernel<DT, 4, SPLIT>), grid, dim3(256), lds, c->stream, m, a);
}

// One attention layer's work between its input and output products, for every design with grouped-query attention over a paged key / value pool: rotation /
// query temperature / pool append, then the attention itself (matrix cores where the layer keeps a transposed value pool, lanes otherwise; a sequence's keys
// divided between workgroups when the step is small and the span of visible keys long).  The projections' row is [q | k | v | ..] at `proj`.
struct GqaSpec {
  float* proj; long long ldp;
  int heads, kv_heads, dim, vdim;
  int rot_dims, rot_pairs; const float* cs;
  ebyte *poolK, *poolV, *poolVT; bool append;      // append false: the pools belong to another layer, which has filled them for this step's tokens already
  int vmode; const float* lam;
  const float* gate; long long ldg;
  float scale, sink; int has_sink;
  int mask_kind, mask_size; float softcap; int dist_bias;
  float q_temp_coef; int q_temp_every;
  float* out; long long ldo;
};
int run_gqa_core(tgx_ctx* c, const tgx::StepMeta& m, const GqaSpec& sp, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const int H = sp.heads, G = sp.kv_heads;
  tgx::GqaAppendArgs ap{};
  ap.proj = sp.proj; ap.ldp = sp.ldp; ap.heads = H; ap.kv_heads = G; ap.dim = sp.dim; ap.vdim = sp.vdim; ap.rot_dims = sp.cs ? sp.rot_dims : 0; ap.rot_pairs = sp.rot_pairs;
  ap.cs = sp.cs; ap.poolK = sp.append ? sp.poolK : nullptr; ap.poolV = sp.poolV; ap.poolVT = sp.poolVT; ap.vfirst = sm->vfirst; ap.vmode = sp.vmode; ap.lam = sp.lam;
  ap.q_temp_coef = sp.q_temp_every > 0 ? sp.q_temp_coef : 0.f; ap.q_temp_every = sp.q_temp_every;
  if (sp.append || ap.rot_dims > 0 || ap.q_temp_coef != 0.f) TGX_DT_SWITCH(c->dt, hipLaunchKernelGGL(tgx::gqa_append_kernel<DT>, dim3(T), dim3(256), 0, c->stream, m, ap))
  // the longest run of keys any workgroup walks: everything before the token, or the mask's span (plus the matrix-core kernel's tile alignment)
  const int span = sp.mask_kind == tgx::MASK_CAUSAL ? max_keys : std::min(max_keys, sp.mask_size + 96);
  if (sp.poolVT && sm->attn_mfma) {
    // rows = (token, query head of the group) pairs of an entry and a key / value head in tiles of 32; few tiles and a long context: the keys are divided
    tgx::GqaMfmaArgs ma{};
    ma.q = sp.proj; ma.ldq = sp.ldp; ma.poolK = sp.poolK; ma.poolVT = sp.poolVT; ma.gate = sp.gate; ma.ldg = sp.ldg; ma.out = sp.out; ma.ldo = sp.ldo;
    ma.heads = H; ma.kv_heads = G; ma.dim = sp.dim; ma.vdim = sp.vdim; ma.terms = c->act16 ? 1 : 2; ma.scale = sp.scale; ma.sink = sp.sink; ma.has_sink = sp.has_sink;
    ma.mask_kind = sp.mask_kind; ma.mask_size = sp.mask_size; ma.softcap = sp.softcap; ma.dist_bias = sp.dist_bias;
    const int tiles = (max_count * (H / G) + 31) / 32;
    const long long wgs = (long long)tiles * S * G;
    int nsplit = 1;
    if (span >= sm->gqa_split_min_keys && wgs < c->num_cus) {
      nsplit = (int)std::min<long long>(64, (2LL * c->num_cus) / wgs);
      const int per = std::max(64, ((span + nsplit - 1) / nsplit + 63) / 64 * 64);      // whole key tiles
      nsplit = (span + per - 1) / per;
      ma.keys_per = per;
    }
    if (nsplit > 1) {
      int rc = ensure_part(c, (size_t)T * H * nsplit * (size_t)(sp.vdim + 2));
      if (rc) return rc;
      ma.part = sm->part; ma.nsplit = nsplit;
      launch_gqa_mfma(c, m, ma, dim3(tiles, S * G, nsplit), true);
      tgx::GqaAttnArgs mg{};
      mg.part = sm->part; mg.nsplit = nsplit; mg.heads = H; mg.vdim = sp.vdim; mg.gate = sp.gate; mg.ldg = sp.ldg; mg.out = sp.out; mg.ldo = sp.ldo;
      hipLaunchKernelGGL(tgx::gqa_attn_merge_kernel, dim3(T, H), dim3(256), 0, c->stream, mg);
    } else {
      launch_gqa_mfma(c, m, ma, dim3(tiles, S * G), false);
    }
    return TGX_OK;
  }
  tgx::GqaAttnArgs aa{};
  aa.q = sp.proj; aa.ldq = sp.ldp; aa.poolK = sp.poolK; aa.poolV = sp.poolV; aa.gate = sp.gate; aa.ldg = sp.ldg; aa.out = sp.out; aa.ldo = sp.ldo;
  aa.heads = H; aa.kv_heads = G; aa.dim = sp.dim; aa.vdim = sp.vdim; aa.scale = sp.scale; aa.sink = sp.sink; aa.has_sink = sp.has_sink;
  aa.mask_kind = sp.mask_kind; aa.mask_size = sp.mask_size; aa.softcap = sp.softcap; aa.dist_bias = sp.dist_bias;
  int nsplit = 1;
  if (span >= sm->gqa_split_min_keys && (long long)T * H < 2LL * c->num_cus) {      // few (token, head) pairs and a long context: the keys are divided between workgroups
    nsplit = (int)std::min<long long>(64, (4LL * c->num_cus) / ((long long)T * H));
    const int per = std::max(256, ((span + nsplit - 1) / nsplit + 63) / 64 * 64);
    nsplit = (span + per - 1) / per;
    aa.keys_per = per;
  }
  if (nsplit > 1) {
    int rc = ensure_part(c, (size_t)T * H * nsplit * (size_t)(sp.vdim + 2));
    if (rc) return rc;
    aa.part = sm->part; aa.nsplit = nsplit;
    TGX_DT_SWITCH(c->dt, (launch_gqa_t<DT, true>(c, m, aa, dim3(T, H, nsplit))))
    hipLaunchKernelGGL(tgx::gqa_attn_merge_kernel, dim3(T, H), dim3(256), 0, c->stream, aa);
  } else {
    TGX_DT_SWITCH(c->dt, (launch_gqa_t<DT, false>(c, m, aa, dim3(T, H))))
  }
  return TGX_OK;
}

int run_attention(tgx_ctx* c, const tgx::StepMeta& m, StackLayerW& w, const float* hin, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const int W = sm->d.width, H = ld.heads, G = ld.kv_heads, qd = H * ld.dim, kd = G * ld.dim, kvv = G * ld.vdim, vd = H * ld.vdim, nin = qd + kd + kvv + vd;
  // [q | k | v | gate] = h . w_in^T + b
  tgx::StackGemmArgs g{};
  g.A = hin; g.lda = W; g.B = w.w_in; g.ldb = W; g.C = sm->proj; g.ldc = nin; g.M = T; g.N = nin; g.K = W; g.scale = 1.f; g.bias = w.b_in;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  GqaSpec sp{};
  sp.proj = sm->proj; sp.ldp = nin; sp.heads = H; sp.kv_heads = G; sp.dim = ld.dim; sp.vdim = ld.vdim; sp.rot_dims = ld.rot_dims;
  sp.cs = w.rot >= 0 ? sm->rot[(size_t)w.rot].cs : nullptr; sp.poolK = w.pool; sp.poolV = w.poolV; sp.poolVT = w.poolVT; sp.append = true; sp.vmode = w.vmode; sp.lam = w.vmix;
  sp.gate = sm->proj + qd + kd + kvv; sp.ldg = nin; sp.scale = ld.scale; sp.sink = 0.f; sp.has_sink = 1; sp.out = sm->o; sp.ldo = vd;
  int rc = run_gqa_core(c, m, sp, T, S, max_keys, max_count);
  if (rc) return rc;
  // y = o . w_o^T
  g = tgx::StackGemmArgs{};
  g.A = sm->o; g.lda = vd; g.B = w.w_o; g.ldb = vd; g.C = sm->yd; g.ldc = W; g.M = T; g.N = W; g.K = vd; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  return TGX_OK;
}

int run_mlstm(tgx_ctx* c, const tgx::StepMeta& m, StackLayerW& w, const float* hin, int T, int S) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const int W = sm->d.width, H = ld.heads, qd = H * ld.dim, vd = H * ld.vdim, nin = 2 * qd + 2 * vd + 2 * H;
  // [q | k | v | gate | i | f] = h . w_in^T (+ the gate biases); i and f through the soft cap (and the log sigmoid) in the product's epilogue
  tgx::StackGemmArgs g{};
  g.A = hin; g.lda = W; g.B = w.w_in; g.ldb = W; g.C = sm->proj; g.ldc = nin; g.M = T; g.N = nin; g.K = W; g.scale = 1.f; g.bias = w.b_in;
  g.gate_col0 = 2 * qd + 2 * vd; g.gate_heads = H; g.gate_cap = ld.gate_cap;      // the two gate rows leave the product as log gates
  launch_gemm(c, g, tgx::SG_STORE, 1);
  tgx::MlstmArgs ma{};
  ma.proj = sm->proj; ma.ldp = nin; ma.heads = H; ma.dim = ld.dim; ma.vdim = ld.vdim; ma.qscale = 1.0f / sqrtf((float)ld.dim);
  ma.S = w.mS; ma.n = w.mn; ma.mx = w.mm; ma.n_buf = (size_t)sm->d.max_seqs * H * ld.dim; ma.mx_buf = (size_t)sm->d.max_seqs * H;
  ma.hs = sm->hs; ma.ldh = vd;
  // columns per wave: 16, or 8 (twice the workgroups, half the rows per lane) while the step's entries and heads leave most of the chip idle
  const bool narrow = ld.dim <= 256 && (sm->mlstm_narrow >= 0 ? sm->mlstm_narrow != 0 : (long long)S * H * ((ld.vdim + 63) / 64) * 2 <= c->num_cus);
  if (narrow) {
    const dim3 grid(S, H, (ld.vdim + 31) / 32);
    const int dper = (ld.dim + 7) / 8;
    if (dper <= 8) hipLaunchKernelGGL((tgx::mlstm_scan_kernel<8, 8>), grid, dim3(256), 0, c->stream, m, ma);
    else if (dper <= 16) hipLaunchKernelGGL((tgx::mlstm_scan_kernel<16, 8>), grid, dim3(256), 0, c->stream, m, ma);
    else hipLaunchKernelGGL((tgx::mlstm_scan_kernel<32, 8>), grid, dim3(256), 0, c->stream, m, ma);
  } else {
    const dim3 grid(S, H, (ld.vdim + 63) / 64);
    const int dper = (ld.dim + 3) / 4;      // rows per lane: four row groups share a column
    if (dper <= 8) hipLaunchKernelGGL((tgx::mlstm_scan_kernel<8, 16>), grid, dim3(256), 0, c->stream, m, ma);
    else if (dper <= 16) hipLaunchKernelGGL((tgx::mlstm_scan_kernel<16, 16>), grid, dim3(256), 0, c->stream, m, ma);
    else if (dper <= 32) hipLaunchKernelGGL((tgx::mlstm_scan_kernel<32, 16>), grid, dim3(256), 0, c->stream, m, ma);
    else if (dper <= 64) hipLaunchKernelGGL((tgx::mlstm_scan_kernel<64, 16>), grid, dim3(256), 0, c->stream, m, ma);
    else hipLaunchKernelGGL((tgx::mlstm_scan_kernel<128, 16>), grid, dim3(256), 0, c->stream, m, ma);
  }
  tgx::HeadNormGateArgs oa{};
  oa.hs = sm->hs; oa.ldh = vd; oa.w = w.head_w; oa.w_hstride = ld.vdim; oa.gate = sm->proj + 2 * qd + vd; oa.ldg = nin; oa.out = sm->o; oa.ldo = vd; oa.vdim = ld.vdim; oa.eps = sm->d.norm_eps;
  hipLaunchKernelGGL(tgx::head_norm_gate_kernel, dim3(T, H), dim3(64), 0, c->stream, oa);
  g = tgx::StackGemmArgs{};
  g.A = sm->o; g.lda = vd; g.B = w.w_o; g.ldb = vd; g.C = sm->yd; g.ldc = W; g.M = T; g.N = W; g.K = vd; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  return TGX_OK;
}

void run_dense_ff(tgx_ctx* c, StackLayerW& w, const float* hin, int T) {
  StackModel* sm = c->stack;
  const int W = sm->d.width, F = w.d.ff;
  tgx::StackGemmArgs g{};
  g.A = hin; g.lda = W; g.B = w.w_up; g.ldb = W; g.C = sm->yh; g.ldc = F; g.M = T; g.N = F; g.K = W; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  hipLaunchKernelGGL(tgx::poly_norm_kernel, dim3(T), dim3(256), 0, c->stream, sm->yh, w.act, F, sm->d.norm_eps);
  g = tgx::StackGemmArgs{};
  g.A = sm->yh; g.lda = F; g.B = w.w_down; g.ldb = F; g.C = sm->yd; g.ldc = W; g.M = T; g.N = W; g.K = F; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
}

// grouped-choice experts: the chosen pairs' rows land in yd (none for identity outputs), the shared expert's in ysh; the seam kernel sums them
void run_choice_experts(tgx_ctx* c, StackLayerW& w, const float* hin, int T) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const int W = sm->d.width, E = ld.experts + ld.identity, top = ld.top, nz = E + (ld.shared_ff > 0 ? 1 : 0);
  tgx::StackGemmArgs g{};
  g.A = hin; g.lda = W; g.B = w.w_router; g.ldb = W; g.C = sm->zr; g.ldc = nz; g.M = T; g.N = nz; g.K = W; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1, 0, 0, 64, tgx::DT_F32);
  tgx::RouterGroupArgs ra{};
  ra.z = sm->zr; ra.ldz = nz; ra.corr = w.b_router; ra.sel = sm->sel; ra.selw = sm->selw; ra.sgw = ld.shared_ff > 0 ? sm->sgw : nullptr;
  ra.E = E; ra.top = top; ra.groups = ld.groups; ra.keep = ld.groups_keep; ra.scale = ld.router_scale;
  hipLaunchKernelGGL(tgx::router_group_kernel, dim3(T), dim3(64), 0, c->stream, ra);
  const int np = T * top;
  if (ld.experts > 0) {
    tgx::MoePlanArgs pa{};
    pa.sel = sm->sel; pa.n_pairs = np; pa.E = E; pa.top = top; pa.tile_m = grouped_tile_rows(c, np, W, ld.ff); pa.E_tiles = ld.experts;
    pa.off = sm->moe_off; pa.perm = sm->perm; pa.tok = sm->ptok; pa.tile_e = sm->tile_e; pa.tile_m0 = sm->tile_m0; pa.n_tiles = sm->n_tiles;
    hipLaunchKernelGGL(tgx::moe_plan_kernel, dim3(1), dim3(1024), 0, c->stream, pa);
    g = tgx::StackGemmArgs{};
    g.A = hin; g.lda = W; g.a_rows = sm->ptok; g.B = w.w_gate; g.B2 = w.w_up; g.ldb = W; g.b_zstride = (long long)ld.ff * W; g.C = sm->yh; g.ldc = ld.ff;
    g.z_off = sm->moe_off; g.tile_z = sm->tile_e; g.tile_m0 = sm->tile_m0; g.n_tiles = sm->n_tiles; g.M = np; g.N = ld.ff; g.K = W;
    launch_gemm(c, g, tgx::SG_SILU_MUL, 1, np, E, pa.tile_m);
    g = tgx::StackGemmArgs{};
    g.A = sm->yh; g.lda = ld.ff; g.B = w.w_down; g.ldb = ld.ff; g.b_zstride = (long long)W * ld.ff; g.C = sm->yd; g.ldc = W; g.c_rows = sm->perm;
    g.z_off = sm->moe_off; g.tile_z = sm->tile_e; g.tile_m0 = sm->tile_m0; g.n_tiles = sm->n_tiles; g.M = np; g.N = W; g.K = ld.ff; g.rw = sm->selw;
    launch_gemm(c, g, tgx::SG_ROWSCALE, 1, np, E, pa.tile_m);
  }
  if (ld.shared_ff > 0) {
    float* hsh = sm->yh + (size_t)np * std::max(1, ld.ff);
    g = tgx::StackGemmArgs{};
    g.A = hin; g.lda = W; g.B = w.ws_gate; g.B2 = w.ws_up; g.ldb = W; g.C = hsh; g.ldc = ld.shared_ff; g.M = T; g.N = ld.shared_ff; g.K = W;
    launch_gemm(c, g, tgx::SG_SILU_MUL, 1);
    g = tgx::StackGemmArgs{};
    g.A = hsh; g.lda = ld.shared_ff; g.B = w.ws_down; g.ldb = ld.shared_ff; g.C = sm->ysh; g.ldc = W; g.M = T; g.N = W; g.K = ld.shared_ff; g.rw = sm->sgw;
    launch_gemm(c, g, tgx::SG_ROWSCALE, 1);
  }
}

int run_layers_sandwich(tgx_ctx* c, const MetaPtrs& mp, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx::StepMeta m = step_meta(sm, mp, T, S);
  const int W = sm->d.width, L = sm->d.layers;
  const float eps = sm->d.norm_eps;
  TGX_DT_SWITCH(c->dt, hipLaunchKernelGGL(tgx::embed_rows_kernel<DT>, dim3(T), dim3(256), 0, c->stream, m, reinterpret_cast<const tgx::elem_t<DT>*>(c->embed), sm->x, W))
  hipLaunchKernelGGL(tgx::scalar_norm_kernel, dim3(T), dim3(256), 0, c->stream, sm->x, nullptr, sm->norm_g, sm->a, W, eps);
  float *hin = sm->a, *hout = sm->a2;
  for (int li = 0; li < L; li++) {
    StackLayerW& w = sm->L[(size_t)li];
    const tgx_layer_desc& ld = w.d;
    const float* ng = sm->norm_g + 4 * (size_t)li;
    const float* next_layer = li + 1 < L ? ng + 4 : nullptr;
    int rc = ld.mixer == TGX_MIXER_ATTENTION ? run_attention(c, m, w, hin, T, S, max_keys, max_count) : run_mlstm(c, m, w, hin, T, S);
    if (rc) return rc;
    tgx::SandwichArgs sa{};
    sa.x = sm->x; sa.y = sm->yd; sa.top = 1; sa.ytmp = sm->ytmp; sa.g_post = ng + 1; sa.g_next = ld.mlp != TGX_MLP_NONE ? ng + 2 : next_layer; sa.out = hout; sa.W = W; sa.eps = eps;
    hipLaunchKernelGGL(tgx::sandwich_kernel, dim3(T), dim3(256), 0, c->stream, sa);
    std::swap(hin, hout);
    if (ld.mlp == TGX_MLP_NONE) continue;
    sa = tgx::SandwichArgs{};
    sa.x = sm->x; sa.y = sm->yd; sa.top = 1; sa.ytmp = sm->ytmp; sa.g_post = ng + 3; sa.g_next = next_layer; sa.out = hout; sa.W = W; sa.eps = eps;
    if (ld.mlp == TGX_MLP_DENSE) run_dense_ff(c, w, hin, T);
    else {
      run_choice_experts(c, w, hin, T);
      sa.top = ld.top; sa.sel = sm->sel; sa.selw = sm->selw; sa.n_real = ld.experts; sa.h = hin; sa.ysh = ld.shared_ff > 0 ? sm->ysh : nullptr;
    }
    hipLaunchKernelGGL(tgx::sandwich_kernel, dim3(T), dim3(256), 0, c->stream, sa);
    std::swap(hin, hout);
  }
  return TGX_OK;
}

// ---- parallel-sublayer designs (Vitudra): per layer  h = norm(x);  x += mult * (mixer(h) + ff(h)).  Every sublayer's last product adds its share to the
// stream in its epilogue (mult, and the half's weight in a parallel mixer, as the product's scale), so no combine launch is needed.
void add_to_stream(tgx_ctx* c, const float* A, int K, const ebyte* Wm, int T, float scale) {
  StackModel* sm = c->stack;
  tgx::StackGemmArgs g{};
  g.A = A; g.lda = K; g.B = Wm; g.ldb = K; g.C = sm->x; g.ldc = sm->d.width; g.M = T; g.N = sm->d.width; g.K = K; g.scale = scale;
  launch_gemm(c, g, tgx::SG_ADD, 1);
}

void launch_rec_scan(tgx_ctx* c, const tgx::StepMeta& m, const tgx::RecScanArgs& a, int kind, int S) {
  const dim3 grid(S, a.heads, (a.vdim + tgx::REC_COLS - 1) / tgx::REC_COLS);
  const int dper = (a.dim + tgx::REC_RG - 1) / tgx::REC_RG;      // rows per lane
  auto go = [&](auto K) {
    constexpr int KIND = decltype(K)::value;
    if (dper <= 4) hipLaunchKernelGGL((tgx::rec_scan_kernel<4, KIND>), grid, dim3(256), 0, c->stream, m, a);
    else if (dper <= 8) hipLaunchKernelGGL((tgx::rec_scan_kernel<8, KIND>), grid, dim3(256), 0, c->stream, m, a);
    else if (dper <= 16) hipLaunchKernelGGL((tgx::rec_scan_kernel<16, KIND>), grid, dim3(256), 0, c->stream, m, a);
    else hipLaunchKernelGGL((tgx::rec_scan_kernel<32, KIND>), grid, dim3(256), 0, c->stream, m, a);
  };
  if (kind == tgx::REC_WKV) go(std::integral_constant<int, tgx::REC_WKV>{}); else go(std::integral_constant<int, tgx::REC_DELTA>{});
}

int run_joint_attention(tgx_ctx* c, const tgx::StepMeta& m, StackLayerW& w, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const bool shared = w.kv_src >= 0;
  const int W = sm->d.width, H = ld.heads, G = ld.kv_heads, qd = H * ld.dim, vd = H * ld.vdim, nin = qd + (shared ? 0 : G * (ld.dim + ld.vdim));
  tgx::StackGemmArgs g{};
  g.A = sm->a; g.lda = W; g.B = w.w_in; g.ldb = W; g.C = sm->proj; g.ldc = nin; g.M = T; g.N = nin; g.K = W; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  GqaSpec sp{};
  sp.proj = sm->proj; sp.ldp = nin; sp.heads = H; sp.kv_heads = G; sp.dim = ld.dim; sp.vdim = ld.vdim; sp.rot_dims = ld.rot_dims; sp.rot_pairs = ld.rot_pairs;
  sp.cs = w.rot >= 0 ? sm->rot[(size_t)w.rot].cs : nullptr; sp.poolK = w.pool; sp.poolV = w.poolV; sp.poolVT = w.poolVT; sp.append = !shared;
  sp.scale = ld.scale; sp.mask_kind = ld.mask_kind; sp.mask_size = ld.mask_size; sp.softcap = ld.softcap; sp.dist_bias = ld.dist_bias;
  sp.q_temp_coef = ld.q_temp_coef; sp.q_temp_every = ld.q_temp_every; sp.out = sm->o; sp.ldo = vd;
  int rc = run_gqa_core(c, m, sp, T, S, max_keys, max_count);
  if (rc) return rc;
  add_to_stream(c, sm->o, vd, w.w_o, T, sm->d.residual_mult);
  return TGX_OK;
}

void run_wkv(tgx_ctx* c, const tgx::StepMeta& m, StackLayerW& w, int T, int S) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const int W = sm->d.width, H = ld.heads, HD = H * ld.dim, R = ld.decay_rank;
  tgx::TokenShiftArgs ts{};
  ts.h = sm->a; ts.mu = w.mu; ts.out = sm->mixed; ts.state = w.shift; ts.state_buf = (size_t)sm->d.max_seqs * W; ts.W = W; ts.n = 5;
  hipLaunchKernelGGL(tgx::token_shift_kernel, dim3(T, (W + 255) / 256), dim3(256), 0, c->stream, m, ts);
  // proj row = [r | k | v | g | w]: the first four as one product batched over their mixes, the decay through its low-rank pair
  tgx::StackGemmArgs g{};
  g.A = sm->mixed; g.lda = 5LL * W; g.a_zoff = W; g.B = w.w_in; g.ldb = W; g.b_zstride = (long long)HD * W; g.C = sm->proj; g.ldc = 5LL * HD; g.c_zoff = HD;
  g.M = T; g.N = HD; g.K = W; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 4);
  g = tgx::StackGemmArgs{};
  g.A = sm->mixed + 4 * (size_t)W; g.lda = 5LL * W; g.B = w.w_w1; g.ldb = W; g.C = sm->lora; g.ldc = R; g.M = T; g.N = R; g.K = W; g.scale = 1.f; g.act = tgx::SG_ACT_TANH;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  g = tgx::StackGemmArgs{};
  g.A = sm->lora; g.lda = R; g.B = w.w_w2; g.ldb = R; g.C = sm->proj + 4 * (size_t)HD; g.ldc = 5LL * HD; g.M = T; g.N = HD; g.K = R; g.scale = 1.f; g.bias = w.w0; g.act = tgx::SG_ACT_DECAY;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  tgx::RecScanArgs ra{};
  ra.a = sm->proj; ra.lda = 5LL * HD; ra.k = sm->proj + HD; ra.ldk = 5LL * HD; ra.v = sm->proj + 2 * (size_t)HD; ra.ldv = 5LL * HD; ra.w = sm->proj + 4 * (size_t)HD; ra.ldw = 5LL * HD;
  ra.u = w.ubonus; ra.S = w.mS; ra.out = sm->hs; ra.ldo = HD; ra.heads = H; ra.kv_heads = H; ra.dim = ld.dim; ra.vdim = ld.dim;
  launch_rec_scan(c, m, ra, tgx::REC_WKV, S);
  tgx::HeadNormGateArgs oa{};
  oa.hs = sm->hs; oa.ldh = HD; oa.w = w.head_w; oa.w_hstride = ld.dim; oa.gate = sm->proj + 3 * (size_t)HD; oa.ldg = 5LL * HD; oa.silu_gate = 1; oa.out = sm->o; oa.ldo = HD; oa.vdim = ld.dim;
  oa.eps = sm->d.norm_eps;
  hipLaunchKernelGGL(tgx::head_norm_gate_kernel, dim3(T, H), dim3(64), 0, c->stream, oa);
  add_to_stream(c, sm->o, HD, w.w_o, T, sm->d.residual_mult);
}

int run_parallel(tgx_ctx* c, const tgx::StepMeta& m, StackLayerW& w, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const int W = sm->d.width, H = ld.heads, G = ld.kv_heads, lq = H * ld.dim, lkv = G * (ld.dim + ld.vdim), lvd = H * ld.vdim;
  const int rH = ld.d_heads, rG = ld.d_kv_heads, rGD = rG * ld.d_dim, rvd = rH * ld.d_vdim, rC = 2 * rGD + rvd, nin = lq + lkv + rC + 2 * rH + rvd;
  // [left q | k | v | right q | k | v | b | a | g] = h . w_in^T: both halves read the same input
  tgx::StackGemmArgs g{};
  g.A = sm->a; g.lda = W; g.B = w.w_in; g.ldb = W; g.C = sm->proj; g.ldc = nin; g.M = T; g.N = nin; g.K = W; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  GqaSpec sp{};
  sp.proj = sm->proj; sp.ldp = nin; sp.heads = H; sp.kv_heads = G; sp.dim = ld.dim; sp.vdim = ld.vdim; sp.rot_dims = ld.rot_dims; sp.rot_pairs = ld.rot_pairs;
  sp.cs = w.rot >= 0 ? sm->rot[(size_t)w.rot].cs : nullptr; sp.poolK = w.pool; sp.poolV = w.poolV; sp.poolVT = w.poolVT; sp.append = true;
  sp.scale = ld.scale; sp.mask_kind = ld.mask_kind; sp.mask_size = ld.mask_size; sp.softcap = ld.softcap; sp.dist_bias = ld.dist_bias;
  sp.q_temp_coef = ld.q_temp_coef; sp.q_temp_every = ld.q_temp_every; sp.out = sm->o; sp.ldo = lvd;
  int rc = run_gqa_core(c, m, sp, T, S, max_keys, max_count);
  if (rc) return rc;
  add_to_stream(c, sm->o, lvd, w.w_o, T, sm->d.residual_mult * ld.left_scale);
  // the right half: rec_in row = [q | k | v | beta | decay]
  const int ldr = rC + 2 * rH, nb = ld.conv_taps - 1;
  tgx::DeltaPrepArgs dp{};
  dp.proj = sm->proj; dp.ldp = nin; dp.col0 = lq + lkv; dp.cw = w.conv_w; dp.a_log = w.a_log; dp.dt_bias = w.dt_bias; dp.out = sm->rec_in; dp.ldo = ldr;
  dp.state = nb > 0 ? w.conv_state : nullptr; dp.state_buf = (size_t)sm->d.max_seqs * nb * rC; dp.heads = rH; dp.kv_heads = rG; dp.dim = ld.d_dim; dp.vdim = ld.d_vdim; dp.taps = ld.conv_taps;
  dp.q_scale = 1.0f / sqrtf((float)ld.d_dim); dp.unit_eps = 1e-6f;
  hipLaunchKernelGGL(tgx::delta_prep_kernel, dim3(T, 2 * rG + rH + 1), dim3(256), 0, c->stream, m, dp);
  tgx::RecScanArgs ra{};
  ra.a = sm->rec_in; ra.lda = ldr; ra.k = sm->rec_in + rGD; ra.ldk = ldr; ra.v = sm->rec_in + 2 * (size_t)rGD; ra.ldv = ldr;
  ra.beta = sm->rec_in + rC; ra.g = sm->rec_in + rC + rH; ra.ldg = ldr; ra.S = w.mS; ra.out = sm->hs; ra.ldo = rvd; ra.heads = rH; ra.kv_heads = rG; ra.dim = ld.d_dim; ra.vdim = ld.d_vdim;
  launch_rec_scan(c, m, ra, tgx::REC_DELTA, S);
  tgx::HeadNormGateArgs oa{};
  oa.hs = sm->hs; oa.ldh = rvd; oa.w = w.head_w; oa.w_hstride = 0; oa.gate = sm->proj + lq + lkv + rC + 2 * rH; oa.ldg = nin; oa.silu_gate = 1; oa.out = sm->o; oa.ldo = rvd; oa.vdim = ld.d_vdim;
  oa.eps = sm->d.norm_eps;
  hipLaunchKernelGGL(tgx::head_norm_gate_kernel, dim3(T, rH), dim3(64), 0, c->stream, oa);
  add_to_stream(c, sm->o, rvd, w.w_o2, T, sm->d.residual_mult * ld.right_scale);
  return TGX_OK;
}

int run_layers_joint(tgx_ctx* c, const MetaPtrs& mp, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx::StepMeta m = step_meta(sm, mp, T, S);
  const int W = sm->d.width;
  TGX_DT_SWITCH(c->dt, hipLaunchKernelGGL(tgx::embed_rows_kernel<DT>, dim3(T), dim3(256), 0, c->stream, m, reinterpret_cast<const tgx::elem_t<DT>*>(c->embed), sm->x, W))
  for (int li = 0; li < sm->d.layers; li++) {
    StackLayerW& w = sm->L[(size_t)li];
    const tgx_layer_desc& ld = w.d;
    hipLaunchKernelGGL(tgx::offset_norm_kernel, dim3(T), dim3(256), 0, c->stream, sm->x, nullptr, w.norm1, 1.0f, sm->a, W, sm->d.norm_eps);
    int rc = TGX_OK;
    if (ld.mixer == TGX_MIXER_ATTENTION) rc = run_joint_attention(c, m, w, T, S, max_keys, max_count);
    else if (ld.mixer == TGX_MIXER_WKV) run_wkv(c, m, w, T, S);
    else rc = run_parallel(c, m, w, T, S, max_keys, max_count);
    if (rc) return rc;
    if (ld.mlp == TGX_MLP_DENSE) {      // x += mult * down(silu(gate h) * (up h))
      tgx::StackGemmArgs g{};
      g.A = sm->a; g.lda = W; g.B = w.w_gate; g.B2 = w.w_up; g.ldb = W; g.C = sm->yh; g.ldc = ld.ff; g.M = T; g.N = ld.ff; g.K = W;
      launch_gemm(c, g, tgx::SG_SILU_MUL, 1);
      add_to_stream(c, sm->yh, ld.ff, w.w_down, T, sm->d.residual_mult);
    }
  }
  return TGX_OK;
}

// ---- layer-norm designs (Zaluvik): per run of a layer  x += mult * LN_b(mixer(LN_a(x)))  and  x += mult * LN_d(ff(LN_c(x))).  A run has its own cache (a layer
// inside the loop runs once per pass); in front of the first layer of every pass the stream is replaced by the loop's input product on [x; x0].  The seam
// kernel applies the norm behind a sublayer, the residual add and the norm in front of the next one.
template <int DT, bool SPLIT>
void launch_mix_attn_t(tgx_ctx* c, const tgx::StepMeta& m, const tgx::MixAttnArgs& a, dim3 grid, size_t lds, bool vec) {
  const int npt = (a.heads * a.vdim / (vec ? 8 : 1) + 255) / 256;      // outputs per thread: channels, or slices of eight
  auto go = [&](auto N, auto V) {
    constexpr int NPT = decltype(N)::value; constexpr bool VEC = decltype(V)::value;
    auto* fn = &tgx::sigmoid_mix_attn_kernel<DT, NPT, VEC, SPLIT>;
    if (lds > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(fn, grid, dim3(256), lds, c->stream, m, a);
  };
  if (vec) {      // slices of eight channels: at most MIX_ATTN_MAX_OUT / 8 / 256 = 4 per thread
    if (npt <= 1) go(std::integral_constant<int, 1>{}, std::true_type{});
    else if (npt <= 2) go(std::integral_constant<int, 2>{}, std::true_type{});
    else go(std::integral_constant<int, 4>{}, std::true_type{});
    return;
  }
  if (npt <= 1) go(std::integral_constant<int, 1>{}, std::false_type{});
  else if (npt <= 2) go(std::integral_constant<int, 2>{}, std::false_type{});
  else if (npt <= 4) go(std::integral_constant<int, 4>{}, std::false_type{});
  else if (npt <= 8) go(std::integral_constant<int, 8>{}, std::false_type{});
  else if (npt <= 16) go(std::integral_constant<int, 16>{}, std::false_type{});
  else go(std::integral_constant<int, 32>{}, std::false_type{});
}
constexpr int MIX_ATTN_MAX_OUT = 32 * 256;            // heads * vdim of the sigmoid attention (output channels per thread <= 32)
constexpr size_t MIX_ATTN_MAX_LDS = 144 * 1024;
int mix_attn_tile_keys(int heads, int dim) {          // keys per tile: 64, or 32 where that keeps the workgroup's LDS within 64 KB
  return tgx::mix_attn_lds_bytes(heads, dim, 64) <= 64 * 1024 ? 64 : 32;
}

// the matrix-core form of the sigmoid attention serves 16-bit storage, key sizes in steps of 16, value sizes in steps of 32 up to 128, 1 / 2 / 4 / 8 query
// heads per key / value head and pages of a multiple of 32 tokens
constexpr int MIX_MFMA_MIN_COUNT = 16;      // portions from this many tokens on take it; shorter ones (and decoded tokens) the lane kernel
bool layer_mix_mfma(const tgx_ctx* c, const tgx_layer_desc& l) {
  const int qpg = l.kv_heads > 0 ? l.heads / l.kv_heads : 0;
  return c->dt != tgx::DT_F32 && l.dim % 16 == 0 && l.vdim % 32 == 0 && l.vdim <= 128 && (qpg == 1 || qpg == 2 || qpg == 4 || qpg == 8) && c->stack->page_shift >= 5 &&
         mix_mfma_wg_lds(l.heads, l.kv_heads) <= MIX_ATTN_MAX_LDS;
}
int run_affine_attention(tgx_ctx* c, const tgx::StepMeta& m, StackLayerW& w, const StackRun& run, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const int W = sm->d.width, H = ld.heads, G = ld.kv_heads, qd = H * ld.dim, kd = G * ld.dim, kvv = G * ld.vdim, vd = H * ld.vdim, nin = qd + kd + kvv + vd;
  // [q | k | v | gate] = h . w_in^T
  tgx::StackGemmArgs g{};
  g.A = sm->a; g.lda = W; g.B = w.w_in; g.ldb = W; g.C = sm->proj; g.ldc = nin; g.M = T; g.N = nin; g.K = W; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  tgx::GqaAppendArgs ap{};
  ap.proj = sm->proj; ap.ldp = nin; ap.heads = H; ap.kv_heads = G; ap.dim = ld.dim; ap.vdim = ld.vdim; ap.poolK = run.pool; ap.poolV = run.poolV;
  ap.qk_unit_eps = ld.qk_norm ? sm->d.norm_eps : 0.f;
  const bool mfma = run.poolT && sm->attn_mfma && max_count >= MIX_MFMA_MIN_COUNT;
  ap.poolVT = run.poolT;
  if (mfma) { ap.q_hi = sm->qplanes; ap.q_lo = sm->qplanes + (((size_t)sm->cap_tokens * sm->max_qd + 7) & ~(size_t)7); }      // (both planes 16-byte aligned)
  TGX_DT_SWITCH(c->dt, hipLaunchKernelGGL(tgx::gqa_append_kernel<DT>, dim3(T), dim3(256), 0, c->stream, m, ap))
  if (mfma) {
    tgx::MixMfmaArgs ma{};
    ma.qh = ap.q_hi; ma.ql = ap.q_lo; ma.poolK = run.pool; ma.poolVT = run.poolT; ma.pb = w.pb; ma.talk = ld.head_mix ? w.talk : nullptr;
    ma.gate = ld.gate_kind == 1 ? sm->proj + qd + kd + kvv : nullptr; ma.ldg = nin; ma.out = sm->o; ma.ldo = vd;
    ma.heads = H; ma.kv_heads = G; ma.dim = ld.dim; ma.vdim = ld.vdim; ma.terms = c->act16 ? 1 : 2; ma.scale = ld.scale; ma.mask_kind = ld.mask_kind; ma.mask_size = ld.mask_size;
    const dim3 grid((max_count + 31) / 32, S, G);
    launch_mix_mfma(c, m, ma, grid);
    tgx::StackGemmArgs go{};
    go.A = sm->o; go.lda = vd; go.B = w.w_o; go.ldb = vd; go.C = sm->yd; go.ldc = W; go.M = T; go.N = W; go.K = vd; go.scale = 1.f;
    launch_gemm(c, go, tgx::SG_STORE, 1);
    return TGX_OK;
  }
  tgx::MixAttnArgs aa{};
  aa.q = sm->proj; aa.ldq = nin; aa.poolK = run.pool; aa.poolV = run.poolV; aa.pb = w.pb; aa.talk = ld.head_mix ? w.talk : nullptr;
  aa.gate = ld.gate_kind == 1 ? sm->proj + qd + kd + kvv : nullptr; aa.ldg = nin; aa.out = sm->o; aa.ldo = vd;
  aa.heads = H; aa.kv_heads = G; aa.dim = ld.dim; aa.vdim = ld.vdim; aa.scale = ld.scale; aa.mask_kind = ld.mask_kind; aa.mask_size = ld.mask_size;
  aa.kt = mix_attn_tile_keys(H, ld.dim);
  const size_t lds = tgx::mix_attn_lds_bytes(H, ld.dim, aa.kt);
  const bool vec = ld.dim % 8 == 0 && ld.vdim % 8 == 0;
  const int span = ld.mask_kind == tgx::MASK_CAUSAL ? max_keys : std::min(max_keys, ld.mask_size);
  int nsplit = 1;
  if (span >= std::min(sm->gqa_split_min_keys, 128) && (long long)T < c->num_cus) {      // few tokens and a long span: the keys are divided between workgroups
    nsplit = (int)std::min<long long>(64, (2LL * c->num_cus) / T);
    const int per = std::max(32, ((span + nsplit - 1) / nsplit + 31) / 32 * 32);
    nsplit = (span + per - 1) / per;
    aa.keys_per = per;
    aa.kt = std::min(aa.kt, per);
  }
  if (nsplit > 1) {
    int rc = ensure_part(c, (size_t)T * nsplit * (size_t)vd);
    if (rc) return rc;
    aa.part = sm->part; aa.nsplit = nsplit;
    TGX_DT_SWITCH(c->dt, (launch_mix_attn_t<DT, true>(c, m, aa, dim3(T, nsplit), lds, vec)))
    hipLaunchKernelGGL(tgx::sigmoid_mix_merge_kernel, dim3(T, std::min(8, (vd + 255) / 256)), dim3(256), 0, c->stream, aa);
  } else {
    TGX_DT_SWITCH(c->dt, (launch_mix_attn_t<DT, false>(c, m, aa, dim3(T), lds, vec)))
  }
  // y = o . w_o^T
  g = tgx::StackGemmArgs{};
  g.A = sm->o; g.lda = vd; g.B = w.w_o; g.ldb = vd; g.C = sm->yd; g.ldc = W; g.M = T; g.N = W; g.K = vd; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  return TGX_OK;
}

// latent attention with a rotated key part that all heads share and a window: the pool row is [normed latent | rotated key part]; every head's query is
// taken into that space ([scale W_uk^T q_plain | scale rot(q_rot)]), so a score is one dot product with the cached row and nothing else is cached
int run_affine_latent(tgx_ctx* c, const tgx::StepMeta& m, StackLayerW& w, const StackRun& run, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const int W = sm->d.width, H = ld.heads, qs = ld.dim + ld.rot_dim, qd = H * qs, R = ld.kv_rank, RR = R + ld.rot_dim, vd = H * ld.vdim, ng = ld.gate_kind == 2 ? H : vd, nin = qd + RR + ng;
  tgx::StackGemmArgs g{};
  g.A = sm->a; g.lda = W; g.B = w.w_in; g.ldb = W; g.C = sm->proj; g.ldc = nin; g.M = T; g.N = nin; g.K = W; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  tgx::LatentAppendArgs la{};
  la.src = sm->proj; la.lds = nin; la.col0 = qd; la.nw = w.lat_norm; la.pool = run.pool; la.poolT = run.poolT; la.rank = R; la.eps = sm->d.norm_eps;
  la.rot_dim = ld.rot_dim; la.rot_dims = ld.rot_dims; la.cs = w.rot >= 0 ? sm->rot[(size_t)w.rot].cs : nullptr;
  la.q = sm->proj; la.heads = H; la.qstride = qs; la.qoff = ld.dim; la.qscale = ld.scale; la.ql = sm->ql;
  TGX_DT_SWITCH(c->dt, hipLaunchKernelGGL(tgx::latent_append_kernel<DT>, dim3(T), dim3(256), 0, c->stream, m, la))
  // the plain part of every head's query into latent space: ql[t][h][0 .. R) = scale * q_plain[t][h] . ukT[h]^T
  g = tgx::StackGemmArgs{};
  g.A = sm->proj; g.lda = nin; g.a_zoff = qs; g.B = w.w_ukT; g.ldb = ld.dim; g.b_zstride = (long long)R * ld.dim; g.C = sm->ql; g.ldc = (long long)H * RR; g.c_zoff = RR;
  g.M = T; g.N = R; g.K = ld.dim; g.scale = ld.scale;
  launch_gemm(c, g, tgx::SG_STORE, H);
  tgx::LatentAttnArgs aa{};
  aa.q = sm->ql; aa.ldq = (long long)H * RR; aa.pool = run.pool; aa.sink = nullptr; aa.out = sm->lat; aa.ldo = (long long)H * RR; aa.rank = RR; aa.heads = H;
  aa.mask_kind = ld.mask_kind; aa.mask_size = ld.mask_size;
  const int span = ld.mask_kind == tgx::MASK_CAUSAL ? max_keys : std::min(max_keys, ld.mask_size + 64);      // (the matrix-core kernel starts at a key tile's edge and a row tile spans up to 32 tokens)
  int nsplit = 1;
  if (run.poolT && sm->attn_mfma) {
    // rows = (token, head) pairs of an entry in tiles of 32; few tiles and a long span: the keys are divided between workgroups
    tgx::LatentMfmaArgs ma{};
    ma.q = sm->ql; ma.pool = run.pool; ma.poolT = run.poolT; ma.sink = nullptr; ma.out = sm->lat; ma.rank = RR; ma.heads = H; ma.terms = c->act16 ? 1 : 2;
    ma.mask_kind = ld.mask_kind; ma.mask_size = ld.mask_size;
    const int tiles = (max_count * H + 31) / 32;
    if (span >= std::min(sm->attn_split_min_keys, 256) && (long long)tiles * S < c->num_cus) {
      nsplit = (int)std::min<long long>(64, (2LL * c->num_cus) / ((long long)tiles * S));
      const int per = std::max(64, ((span + nsplit - 1) / nsplit + 31) / 32 * 32);      // two key tiles per workgroup at least
      nsplit = (span + per - 1) / per;
      ma.keys_per = per;
    }
    if (nsplit > 1) {
      int rc = ensure_part(c, (size_t)T * H * nsplit * (size_t)(RR + 2));
      if (rc) return rc;
      ma.part = sm->part; ma.nsplit = nsplit;
      aa.part = sm->part; aa.nsplit = nsplit;
      if (c->dt == tgx::DT_F16) launch_attn_mfma_t<tgx::DT_F16, true>(c, m, ma, dim3(tiles, S, nsplit)); else launch_attn_mfma_t<tgx::DT_BF16, true>(c, m, ma, dim3(tiles, S, nsplit));
      hipLaunchKernelGGL(tgx::latent_attn_merge_kernel, dim3(T, H), dim3(256), 0, c->stream, aa);
    } else {
      if (c->dt == tgx::DT_F16) launch_attn_mfma_t<tgx::DT_F16, false>(c, m, ma, dim3(tiles, S)); else launch_attn_mfma_t<tgx::DT_BF16, false>(c, m, ma, dim3(tiles, S));
    }
  } else {
  if (span >= std::min(sm->attn_split_min_keys, 512) && (long long)T * H < 2LL * c->num_cus) {
    nsplit = (int)std::min<long long>(64, (4LL * c->num_cus) / ((long long)T * H));
    const int per = std::max(256, ((span + nsplit - 1) / nsplit + 63) / 64 * 64);
    nsplit = (span + per - 1) / per;
    aa.keys_per = per;
  }
  if (nsplit > 1) {
    int rc = ensure_part(c, (size_t)T * H * nsplit * (size_t)(RR + 2));
    if (rc) return rc;
    aa.part = sm->part; aa.nsplit = nsplit;
    TGX_DT_SWITCH(c->dt, (launch_attn_t<DT, true>(c, m, aa, dim3(T, H, nsplit))))
    hipLaunchKernelGGL(tgx::latent_attn_merge_kernel, dim3(T, H), dim3(256), 0, c->stream, aa);
  } else {
    TGX_DT_SWITCH(c->dt, (launch_attn_t<DT, false>(c, m, aa, dim3(T, H))))
  }
  }
  // o[t][h] = (lat[t][h][0 .. R) . uv[h]^T) * sigmoid(gate of the head, or of the channel)
  g = tgx::StackGemmArgs{};
  g.A = sm->lat; g.lda = (long long)H * RR; g.a_zoff = RR; g.B = w.w_uv; g.ldb = R; g.b_zstride = (long long)ld.vdim * R; g.C = sm->o; g.ldc = vd; g.c_zoff = ld.vdim;
  g.M = T; g.N = ld.vdim; g.K = R; g.G = sm->proj; g.ldg = nin; g.g_col0 = qd + RR; g.g_per_z = ld.gate_kind == 2;
  launch_gemm(c, g, tgx::SG_GATE, H);
  g = tgx::StackGemmArgs{};
  g.A = sm->o; g.lda = vd; g.B = w.w_o; g.ldb = vd; g.C = sm->yd; g.ldc = W; g.M = T; g.N = W; g.K = vd; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1);
  return TGX_OK;
}

// the feed-forward of a layer-norm design into yd (one row per token, or `top` rows per token for experts) and ysh (the shared expert's row)
void run_affine_ff(tgx_ctx* c, StackLayerW& w, int T) {
  StackModel* sm = c->stack;
  const tgx_layer_desc& ld = w.d;
  const int W = sm->d.width;
  tgx::StackGemmArgs g{};
  if (ld.mlp == TGX_MLP_DENSE) {      // down(act(up h))
    g.A = sm->a; g.lda = W; g.B = w.w_up; g.ldb = W; g.C = sm->yh; g.ldc = ld.ff; g.M = T; g.N = ld.ff; g.K = W; g.scale = 1.f; g.act = ld.ff_act == 1 ? tgx::SG_ACT_GELU : tgx::SG_ACT_NONE;
    launch_gemm(c, g, tgx::SG_STORE, 1);
    g = tgx::StackGemmArgs{};
    g.A = sm->yh; g.lda = ld.ff; g.B = w.w_down; g.ldb = ld.ff; g.C = sm->yd; g.ldc = W; g.M = T; g.N = W; g.K = ld.ff; g.scale = 1.f;
    launch_gemm(c, g, tgx::SG_STORE, 1);
    return;
  }
  const int E = ld.experts, top = ld.top, np = T * top;
  g.A = sm->a; g.lda = W; g.B = w.w_router; g.ldb = W; g.C = sm->zr; g.ldc = E; g.M = T; g.N = E; g.K = W; g.scale = 1.f;
  launch_gemm(c, g, tgx::SG_STORE, 1, 0, 0, 64, tgx::DT_F32);
  tgx::RouterGroupArgs ra{};
  ra.z = sm->zr; ra.ldz = E; ra.corr = nullptr; ra.sel = sm->sel; ra.selw = sm->selw; ra.sgw = nullptr;
  ra.E = E; ra.top = top; ra.groups = ld.groups; ra.keep = ld.groups_keep; ra.scale = 1.f;
  ra.sigmoid_scores = ld.router_fn == 1; ra.group_top2 = ld.group_score == 1; ra.normalise = ld.router_norm;
  hipLaunchKernelGGL(tgx::router_group_kernel, dim3(T), dim3(64), 0, c->stream, ra);
  tgx::MoePlanArgs pa{};
  pa.sel = sm->sel; pa.n_pairs = np; pa.E = E; pa.top = top; pa.tile_m = grouped_tile_rows(c, np, W, ld.ff); pa.E_tiles = E;
  pa.off = sm->moe_off; pa.perm = sm->perm; pa.tok = sm->ptok; pa.tile_e = sm->tile_e; pa.tile_m0 = sm->tile_m0; pa.n_tiles = sm->n_tiles;
  hipLaunchKernelGGL(tgx::moe_plan_kernel, dim3(1), dim3(1024), 0, c->stream, pa);
  g = tgx::StackGemmArgs{};
  g.A = sm->a; g.lda = W; g.a_rows = sm->ptok; g.B = w.w_gate; g.B2 = w.w_up; g.ldb = W; g.b_zstride = (long long)ld.ff * W; g.C = sm->yh; g.ldc = ld.ff;
  g.z_off = sm->moe_off; g.tile_z = sm->tile_e; g.tile_m0 = sm->tile_m0; g.n_tiles = sm->n_tiles; g.M = np; g.N = ld.ff; g.K = W;
  launch_gemm(c, g, tgx::SG_SILU_MUL, 1, np, E, pa.tile_m);
  g = tgx::StackGemmArgs{};
  g.A = sm->yh; g.lda = ld.ff; g.B = w.w_down; g.ldb = ld.ff; g.b_zstride = (long long)W * ld.ff; g.C = sm->yd; g.ldc = W; g.c_rows = sm->perm;
  g.z_off = sm->moe_off; g.tile_z = sm->tile_e; g.tile_m0 = sm->tile_m0; g.n_tiles = sm->n_tiles; g.M = np; g.N = W; g.K = ld.ff; g.rw = sm->selw;
  launch_gemm(c, g, tgx::SG_ROWSCALE, 1, np, E, pa.tile_m);
  if (ld.shared_ff > 0) {      // the shared expert runs for every token, without a gate of its own
    float* hsh = sm->yh + (size_t)np * std::max(1, ld.ff);
    g = tgx::StackGemmArgs{};
    g.A = sm->a; g.lda = W; g.B = w.ws_gate; g.B2 = w.ws_up; g.ldb = W; g.C = hsh; g.ldc = ld.shared_ff; g.M = T; g.N = ld.shared_ff; g.K = W;
    launch_gemm(c, g, tgx::SG_SILU_MUL, 1);
    g = tgx::StackGemmArgs{};
    g.A = hsh; g.lda = ld.shared_ff; g.B = w.ws_down; g.ldb = ld.shared_ff; g.C = sm->ysh; g.ldc = W; g.M = T; g.N = W; g.K = ld.shared_ff; g.scale = 1.f;
    launch_gemm(c, g, tgx::SG_STORE, 1);
  }
}

int run_layers_affine(tgx_ctx* c, const MetaPtrs& mp, int T, int S, int max_keys, int max_count) {
  StackModel* sm = c->stack;
  const tgx::StepMeta m = step_meta(sm, mp, T, S);
  const int W = sm->d.width;
  const float eps = sm->d.norm_eps, mult = sm->d.residual_mult;
  const bool looped = sm->w_loop != nullptr;
  TGX_DT_SWITCH(c->dt, hipLaunchKernelGGL(tgx::embed_scale_rows_kernel<DT>, dim3(T), dim3(256), 0, c->stream, m, reinterpret_cast<const tgx::elem_t<DT>*>(c->embed), sm->d.embed_scale,
                                          sm->x, looped ? sm->xcat + W : nullptr, 2LL * W, W))
  bool normed = false;      // whether sm->a holds the next sublayer's normed input
  for (size_t ri = 0; ri < sm->runs.size(); ri++) {
    const StackRun& run = sm->runs[ri];
    StackLayerW& w = sm->L[(size_t)run.layer];
    const tgx_layer_desc& ld = w.d;
    const float* ln = w.ln;
    if (run.inject) {      // x <- W_loop [x; x0]
      hipLaunchKernelGGL(tgx::copy_rows_kernel, dim3(T), dim3(256), 0, c->stream, sm->x, (long long)W, sm->xcat, 2LL * W, W);
      tgx::StackGemmArgs g{};
      g.A = sm->xcat; g.lda = 2LL * W; g.B = sm->w_loop; g.ldb = 2LL * W; g.C = sm->x; g.ldc = W; g.M = T; g.N = W; g.K = 2 * W; g.scale = 1.f;
      launch_gemm(c, g, tgx::SG_STORE, 1);
      normed = false;
    }
    if (!normed) hipLaunchKernelGGL(tgx::layer_norm_rows_kernel, dim3(T), dim3(256), 0, c->stream, sm->x, nullptr, ln, ln + W, sm->a, W, eps);
    int rc = ld.mixer == TGX_MIXER_ATTENTION ? run_affine_attention(c, m, w, run, T, S, max_keys, max_count) : run_affine_latent(c, m, w, run, T, S, max_keys, max_count);
    if (rc) return rc;
    const bool last = ri + 1 == sm->runs.size();
    const bool next_direct = !last && !sm->runs[ri + 1].inject;      // the next run's first norm can ride in this run's last seam
    const float* next_ln = next_direct ? sm->L[(size_t)sm->runs[ri + 1].layer].ln : nullptr;
    tgx::AffineSeamArgs sa{};
    sa.x = sm->x; sa.y = sm->yd; sa.top = 1; sa.ytmp = sm->ytmp; sa.w_post = ln + 2 * (size_t)W; sa.b_post = ln + 3 * (size_t)W; sa.mult = mult; sa.out = sm->a; sa.W = W; sa.eps = eps;
    if (ld.mlp != TGX_MLP_NONE) { sa.w_next = ln + 4 * (size_t)W; sa.b_next = ln + 5 * (size_t)W; }
    else if (next_ln) { sa.w_next = next_ln; sa.b_next = next_ln + W; }
    hipLaunchKernelGGL(tgx::affine_seam_kernel, dim3(T), dim3(256), 0, c->stream, sa);
    normed = sa.w_next != nullptr;
    if (ld.mlp == TGX_MLP_NONE) continue;
    run_affine_ff(c, w, T);
    sa = tgx::AffineSeamArgs{};
    sa.x = sm->x; sa.y = sm->yd; sa.top = ld.mlp == TGX_MLP_MOE ? ld.top : 1; sa.ysh = ld.mlp == TGX_MLP_MOE && ld.shared_ff > 0 ? sm->ysh : nullptr; sa.ytmp = sm->ytmp;
    sa.w_post = ln + 6 * (size_t)W; sa.b_post = ln + 7 * (size_t)W; sa.mult = mult; sa.out = sm->a; sa.W = W; sa.eps = eps;
    if (next_ln) { sa.w_next = next_ln; sa.b_next = next_ln + W; }
    hipLaunchKernelGGL(tgx::affine_seam_kernel, dim3(T), dim3(256), 0, c->stream, sa);
    normed = sa.w_next != nullptr;
  }
  return TGX_OK;
}

// parameter storage of a layer-norm design (Zaluvik) and the list of its layer runs
int create_affine_layers(tgx_ctx* c, const tgx_layer_desc* layers) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  const size_t W = (size_t)d.width, es = c->esz;
  int rc;
  auto need = [&](const std::string& p, std::initializer_list<const char*> names) { for (const char* n : names) sm->missing.insert(p + n); };
  sm->missing.insert("final.norm.b");
  const bool looped = d.loop_times >= 1 && d.loop_stop > d.loop_start;      // (one pass still has the input product in front)
  if (looped) {
    if ((rc = dev_alloc(c, &sm->w_loop, W * 2 * W * es))) return rc;
    sm->missing.insert("loop.in");
  }
  for (int i = 0; i < d.layers; i++) {
    const int reps = looped && i >= d.loop_start && i < d.loop_stop ? 1 : 0;
    if (looped && i == d.loop_start) {
      for (int t = 0; t < d.loop_times; t++)
        for (int j = d.loop_start; j < d.loop_stop; j++) { StackRun r; r.layer = j; r.inject = j == d.loop_start; sm->runs.push_back(r); }
    }
    if (!reps) { StackRun r; r.layer = i; sm->runs.push_back(r); }
  }
  sm->max_top = 1; sm->max_E = 1; sm->max_ff = 1;      // the mixers' outputs and the dense feed-forward use the expert buffers with one row per token
  for (int i = 0; i < d.layers; i++) {
    StackLayerW& w = sm->L[(size_t)i];
    w.d = layers[i];
    const tgx_layer_desc& l = w.d;
    const std::string p = "l" + std::to_string(i) + ".";
    const size_t H = (size_t)l.heads, vd = H * l.vdim;
    if ((rc = dev_alloc(c, &w.ln, 8 * W))) return rc;
    HIP_OK(c, hipMemset(w.ln, 0, 8 * W * 4));
    need(p, {"norm1", "norm1.b", "norm1b", "norm1b.b", "mix.q", "mix.g", "mix.o"});
    size_t nin;
    if (l.mixer == TGX_MIXER_ATTENTION) {
      const size_t qd = H * l.dim, kd = (size_t)l.kv_heads * l.dim, kvv = (size_t)l.kv_heads * l.vdim;
      nin = qd + kd + kvv + vd;
      sm->max_qd = std::max(sm->max_qd, (int)qd);
      if ((rc = dev_alloc(c, &w.talk, H * H)) || (rc = dev_alloc(c, &w.pb, H))) return rc;
      HIP_OK(c, hipMemset(w.pb, 0, H * 4));
      need(p, {"mix.k", "mix.v"});
      if (l.head_mix) need(p, {"mix.talk"});
      if (l.score_fn == 1) need(p, {"mix.pb"});
    } else {
      const size_t qd = H * (size_t)(l.dim + l.rot_dim), R = (size_t)l.kv_rank, RR = R + l.rot_dim;
      nin = qd + RR + (l.gate_kind == 2 ? H : vd);
      if ((rc = dev_alloc(c, &w.w_ukT, H * l.dim * R * es)) || (rc = dev_alloc(c, &w.w_uv, vd * R * es)) || (rc = dev_alloc(c, &w.lat_norm, R))) return rc;
      need(p, {"mix.dkv", "mix.dkv.norm", "mix.uk", "mix.uv"});
      if (l.rot_dim > 0 && l.rot_dims > 0) {
        for (size_t r = 0; r < sm->rot.size(); r++) if (sm->rot[r].dims == l.rot_dims && sm->rot[r].base == l.rot_base) w.rot = (int)r;
        if (w.rot < 0) { w.rot = (int)sm->rot.size(); sm->rot.push_back(RotTable{l.rot_dims, l.rot_base, 1.f, nullptr}); }
      }
      sm->max_hr = std::max(sm->max_hr, (int)(H * RR));
    }
    if ((rc = dev_alloc(c, &w.w_in, nin * W * es)) || (rc = dev_alloc(c, &w.w_o, W * vd * es))) return rc;
    sm->max_in = std::max(sm->max_in, (int)nin); sm->max_hv = std::max(sm->max_hv, (int)vd);
    if (l.mlp == TGX_MLP_NONE) continue;
    need(p, {"norm2", "norm2.b", "norm2b", "norm2b.b"});
    if (l.mlp == TGX_MLP_DENSE) {
      const size_t F = (size_t)l.ff;
      if ((rc = dev_alloc(c, &w.w_up, F * W * es)) || (rc = dev_alloc(c, &w.w_down, W * F * es))) return rc;
      need(p, {"mlp.up", "mlp.down"});
      sm->max_ff = std::max(sm->max_ff, l.ff);
      continue;
    }
    const size_t E = (size_t)l.experts, F = (size_t)l.ff, SF = (size_t)l.shared_ff;
    if ((rc = dev_alloc(c, &w.w_router, E * W)) || (rc = dev_alloc(c, &w.w_gate, E * F * W * es)) || (rc = dev_alloc(c, &w.w_up, E * F * W * es)) || (rc = dev_alloc(c, &w.w_down, E * W * F * es))) return rc;
    need(p, {"mlp.router"});
    for (int e = 0; e < l.experts; e++)
      for (const char* n : {".gate", ".up", ".down"}) sm->missing.insert(p + "mlp.e" + std::to_string(e) + n);
    if (SF > 0) {
      if ((rc = dev_alloc(c, &w.ws_gate, SF * W * es)) || (rc = dev_alloc(c, &w.ws_up, SF * W * es)) || (rc = dev_alloc(c, &w.ws_down, W * SF * es))) return rc;
      need(p, {"mlp.shared.gate", "mlp.shared.up", "mlp.shared.down"});
    }
    sm->max_top = std::max(sm->max_top, l.top); sm->max_ff = std::max(sm->max_ff, l.ff); sm->max_E = std::max(sm->max_E, l.experts); sm->max_sff = std::max(sm->max_sff, l.shared_ff);
  }
  return TGX_OK;
}

// tensors of a layer-norm design by checkpoint name; a norm is a weight vector and a bias vector ("<name>.b")
int upload_affine(tgx_ctx* c, const char* name, const void* host, const int64_t* shape, int nd, int src_dtype) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  const int64_t W = d.width;
  const bool probe = nd < 0;
  auto bad_shape = [&]() { return set_err(c, TGX_ERR_SHAPE, "shape not equal for tensor: %s", name); };
  auto is = [&](int64_t a, int64_t b) { return b < 0 ? (nd == 1 && shape[0] == a) : (nd == 2 && shape[0] == a && shape[1] == b); };
  auto done = [&](int rc) { if (!rc) sm->missing.erase(name); return rc; };
  auto mat = [&](ebyte* dst, int64_t row0, int64_t rows, int64_t cols) {
    if (probe) return (int)TGX_ERR_SHAPE;
    if (!is(rows, cols)) return bad_shape();
    return done(upload_param_ext(c, dst + (size_t)(row0 * cols) * c->esz, host, rows * cols, src_dtype));
  };
  auto vec = [&](float* dst, int64_t n, int64_t n2 = -1) {      // an fp32 vector, or (n2 >= 0) an fp32 matrix [n][n2]
    if (probe) return (int)TGX_ERR_SHAPE;
    if (!is(n, n2)) return bad_shape();
    return done(upload_f32(c, dst, host, n2 < 0 ? n : n * n2, src_dtype));
  };
  if (!strcmp(name, "embed")) return mat(c->embed, 0, d.vocab, W);
  if (!strcmp(name, "final.norm")) return vec(sm->final_norm, W);
  if (!strcmp(name, "final.norm.b")) return vec(sm->final_norm + W, W);
  if (sm->w_loop && !strcmp(name, "loop.in")) return mat(sm->w_loop, 0, W, 2 * W);
  int li = -1;
  char rest[128] = {0};
  if (sscanf(name, "l%d.%127s", &li, rest) != 2 || li < 0 || li >= d.layers) return set_err(c, TGX_ERR_NAME, "Unexpected key: %s", name);
  StackLayerW& w = sm->L[(size_t)li];
  const tgx_layer_desc& l = w.d;
  const int64_t H = l.heads, vd = H * l.vdim;
  static const char* const norms[8] = {"norm1", "norm1.b", "norm1b", "norm1b.b", "norm2", "norm2.b", "norm2b", "norm2b.b"};
  for (int k = 0; k < (l.mlp == TGX_MLP_NONE ? 4 : 8); k++) if (!strcmp(rest, norms[k])) return vec(w.ln + (size_t)k * W, W);
  if (!strcmp(rest, "mix.o")) return mat(w.w_o, 0, W, vd);
  if (l.mixer == TGX_MIXER_ATTENTION) {
    const int64_t qd = H * l.dim, kd = (int64_t)l.kv_heads * l.dim, kvv = (int64_t)l.kv_heads * l.vdim;
    if (!strcmp(rest, "mix.q")) return mat(w.w_in, 0, qd, W);
    if (!strcmp(rest, "mix.k")) return mat(w.w_in, qd, kd, W);
    if (!strcmp(rest, "mix.v")) return mat(w.w_in, qd + kd, kvv, W);
    if (!strcmp(rest, "mix.g")) return mat(w.w_in, qd + kd + kvv, vd, W);
    if (l.head_mix && !strcmp(rest, "mix.talk")) return vec(w.talk, H, H);
    if (l.score_fn == 1 && !strcmp(rest, "mix.pb")) return vec(w.pb, H);
  } else {
    const int64_t qd = H * (int64_t)(l.dim + l.rot_dim), R = l.kv_rank, RR = R + l.rot_dim;
    if (!strcmp(rest, "mix.q")) return mat(w.w_in, 0, qd, W);
    if (!strcmp(rest, "mix.dkv")) return mat(w.w_in, qd, RR, W);
    if (!strcmp(rest, "mix.g")) return mat(w.w_in, qd + RR, l.gate_kind == 2 ? H : vd, W);
    if (!strcmp(rest, "mix.dkv.norm")) return vec(w.lat_norm, R);
    if (!strcmp(rest, "mix.uv")) return mat(w.w_uv, 0, vd, R);
    if (!strcmp(rest, "mix.uk")) {      // [heads * dim][rank] -> per head [rank][dim]
      if (probe) return TGX_ERR_SHAPE;
      if (!is(H * l.dim, R)) return bad_shape();
      const size_t es = esize(src_dtype);
      std::vector<unsigned char> t((size_t)(H * l.dim * R) * es);
      const unsigned char* src = (const unsigned char*)host;
      for (int64_t h = 0; h < H; h++)
        for (int64_t dd = 0; dd < l.dim; dd++)
          for (int64_t r = 0; r < R; r++) memcpy(&t[(size_t)((h * R + r) * l.dim + dd) * es], src + (size_t)((h * l.dim + dd) * R + r) * es, es);
      return done(upload_param_ext(c, w.w_ukT, t.data(), H * l.dim * R, src_dtype));
    }
  }
  if (l.mlp == TGX_MLP_DENSE) {
    if (!strcmp(rest, "mlp.up")) return mat(w.w_up, 0, l.ff, W);
    if (!strcmp(rest, "mlp.down")) return mat(w.w_down, 0, W, l.ff);
  }
  if (l.mlp == TGX_MLP_MOE) {
    const int64_t E = l.experts, F = l.ff, SF = l.shared_ff;
    if (!strcmp(rest, "mlp.router")) return vec(w.w_router, E, W);
    if (SF > 0) {
      if (!strcmp(rest, "mlp.shared.gate")) return mat(w.ws_gate, 0, SF, W);
      if (!strcmp(rest, "mlp.shared.up")) return mat(w.ws_up, 0, SF, W);
      if (!strcmp(rest, "mlp.shared.down")) return mat(w.ws_down, 0, W, SF);
    }
    int e = -1;
    char leaf[32] = {0};
    if (sscanf(rest, "mlp.e%d.%31s", &e, leaf) == 2 && e >= 0 && e < E) {
      if (!strcmp(leaf, "gate")) return mat(w.w_gate, e * F, F, W);
      if (!strcmp(leaf, "up")) return mat(w.w_up, e * F, F, W);
      if (!strcmp(leaf, "down")) return mat(w.w_down, e * W, W, F);
    }
  }
  return set_err(c, TGX_ERR_NAME, "Unexpected key: %s", name);
}

// what a layer-norm design's description may ask for
int check_affine_desc(const tgx_stack_desc& d, const tgx_layer_desc* layers) {
  if (d.loop_times >= 1 && d.loop_stop > d.loop_start && (d.loop_start < 0 || d.loop_stop > d.layers)) return set_err(nullptr, TGX_ERR_INVALID, "loop %d .. %d outside the %d layers", d.loop_start, d.loop_stop, d.layers);
  for (int i = 0; i < d.layers; i++) {
    const tgx_layer_desc& l = layers[i];
    if (l.heads <= 0 || l.dim <= 0 || l.vdim <= 0) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: non-positive mixer size", i);
    if (l.mask_kind < 0 || l.mask_kind > 2 || (l.mask_kind != 0 && l.mask_size < 1)) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: mask", i);
    if (l.mixer == TGX_MIXER_ATTENTION) {
      if (l.kv_heads <= 0 || l.heads % l.kv_heads) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: %d query heads over %d key / value heads", i, l.heads, l.kv_heads);
      if (l.score_fn != 1) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: this family's attention takes sigmoid weights (score_fn 1)", i);
      if ((long long)l.heads * l.vdim > MIX_ATTN_MAX_OUT || tgx::mix_attn_lds_bytes(l.heads, l.dim, 32) > MIX_ATTN_MAX_LDS)
        return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: sigmoid attention: %d heads of %d / %d exceed the kernel's %d output channels or its LDS", i, l.heads, l.dim, l.vdim, MIX_ATTN_MAX_OUT);
      if (l.gate_kind != 0 && l.gate_kind != 1) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: attention gates are per channel", i);
    } else if (l.mixer == TGX_MIXER_LATENT_ATTENTION) {
      if (l.kv_rank <= 0 || l.rot_dim < 0 || l.kv_rank + l.rot_dim > 64 * tgx::LAT_MAX_RPL) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: kv_rank %d + rot_dim %d (1 .. %d)", i, l.kv_rank, l.rot_dim, 64 * tgx::LAT_MAX_RPL);
      if (l.rot_dim > 0 && (l.rot_dims < 0 || l.rot_dims > l.rot_dim || (l.rot_dims & 1) || (l.rot_dims > 0 && !(l.rot_base > 0.f)))) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: %d rotated dimensions of %d (base %g)", i, l.rot_dims, l.rot_dim, l.rot_base);
      if (l.gate_kind != 1 && l.gate_kind != 2) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: latent attention gates are per channel or per head", i);
    } else return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: mixer %d is not part of this family (attention and latent_attention are)", i, l.mixer);
    if (l.mlp != TGX_MLP_NONE && l.mlp != TGX_MLP_MOE && l.mlp != TGX_MLP_DENSE) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: feed-forward kind %d is not implemented", i, l.mlp);
    if (l.mlp == TGX_MLP_DENSE && l.ff <= 0) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: ff %d", i, l.ff);
    if (l.mlp == TGX_MLP_MOE) {
      const int E = l.experts;
      if (E <= 0 || E >= tgx::ROUTER_MAX_E || l.top <= 0 || l.top > E || l.top > tgx::ROUTER_MAX_TOP || l.ff <= 0 || l.shared_ff < 0 || l.identity != 0)
        return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: experts %d (< %d), top %d (<= %d), ff %d", i, E, tgx::ROUTER_MAX_E, l.top, tgx::ROUTER_MAX_TOP, l.ff);
      if (l.groups > 1 && (E % l.groups || l.groups_keep < 1 || l.groups_keep > l.groups || (long long)l.groups_keep * (E / l.groups) < l.top))
        return set_err(nullptr, TGX_ERR_INVALID, "layer %d: %d experts in %d groups, %d kept, top %d", i, E, l.groups, l.groups_keep, l.top);
    }
  }
  return TGX_OK;
}

int run_layers(tgx_ctx* c, const MetaPtrs& mp, int T, int S, int max_keys, int max_count) {
  if (c->stack->affine) return run_layers_affine(c, mp, T, S, max_keys, max_count);
  if (c->stack->joint) return run_layers_joint(c, mp, T, S, max_keys, max_count);
  return c->stack->sandwich ? run_layers_sandwich(c, mp, T, S, max_keys, max_count) : run_layers_latent(c, mp, T, S, max_keys, max_count);
}

// logits of the rows listed in want_dev (indices into the step's tokens): C[crow(i)] = embed . norm(x[want[i]]) * logit_scale
void run_logits(tgx_ctx* c, const int* want_dev, int nw, float* C, const int* c_rows) {
  StackModel* sm = c->stack;
  const int W = sm->d.width, V = sm->d.vocab;
  if (sm->affine) hipLaunchKernelGGL(tgx::layer_norm_rows_kernel, dim3(nw), dim3(256), 0, c->stream, sm->x, want_dev, sm->final_norm, sm->final_norm + W, sm->xn, W, sm->d.norm_eps);
  else if (sm->joint) hipLaunchKernelGGL(tgx::offset_norm_kernel, dim3(nw), dim3(256), 0, c->stream, sm->x, want_dev, sm->final_norm, 1.0f, sm->xn, W, sm->d.norm_eps);
  else if (sm->sandwich) hipLaunchKernelGGL(tgx::scalar_norm_kernel, dim3(nw), dim3(256), 0, c->stream, sm->x, want_dev, sm->norm_g + 4 * (size_t)sm->d.layers, sm->xn, W, sm->d.norm_eps);
  else hipLaunchKernelGGL(tgx::final_norm_rows_kernel, dim3(nw), dim3(256), 0, c->stream, sm->x, want_dev, sm->final_norm, sm->xn, W, sm->d.norm_groups, sm->d.norm_eps);
  tgx::StackGemmArgs g{};
  g.A = sm->xn; g.lda = W; g.B = sm->head ? sm->head : c->embed; g.ldb = W; g.C = C; g.ldc = V; g.c_rows = c_rows; g.M = nw; g.N = V; g.K = W; g.scale = sm->d.logit_scale;
  launch_gemm(c, g, tgx::SG_STORE, 1);
}

// pages for `tokens` tokens of a slot; the caller has checked that enough are free
void assign_pages(StackModel* sm, int row, long long tokens) {
  const int need = (int)((tokens + sm->page - 1) / sm->page);
  int& have = sm->row_pages[(size_t)row];
  for (; have < need; have++) {
    sm->tbl_host[(size_t)row * sm->tbl_stride + have] = sm->free_pages.back();
    sm->free_pages.pop_back();
    sm->row_dirty[(size_t)row] = 1;
  }
}
int push_tables(tgx_ctx* c) {
  StackModel* sm = c->stack;
  for (int r = 0; r < sm->d.max_seqs; r++)
    if (sm->row_dirty[(size_t)r]) {
      const size_t o = (size_t)r * sm->tbl_stride;
      HIP_OK(c, hipMemcpyAsync(sm->tbl_dev + o, sm->tbl_host + o, (size_t)std::max(1, sm->row_pages[(size_t)r]) * 4, hipMemcpyHostToDevice, c->stream));
      sm->row_dirty[(size_t)r] = 0;
    }
  return TGX_OK;
}
int push_meta(tgx_ctx* c, size_t n) {
  StackModel* sm = c->stack;
  HIP_OK(c, hipMemcpyAsync(sm->meta_dev, sm->meta_host, n * 4, hipMemcpyHostToDevice, c->stream));
  HIP_OK(c, hipEventRecord(sm->meta_ev, c->stream));
  sm->meta_pending = true;
  return TGX_OK;
}
int meta_host_free(tgx_ctx* c) {      // the pinned staging block may be rewritten once the last copy out of it has run
  StackModel* sm = c->stack;
  if (sm->meta_pending) { HIP_OK(c, hipEventSynchronize(sm->meta_ev)); sm->meta_pending = false; }
  return TGX_OK;
}

void refresh_rows(tgx_ctx* c) {
  int64_t m = 0; int live = 0; bool all = true;
  for (int b = 0; b < c->batch; b++) {
    if (c->row_idle[(size_t)b]) continue;
    live++; m = std::max(m, c->row_past[(size_t)b]); all = all && c->row_tok[(size_t)b];
  }
  c->past = m; c->have_token = live > 0 && all;
}

// parameter storage of a sandwich-norm design (Modepel): per layer the four norm numbers, the mixer's merged input projection with its bias row, the
// output projection, and the feed-forward of its kind
int create_sandwich_layers(tgx_ctx* c, const tgx_layer_desc* layers) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  const size_t W = (size_t)d.width, es = c->esz;
  int rc;
  if ((rc = dev_alloc(c, &sm->head, (size_t)d.vocab * W * es)) || (rc = dev_alloc(c, &sm->norm_g, (size_t)4 * d.layers + 1))) return rc;
  HIP_OK(c, hipMemset(sm->norm_g, 0, ((size_t)4 * d.layers + 1) * 4));
  sm->missing.insert("head");
  sm->max_top = 1; sm->max_E = 1; sm->max_ff = 1;      // the mixers' outputs and the dense feed-forward use the expert buffers with one row per token
  bool mixing = false;
  for (int i = 0; i < d.layers; i++) {
    StackLayerW& w = sm->L[(size_t)i];
    w.d = layers[i];
    const tgx_layer_desc& l = w.d;
    const std::string p = "l" + std::to_string(i) + ".";
    const size_t H = (size_t)l.heads, qd = H * l.dim, vd = H * l.vdim;
    size_t nin;
    for (const char* n : {"norm1", "norm1b", "mix.q", "mix.k", "mix.v", "mix.g", "mix.o"}) sm->missing.insert(p + n);
    if (l.mixer == TGX_MIXER_ATTENTION) {
      const size_t kd = (size_t)l.kv_heads * l.dim, kvv = (size_t)l.kv_heads * l.vdim;
      nin = qd + kd + kvv + vd;
      for (const char* n : {"mix.q.b", "mix.k.b", "mix.v.b"}) sm->missing.insert(p + n);
      if (l.v_mix) {
        if ((rc = dev_alloc(c, &w.vmix, 1))) return rc;
        HIP_OK(c, hipMemset(w.vmix, 0, 4));
        w.vmode = mixing ? 2 : 1;
        if (w.vmode == 2) sm->missing.insert(p + "mix.vmix");      // (the first mixing layer's number is never read: taken if the checkpoint has it, not asked for)
        mixing = true;
      }
      if (l.rot_dims > 0) {
        for (size_t r = 0; r < sm->rot.size(); r++) if (sm->rot[r].dims == l.rot_dims && sm->rot[r].base == l.rot_base) w.rot = (int)r;
        if (w.rot < 0) { w.rot = (int)sm->rot.size(); sm->rot.push_back(RotTable{l.rot_dims, l.rot_base, 1.f, nullptr}); }
      }
      sm->max_kvv = std::max(sm->max_kvv, (int)kvv);
    } else {
      nin = 2 * qd + 2 * vd + 2 * H;
      if ((rc = dev_alloc(c, &w.head_w, vd))) return rc;
      for (const char* n : {"mix.norm", "mix.i", "mix.i.b", "mix.f", "mix.f.b"}) sm->missing.insert(p + n);
    }
    if ((rc = dev_alloc(c, &w.w_in, nin * W * es)) || (rc = dev_alloc(c, &w.b_in, nin)) || (rc = dev_alloc(c, &w.w_o, W * vd * es))) return rc;
    HIP_OK(c, hipMemset(w.b_in, 0, nin * 4));
    sm->max_in = std::max(sm->max_in, (int)nin); sm->max_hv = std::max(sm->max_hv, (int)vd);
    if (l.mlp == TGX_MLP_NONE) continue;
    for (const char* n : {"norm2", "norm2b"}) sm->missing.insert(p + n);
    if (l.mlp == TGX_MLP_DENSE) {
      const size_t F = (size_t)l.ff;
      if ((rc = dev_alloc(c, &w.w_up, F * W * es)) || (rc = dev_alloc(c, &w.w_down, W * F * es)) || (rc = dev_alloc(c, &w.act, 4))) return rc;
      for (const char* n : {"mlp.up", "mlp.down", "mlp.act"}) sm->missing.insert(p + n);
      sm->max_ff = std::max(sm->max_ff, l.ff);
      continue;
    }
    const size_t E = (size_t)l.experts, Et = E + (size_t)l.identity, F = (size_t)l.ff, SF = (size_t)l.shared_ff;
    if ((rc = dev_alloc(c, &w.w_router, (Et + 1) * W)) || (rc = dev_alloc(c, &w.b_router, Et))) return rc;
    for (const char* n : {"mlp.router", "mlp.correction"}) sm->missing.insert(p + n);
    if (E > 0) {
      if ((rc = dev_alloc(c, &w.w_gate, E * F * W * es)) || (rc = dev_alloc(c, &w.w_up, E * F * W * es)) || (rc = dev_alloc(c, &w.w_down, E * W * F * es))) return rc;
      for (int e = 0; e < l.experts; e++)
        for (const char* n : {".gate", ".up", ".down"}) sm->missing.insert(p + "mlp.e" + std::to_string(e) + n);
    }
    if (SF > 0) {
      if ((rc = dev_alloc(c, &w.ws_gate, SF * W * es)) || (rc = dev_alloc(c, &w.ws_up, SF * W * es)) || (rc = dev_alloc(c, &w.ws_down, W * SF * es))) return rc;
      for (const char* n : {"mlp.shared.gate", "mlp.shared.up", "mlp.shared.down", "mlp.shared.sg"}) sm->missing.insert(p + n);
    }
    sm->max_top = std::max(sm->max_top, l.top); sm->max_ff = std::max(sm->max_ff, l.ff); sm->max_E = std::max(sm->max_E, (int)Et); sm->max_sff = std::max(sm->max_sff, l.shared_ff);
  }
  return TGX_OK;
}

// tensors of a sandwich-norm design by checkpoint name.  A norm is one number (shape [] or [1]).
int upload_sandwich(tgx_ctx* c, const char* name, const void* host, const int64_t* shape, int nd, int src_dtype) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  const int64_t W = d.width;
  const bool probe = nd < 0;
  auto bad_shape = [&]() { return set_err(c, TGX_ERR_SHAPE, "shape not equal for tensor: %s", name); };
  auto is = [&](int64_t a, int64_t b) { return b < 0 ? (nd == 1 && shape[0] == a) : (nd == 2 && shape[0] == a && shape[1] == b); };
  auto is_one = [&]() { return nd == 0 || (nd == 1 && shape[0] == 1); };
  auto done = [&](int rc) { if (!rc) sm->missing.erase(name); return rc; };
  auto mat = [&](ebyte* dst, int64_t row0, int64_t rows, int64_t cols) {
    if (probe) return (int)TGX_ERR_SHAPE;
    if (!is(rows, cols)) return bad_shape();
    return done(upload_param_ext(c, dst + (size_t)(row0 * cols) * c->esz, host, rows * cols, src_dtype));
  };
  auto vec = [&](float* dst, int64_t n) {
    if (probe) return (int)TGX_ERR_SHAPE;
    if (!(n == 1 ? is_one() : is(n, -1))) return bad_shape();
    return done(upload_f32(c, dst, host, n, src_dtype));
  };
  if (!strcmp(name, "embed")) return mat(c->embed, 0, d.vocab, W);
  if (!strcmp(name, "head")) return mat(sm->head, 0, d.vocab, W);
  if (!strcmp(name, "final.norm")) return vec(sm->norm_g + 4 * (size_t)d.layers, 1);
  int li = -1;
  char rest[128] = {0};
  if (sscanf(name, "l%d.%127s", &li, rest) != 2 || li < 0 || li >= d.layers) return set_err(c, TGX_ERR_NAME, "Unexpected key: %s", name);
  StackLayerW& w = sm->L[(size_t)li];
  const tgx_layer_desc& l = w.d;
  const int64_t H = l.heads, qd = H * l.dim, vd = H * l.vdim;
  float* ng = sm->norm_g + 4 * (size_t)li;
  if (!strcmp(rest, "norm1")) return vec(ng, 1);
  if (!strcmp(rest, "norm1b")) return vec(ng + 1, 1);
  if (l.mlp != TGX_MLP_NONE && !strcmp(rest, "norm2")) return vec(ng + 2, 1);
  if (l.mlp != TGX_MLP_NONE && !strcmp(rest, "norm2b")) return vec(ng + 3, 1);
  if (!strcmp(rest, "mix.o")) return mat(w.w_o, 0, W, vd);
  if (l.mixer == TGX_MIXER_ATTENTION) {
    const int64_t kd = (int64_t)l.kv_heads * l.dim, kvv = (int64_t)l.kv_heads * l.vdim;
    if (!strcmp(rest, "mix.q")) return mat(w.w_in, 0, qd, W);
    if (!strcmp(rest, "mix.k")) return mat(w.w_in, qd, kd, W);
    if (!strcmp(rest, "mix.v")) return mat(w.w_in, qd + kd, kvv, W);
    if (!strcmp(rest, "mix.g")) return mat(w.w_in, qd + kd + kvv, vd, W);
    if (!strcmp(rest, "mix.q.b")) return vec(w.b_in, qd);
    if (!strcmp(rest, "mix.k.b")) return vec(w.b_in + qd, kd);
    if (!strcmp(rest, "mix.v.b")) return vec(w.b_in + qd + kd, kvv);
    if (w.vmix && !strcmp(rest, "mix.vmix")) return vec(w.vmix, 1);
  } else {
    if (!strcmp(rest, "mix.q")) return mat(w.w_in, 0, qd, W);
    if (!strcmp(rest, "mix.k")) return mat(w.w_in, qd, qd, W);
    if (!strcmp(rest, "mix.v")) return mat(w.w_in, 2 * qd, vd, W);
    if (!strcmp(rest, "mix.g")) return mat(w.w_in, 2 * qd + vd, vd, W);
    if (!strcmp(rest, "mix.i")) return mat(w.w_in, 2 * qd + 2 * vd, H, W);
    if (!strcmp(rest, "mix.f")) return mat(w.w_in, 2 * qd + 2 * vd + H, H, W);
    if (!strcmp(rest, "mix.i.b")) return vec(w.b_in + 2 * qd + 2 * vd, H);
    if (!strcmp(rest, "mix.f.b")) return vec(w.b_in + 2 * qd + 2 * vd + H, H);
    if (!strcmp(rest, "mix.norm")) return vec(w.head_w, vd);
  }
  if (l.mlp == TGX_MLP_DENSE) {
    if (!strcmp(rest, "mlp.up")) return mat(w.w_up, 0, l.ff, W);
    if (!strcmp(rest, "mlp.down")) return mat(w.w_down, 0, W, l.ff);
    if (!strcmp(rest, "mlp.act")) return vec(w.act, 4);
  }
  if (l.mlp == TGX_MLP_MOE) {
    const int64_t E = l.experts, Et = E + l.identity, F = l.ff, SF = l.shared_ff;
    if (!strcmp(rest, "mlp.router")) { if (probe) return TGX_ERR_SHAPE; if (!is(Et, W)) return bad_shape(); return done(upload_f32(c, w.w_router, host, Et * W, src_dtype)); }
    if (!strcmp(rest, "mlp.correction")) return vec(w.b_router, Et);
    if (SF > 0) {
      if (!strcmp(rest, "mlp.shared.gate")) return mat(w.ws_gate, 0, SF, W);
      if (!strcmp(rest, "mlp.shared.up")) return mat(w.ws_up, 0, SF, W);
      if (!strcmp(rest, "mlp.shared.down")) return mat(w.ws_down, 0, W, SF);
      if (!strcmp(rest, "mlp.shared.sg")) {      // the shared expert's gate row rides behind the router rows: one fp32 product serves both
        if (probe) return TGX_ERR_SHAPE;
        if (!is(1, W) && !is(W, -1)) return bad_shape();
        return done(upload_f32(c, w.w_router + (size_t)(Et * W), host, W, src_dtype));
      }
    }
    int e = -1;
    char leaf[32] = {0};
    if (sscanf(rest, "mlp.e%d.%31s", &e, leaf) == 2 && e >= 0 && e < E) {
      if (!strcmp(leaf, "gate")) return mat(w.w_gate, e * F, F, W);
      if (!strcmp(leaf, "up")) return mat(w.w_up, e * F, F, W);
      if (!strcmp(leaf, "down")) return mat(w.w_down, e * W, W, F);
    }
  }
  return set_err(c, TGX_ERR_NAME, "Unexpected key: %s", name);
}

// parameter storage of a parallel-sublayer design (Vitudra): per layer the norm weight, the mixer of its kind and the gated feed-forward
int create_joint_layers(tgx_ctx* c, const tgx_layer_desc* layers) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  const size_t W = (size_t)d.width, es = c->esz;
  int rc;
  if ((rc = dev_alloc(c, &sm->head, (size_t)d.vocab * W * es))) return rc;
  sm->missing.insert("head");
  sm->max_top = 1; sm->max_E = 1; sm->max_ff = 1;      // the feed-forward's hidden row uses the expert buffers with one row per token
  auto need = [&](const std::string& p, std::initializer_list<const char*> names) { for (const char* n : names) sm->missing.insert(p + n); };
  for (int i = 0; i < d.layers; i++) {
    StackLayerW& w = sm->L[(size_t)i];
    w.d = layers[i];
    const tgx_layer_desc& l = w.d;
    const std::string p = "l" + std::to_string(i) + ".";
    if ((rc = dev_alloc(c, &w.norm1, W))) return rc;
    need(p, {"norm1"});
    auto rotation = [&]() {
      if (l.rot_dims <= 0) return;
      const float factor = l.rot_factor > 0.f ? l.rot_factor : 1.f;
      for (size_t r = 0; r < sm->rot.size(); r++) if (sm->rot[r].dims == l.rot_dims && sm->rot[r].base == l.rot_base && sm->rot[r].factor == factor) w.rot = (int)r;
      if (w.rot < 0) { w.rot = (int)sm->rot.size(); sm->rot.push_back(RotTable{l.rot_dims, l.rot_base, factor, nullptr}); }
    };
    if (l.mixer == TGX_MIXER_ATTENTION) {
      w.kv_src = l.kv_share - 1;
      const size_t qd = (size_t)l.heads * l.dim, vd = (size_t)l.heads * l.vdim, nin = qd + (w.kv_src >= 0 ? 0 : (size_t)l.kv_heads * (l.dim + l.vdim));
      if ((rc = dev_alloc(c, &w.w_in, nin * W * es)) || (rc = dev_alloc(c, &w.w_o, W * vd * es))) return rc;
      need(p, {"mix.q", "mix.o"});
      if (w.kv_src < 0) need(p, {"mix.k", "mix.v"});
      rotation();
      sm->max_in = std::max(sm->max_in, (int)nin); sm->max_hv = std::max(sm->max_hv, (int)vd);
    } else if (l.mixer == TGX_MIXER_WKV) {
      const size_t HD = (size_t)l.heads * l.dim;
      if ((rc = dev_alloc(c, &w.w_in, 4 * HD * W * es)) || (rc = dev_alloc(c, &w.w_o, W * HD * es)) || (rc = dev_alloc(c, &w.mu, 5 * W)) || (rc = dev_alloc(c, &w.w0, HD)) ||
          (rc = dev_alloc(c, &w.ubonus, HD)) || (rc = dev_alloc(c, &w.head_w, HD))) return rc;
      if (l.decay_rank > 0 && ((rc = dev_alloc(c, &w.w_w1, (size_t)l.decay_rank * W * es)) || (rc = dev_alloc(c, &w.w_w2, HD * l.decay_rank * es)))) return rc;
      need(p, {"mix.mu.r", "mix.mu.k", "mix.mu.v", "mix.mu.g", "mix.mu.w", "mix.r", "mix.k", "mix.v", "mix.g", "mix.w1", "mix.w2", "mix.w0", "mix.u", "mix.norm", "mix.o"});
      sm->max_in = std::max(sm->max_in, (int)(5 * HD)); sm->max_hv = std::max(sm->max_hv, (int)HD); sm->max_shift = std::max(sm->max_shift, (int)(5 * W));
      sm->max_lora = std::max(sm->max_lora, l.decay_rank);
    } else {
      const size_t lq = (size_t)l.heads * l.dim, lkv = (size_t)l.kv_heads * (l.dim + l.vdim), lvd = (size_t)l.heads * l.vdim;
      const size_t rGD = (size_t)l.d_kv_heads * l.d_dim, rvd = (size_t)l.d_heads * l.d_vdim, rC = 2 * rGD + rvd, nin = lq + lkv + rC + 2 * (size_t)l.d_heads + rvd;
      if ((rc = dev_alloc(c, &w.w_in, nin * W * es)) || (rc = dev_alloc(c, &w.w_o, W * lvd * es)) || (rc = dev_alloc(c, &w.w_o2, W * rvd * es)) ||
          (rc = dev_alloc(c, &w.conv_w, rC * (size_t)l.conv_taps)) || (rc = dev_alloc(c, &w.a_log, (size_t)l.d_heads)) || (rc = dev_alloc(c, &w.dt_bias, (size_t)l.d_heads)) ||
          (rc = dev_alloc(c, &w.head_w, (size_t)l.d_vdim))) return rc;
      need(p, {"mix.left.q", "mix.left.k", "mix.left.v", "mix.left.o", "mix.right.q", "mix.right.k", "mix.right.v", "mix.right.q.conv", "mix.right.k.conv", "mix.right.v.conv",
               "mix.right.b", "mix.right.a", "mix.right.A_log", "mix.right.dt_bias", "mix.right.g", "mix.right.norm", "mix.right.o"});
      rotation();
      sm->max_in = std::max(sm->max_in, (int)nin); sm->max_hv = std::max(sm->max_hv, (int)std::max(lvd, rvd)); sm->max_rec = std::max(sm->max_rec, (int)(rC + 2 * (size_t)l.d_heads));
    }
    if (l.mlp == TGX_MLP_DENSE) {
      const size_t F = (size_t)l.ff;
      if ((rc = dev_alloc(c, &w.w_gate, F * W * es)) || (rc = dev_alloc(c, &w.w_up, F * W * es)) || (rc = dev_alloc(c, &w.w_down, W * F * es))) return rc;
      need(p, {"mlp.gate", "mlp.up", "mlp.down"});
      sm->max_ff = std::max(sm->max_ff, l.ff);
    }
  }
  return TGX_OK;
}

// tensors of a parallel-sublayer design by checkpoint name
int upload_joint(tgx_ctx* c, const char* name, const void* host, const int64_t* shape, int nd, int src_dtype) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  const int64_t W = d.width;
  const bool probe = nd < 0;
  auto bad_shape = [&]() { return set_err(c, TGX_ERR_SHAPE, "shape not equal for tensor: %s", name); };
  auto is = [&](int64_t a, int64_t b) { return b < 0 ? (nd == 1 && shape[0] == a) : (nd == 2 && shape[0] == a && shape[1] == b); };
  auto done = [&](int rc) { if (!rc) sm->missing.erase(name); return rc; };
  auto mat = [&](ebyte* dst, int64_t row0, int64_t rows, int64_t cols) {
    if (probe) return (int)TGX_ERR_SHAPE;
    if (!is(rows, cols)) return bad_shape();
    return done(upload_param_ext(c, dst + (size_t)(row0 * cols) * c->esz, host, rows * cols, src_dtype));
  };
  auto vec = [&](float* dst, int64_t n, int64_t n2 = -1) {      // an fp32 vector, or (n2 >= 0) an fp32 matrix [n][n2]
    if (probe) return (int)TGX_ERR_SHAPE;
    if (!is(n, n2)) return bad_shape();
    return done(upload_f32(c, dst, host, n2 < 0 ? n : n * n2, src_dtype));
  };
  if (!strcmp(name, "embed")) return mat(c->embed, 0, d.vocab, W);
  if (!strcmp(name, "head")) return mat(sm->head, 0, d.vocab, W);
  if (!strcmp(name, "final.norm")) return vec(sm->final_norm, W);
  int li = -1;
  char rest[128] = {0};
  if (sscanf(name, "l%d.%127s", &li, rest) != 2 || li < 0 || li >= d.layers) return set_err(c, TGX_ERR_NAME, "Unexpected key: %s", name);
  StackLayerW& w = sm->L[(size_t)li];
  tgx_layer_desc& l = w.d;
  if (!strcmp(rest, "norm1")) return vec(w.norm1, W);
  if (l.mlp == TGX_MLP_DENSE) {
    if (!strcmp(rest, "mlp.gate")) return mat(w.w_gate, 0, l.ff, W);
    if (!strcmp(rest, "mlp.up")) return mat(w.w_up, 0, l.ff, W);
    if (!strcmp(rest, "mlp.down")) return mat(w.w_down, 0, W, l.ff);
  }
  if (l.mixer == TGX_MIXER_ATTENTION) {
    const int64_t qd = (int64_t)l.heads * l.dim, kd = (int64_t)l.kv_heads * l.dim, kvv = (int64_t)l.kv_heads * l.vdim;
    if (!strcmp(rest, "mix.q")) return mat(w.w_in, 0, qd, W);
    if (!strcmp(rest, "mix.o")) return mat(w.w_o, 0, W, (int64_t)l.heads * l.vdim);
    if (w.kv_src < 0 && !strcmp(rest, "mix.k")) return mat(w.w_in, qd, kd, W);
    if (w.kv_src < 0 && !strcmp(rest, "mix.v")) return mat(w.w_in, qd + kd, kvv, W);
  } else if (l.mixer == TGX_MIXER_WKV) {
    const int64_t HD = (int64_t)l.heads * l.dim;
    const char* order = "rkvgw";
    if (!strncmp(rest, "mix.mu.", 7) && rest[7] && !rest[8] && strchr(order, rest[7])) return vec(w.mu + (size_t)(strchr(order, rest[7]) - order) * W, W);
    if (!strncmp(rest, "mix.", 4) && rest[4] && !rest[5] && strchr("rkvg", rest[4])) return mat(w.w_in, (strchr(order, rest[4]) - order) * HD, HD, W);
    if (!strcmp(rest, "mix.w1") || !strcmp(rest, "mix.w2")) {      // the inner size of the decay's product is the tensors' own where the description leaves it open
      if (probe) return TGX_ERR_SHAPE;
      const bool first = rest[5] == '1';
      if (nd != 2) return bad_shape();
      if (l.decay_rank <= 0) {
        const int64_t R = first ? shape[0] : shape[1];
        if (R <= 0 || R > 65536) return bad_shape();
        int rc;
        if ((rc = dev_alloc(c, &w.w_w1, (size_t)(R * W) * c->esz)) || (rc = dev_alloc(c, &w.w_w2, (size_t)(HD * R) * c->esz))) return rc;
        l.decay_rank = (int32_t)R;
        sm->max_lora = std::max(sm->max_lora, l.decay_rank);
      }
      return first ? mat(w.w_w1, 0, l.decay_rank, W) : mat(w.w_w2, 0, HD, l.decay_rank);
    }
    if (!strcmp(rest, "mix.w0")) return vec(w.w0, HD);
    if (!strcmp(rest, "mix.u")) return nd == 1 ? vec(w.ubonus, HD) : vec(w.ubonus, l.heads, l.dim);
    if (!strcmp(rest, "mix.norm")) return vec(w.head_w, HD);
    if (!strcmp(rest, "mix.o")) return mat(w.w_o, 0, W, HD);
  } else {
    const int64_t lq = (int64_t)l.heads * l.dim, lk = (int64_t)l.kv_heads * l.dim, lv = (int64_t)l.kv_heads * l.vdim, lvd = (int64_t)l.heads * l.vdim;
    const int64_t rGD = (int64_t)l.d_kv_heads * l.d_dim, rvd = (int64_t)l.d_heads * l.d_vdim, r0 = lq + lk + lv, rH = l.d_heads;
    if (!strcmp(rest, "mix.left.q")) return mat(w.w_in, 0, lq, W);
    if (!strcmp(rest, "mix.left.k")) return mat(w.w_in, lq, lk, W);
    if (!strcmp(rest, "mix.left.v")) return mat(w.w_in, lq + lk, lv, W);
    if (!strcmp(rest, "mix.left.o")) return mat(w.w_o, 0, W, lvd);
    if (!strcmp(rest, "mix.right.q")) return mat(w.w_in, r0, rGD, W);
    if (!strcmp(rest, "mix.right.k")) return mat(w.w_in, r0 + rGD, rGD, W);
    if (!strcmp(rest, "mix.right.v")) return mat(w.w_in, r0 + 2 * rGD, rvd, W);
    if (!strcmp(rest, "mix.right.b")) return mat(w.w_in, r0 + 2 * rGD + rvd, rH, W);
    if (!strcmp(rest, "mix.right.a")) return mat(w.w_in, r0 + 2 * rGD + rvd + rH, rH, W);
    if (!strcmp(rest, "mix.right.g")) return mat(w.w_in, r0 + 2 * rGD + rvd + 2 * rH, rvd, W);
    if (!strcmp(rest, "mix.right.o")) return mat(w.w_o2, 0, W, rvd);
    if (!strcmp(rest, "mix.right.q.conv")) return vec(w.conv_w, rGD, l.conv_taps);
    if (!strcmp(rest, "mix.right.k.conv")) return vec(w.conv_w + (size_t)rGD * l.conv_taps, rGD, l.conv_taps);
    if (!strcmp(rest, "mix.right.v.conv")) return vec(w.conv_w + (size_t)2 * rGD * l.conv_taps, rvd, l.conv_taps);
    if (!strcmp(rest, "mix.right.A_log")) return vec(w.a_log, rH);
    if (!strcmp(rest, "mix.right.dt_bias")) return vec(w.dt_bias, rH);
    if (!strcmp(rest, "mix.right.norm")) return vec(w.head_w, l.d_vdim);
  }
  return set_err(c, TGX_ERR_NAME, "Unexpected key: %s", name);
}

}  // namespace

// ================================================================================================================================================
int stack_create(const tgx_stack_desc* desc, const tgx_layer_desc* layers, int device_ordinal, tgx_ctx** out_ctx) {
  if (!desc || !layers || !out_ctx) return set_err(nullptr, TGX_ERR_INVALID, "null argument");
  *out_ctx = nullptr;
  const tgx_stack_desc& d = *desc;
  if (d.family != TGX_FAMILY_ZAKUSUN && d.family != TGX_FAMILY_MODEPEL && d.family != TGX_FAMILY_VITUDRA && d.family != TGX_FAMILY_ZALUVIK) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "family %d is not a layered model", d.family);
  const bool sandwich = d.family == TGX_FAMILY_MODEPEL, joint = d.family == TGX_FAMILY_VITUDRA, affine = d.family == TGX_FAMILY_ZALUVIK;
  if (d.width <= 0 || d.layers <= 0 || d.vocab <= 0 || d.max_seqs <= 0 || d.max_ctx <= 0) return set_err(nullptr, TGX_ERR_INVALID, "non-positive model dimension");
  if (d.compute_dtype != TGX_BF16 && d.compute_dtype != TGX_F16 && d.compute_dtype != TGX_F32) return set_err(nullptr, TGX_ERR_INVALID, "unknown compute dtype %d", d.compute_dtype);
  if (affine) { const int rc = check_affine_desc(d, layers); if (rc) return rc; }
  if (!sandwich && !joint && !affine && (d.norm_groups < 1 || d.norm_groups > tgx::NORM_MAX_GROUPS || d.width % d.norm_groups)) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "norm groups %d: 1..%d, dividing the width", d.norm_groups, tgx::NORM_MAX_GROUPS);
  if (!sandwich && !joint && !affine && (d.canon_taps < 1 || d.canon_taps > tgx::CONV_MAX_TAPS)) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "convolution taps %d: 1..%d", d.canon_taps, tgx::CONV_MAX_TAPS);
  int page = d.page_tokens > 0 ? d.page_tokens : 64;
  if (page & (page - 1)) return set_err(nullptr, TGX_ERR_INVALID, "page_tokens %d is not a power of two", page);
  int first_mix = -1;
  for (int i = 0; i < d.layers && !affine; i++) {
    const tgx_layer_desc& l = layers[i];
    if (joint) {
      auto attention_ok = [&](const char*& why) {
        if (l.heads <= 0 || l.dim <= 0 || l.vdim <= 0 || l.kv_heads <= 0 || l.heads % l.kv_heads) { why = "head counts / sizes"; return false; }
        if (l.dim > 64 * tgx::GQA_MAX_RPL || l.vdim > 64 * tgx::GQA_MAX_RPL) { why = "head size beyond 256"; return false; }
        if (l.rot_dims < 0 || l.rot_dims > l.dim || (l.rot_dims & 1) || (l.rot_dims > 0 && !(l.rot_base > 0.f))) { why = "rotated dimensions"; return false; }
        if (l.mask_kind < 0 || l.mask_kind > 2 || (l.mask_kind != 0 && l.mask_size < 1)) { why = "mask"; return false; }
        if (l.q_temp_coef != 0.f && l.q_temp_every < 1) { why = "query temperature period"; return false; }
        return true;
      };
      const char* why = "";
      if (l.mixer == TGX_MIXER_ATTENTION) {
        if (!attention_ok(why)) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: attention: %s", i, why);
        if (l.kv_share) {
          const int j = l.kv_share - 1;
          if (j < 0 || j >= i || layers[j].mixer != TGX_MIXER_ATTENTION || layers[j].kv_share || layers[j].kv_heads != l.kv_heads || layers[j].dim != l.dim || layers[j].vdim != l.vdim)
            return set_err(nullptr, TGX_ERR_INVALID, "layer %d: reads the keys and values of layer %d, which must be an earlier attention layer with its own projections and the same key / value heads", i, j);
        }
      } else if (l.mixer == TGX_MIXER_WKV) {
        if (l.heads <= 0 || l.dim <= 0 || l.dim > 256 || l.decay_rank < 0) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: wkv: %d heads of %d (1 .. 256), decay rank %d", i, l.heads, l.dim, l.decay_rank);
      } else if (l.mixer == TGX_MIXER_PARALLEL) {
        if (!attention_ok(why) || l.kv_share) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: parallel, attention half: %s", i, l.kv_share ? "shared keys are not part of it" : why);
        if (l.d_heads <= 0 || l.d_kv_heads <= 0 || l.d_heads % l.d_kv_heads || l.d_dim <= 0 || l.d_dim > 256 || l.d_vdim <= 0 || l.conv_taps < 1 || l.conv_taps > tgx::DELTA_MAX_TAPS)
          return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: parallel, delta-rule half: %d heads over %d key heads of %d (1 .. 256) x %d, %d taps (1 .. %d)", i, l.d_heads, l.d_kv_heads, l.d_dim, l.d_vdim, l.conv_taps, tgx::DELTA_MAX_TAPS);
      } else return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: mixer %d is not part of this family (attention, wkv and parallel are)", i, l.mixer);
      if (l.mlp != TGX_MLP_NONE && l.mlp != TGX_MLP_DENSE) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: feed-forward kind %d is not implemented", i, l.mlp);
      if (l.mlp == TGX_MLP_DENSE && l.ff <= 0) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: ff %d", i, l.ff);
      continue;
    }
    if (sandwich) {
      if (l.mixer != TGX_MIXER_ATTENTION && l.mixer != TGX_MIXER_MLSTM) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: mixer %d is not part of this family (attention and mlstm are)", i, l.mixer);
      if (l.heads <= 0 || l.dim <= 0 || l.vdim <= 0) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: non-positive mixer size", i);
      if (l.mixer == TGX_MIXER_ATTENTION) {
        if (l.kv_heads <= 0 || l.heads % l.kv_heads) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: %d query heads over %d key / value heads", i, l.heads, l.kv_heads);
        if (l.dim > 64 * tgx::GQA_MAX_RPL || l.vdim > 64 * tgx::GQA_MAX_RPL) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: head sizes %d / %d > %d", i, l.dim, l.vdim, 64 * tgx::GQA_MAX_RPL);
        if (l.rot_dims < 0 || l.rot_dims > l.dim || (l.rot_dims & 1) || (l.rot_dims > 0 && !(l.rot_base > 0.f))) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: %d rotated dimensions of %d (base %g)", i, l.rot_dims, l.dim, l.rot_base);
        if (l.v_mix) {
          if (first_mix >= 0 && layers[first_mix].kv_heads * layers[first_mix].vdim != l.kv_heads * l.vdim)
            return set_err(nullptr, TGX_ERR_INVALID, "layer %d: value mixing needs the value size of layer %d (%d != %d)", i, first_mix, l.kv_heads * l.vdim, layers[first_mix].kv_heads * layers[first_mix].vdim);
          if (first_mix < 0) first_mix = i;
        }
      } else {
        if (l.dim > 512) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: mlstm key size %d > 512", i, l.dim);
        if (!(l.gate_cap > 0.f)) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: gate_cap %g", i, l.gate_cap);
      }
      if (l.mlp != TGX_MLP_NONE && l.mlp != TGX_MLP_MOE && l.mlp != TGX_MLP_DENSE) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: feed-forward kind %d is not implemented", i, l.mlp);
      if (l.mlp == TGX_MLP_DENSE && l.ff <= 0) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: ff %d", i, l.ff);
      if (l.mlp == TGX_MLP_MOE) {
        const int E = l.experts + l.identity;
        if (l.experts < 0 || l.identity < 0 || E <= 0 || E >= tgx::ROUTER_MAX_E || l.top <= 0 || l.top > E || l.top > tgx::ROUTER_MAX_TOP || (l.experts > 0 && l.ff <= 0) || l.shared_ff < 0)
          return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: experts %d + identity %d (< %d), top %d (<= %d), ff %d", i, l.experts, l.identity, tgx::ROUTER_MAX_E, l.top, tgx::ROUTER_MAX_TOP, l.ff);
        if (l.groups > 1 && (E % l.groups || l.groups_keep < 1 || l.groups_keep > l.groups || (long long)l.groups_keep * (E / l.groups) < l.top))
          return set_err(nullptr, TGX_ERR_INVALID, "layer %d: %d router outputs in %d groups, %d kept, top %d", i, E, l.groups, l.groups_keep, l.top);
      }
      continue;
    }
    if (l.mixer != TGX_MIXER_LATENT_ATTENTION) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: mixer %d is not implemented (latent_attention is)", i, l.mixer);
    if (l.heads <= 0 || l.dim <= 0 || l.vdim <= 0 || l.kv_rank <= 0) return set_err(nullptr, TGX_ERR_INVALID, "layer %d: non-positive mixer size", i);
    if (l.kv_rank > 64 * tgx::LAT_MAX_RPL) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: kv_rank %d > %d", i, l.kv_rank, 64 * tgx::LAT_MAX_RPL);
    if (l.mlp != TGX_MLP_NONE && l.mlp != TGX_MLP_MOE) return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: feed-forward kind %d is not implemented", i, l.mlp);
    if (l.mlp == TGX_MLP_MOE && (l.experts <= 0 || l.experts > tgx::ROUTER_MAX_E || l.top <= 0 || l.top > l.experts || l.top > tgx::ROUTER_MAX_TOP || l.ff <= 0))
      return set_err(nullptr, TGX_ERR_UNSUPPORTED, "layer %d: experts %d (<= %d), top %d (<= %d), ff %d", i, l.experts, tgx::ROUTER_MAX_E, l.top, tgx::ROUTER_MAX_TOP, l.ff);
  }
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0) return set_err(nullptr, TGX_ERR_DEVICE, "no HIP device visible (--device mi355x needs a GPU; there is no CPU fallback)");
  if (device_ordinal < 0 || device_ordinal >= ndev) return set_err(nullptr, TGX_ERR_INVALID, "device ordinal %d out of range [0,%d)", device_ordinal, ndev);

  tgx_ctx* c = new (std::nothrow) tgx_ctx();
  StackModel* sm = new (std::nothrow) StackModel();
  if (!c || !sm) { delete c; delete sm; return set_err(nullptr, TGX_ERR_NOMEM, "host allocation failed"); }
  *out_ctx = c;
  c->stack = sm;
  sm->d = d;
  sm->page = page; sm->page_shift = 0;
  while ((1 << sm->page_shift) < page) sm->page_shift++;
  // what the shared sampler / token rings read from the flat description
  c->d.family = d.family; c->d.hidden = d.width; c->d.layers = d.layers; c->d.vocab = d.vocab; c->d.max_ctx = d.max_ctx; c->d.max_batch = d.max_seqs;
  c->d.compute_dtype = d.compute_dtype; c->d.tied = sandwich || joint ? 0 : 1; c->d.norm_eps = d.norm_eps;      // (a layer-norm design multiplies by the embedding table)
  sm->sandwich = sandwich; sm->joint = joint; sm->affine = affine;
  c->device = device_ordinal;
  c->dt = d.compute_dtype == TGX_BF16 ? tgx::DT_BF16 : (d.compute_dtype == TGX_F16 ? tgx::DT_F16 : tgx::DT_F32);
  c->esz = d.compute_dtype == TGX_F32 ? 4 : 2;
  HIP_OK(c, hipSetDevice(device_ordinal));
  hipDeviceProp_t prop;
  HIP_OK(c, hipGetDeviceProperties(&prop, device_ordinal));
  c->num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  HIP_OK(c, hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));

  const size_t W = (size_t)d.width, es = c->esz;
  int rc;
  if ((rc = dev_alloc(c, &c->embed, (size_t)d.vocab * W * es)) || (rc = dev_alloc(c, &sm->final_norm, 2 * W))) return rc;      // (weight, and a bias where the norm has one)
  sm->missing.insert("embed"); sm->missing.insert("final.norm");
  sm->L.resize((size_t)d.layers);
  if (sandwich) return create_sandwich_layers(c, layers);
  if (joint) return create_joint_layers(c, layers);
  if (affine) return create_affine_layers(c, layers);
  for (int i = 0; i < d.layers; i++) {
    StackLayerW& w = sm->L[(size_t)i];
    w.d = layers[i];
    const tgx_layer_desc& l = w.d;
    const std::string p = "l" + std::to_string(i) + ".";
    const size_t H = (size_t)l.heads, qd = H * l.dim, R = (size_t)l.kv_rank, vd = H * l.vdim;
    if ((rc = dev_alloc(c, &w.norm1, W)) || (rc = dev_alloc(c, &w.dwa, (size_t)i + 2)) || (rc = dev_alloc(c, &w.w_in, (qd + R + vd) * W * es)) ||
        (rc = dev_alloc(c, &w.w_ukT, qd * R * es)) || (rc = dev_alloc(c, &w.w_uv, vd * R * es)) || (rc = dev_alloc(c, &w.w_o, W * vd * es)) ||
        (rc = dev_alloc(c, &w.lat_norm, R)) || (rc = dev_alloc(c, &w.sink, H))) return rc;
    for (const char* n : {"norm1", "dwa", "mix.q", "mix.dkv", "mix.dkv.norm", "mix.uk", "mix.uv", "mix.sink", "mix.g", "mix.o"}) sm->missing.insert(p + n);
    if ((rc = dev_alloc(c, &w.canon1, W * d.canon_taps))) return rc;      // (one tap: the filter still scales the sublayer's input)
    sm->missing.insert(p + "canon1");
    if (l.mlp == TGX_MLP_MOE) {
      const size_t E = (size_t)l.experts, F = (size_t)l.ff;
      if ((rc = dev_alloc(c, &w.norm2, W)) || (rc = dev_alloc(c, &w.w_gate, E * F * W * es)) || (rc = dev_alloc(c, &w.w_up, E * F * W * es)) ||
          (rc = dev_alloc(c, &w.w_down, E * W * F * es)) || (rc = dev_alloc(c, &w.w_router, E * W)) || (rc = dev_alloc(c, &w.b_router, E))) return rc;
      for (const char* n : {"norm2", "mlp.router", "mlp.router.b"}) sm->missing.insert(p + n);
      if ((rc = dev_alloc(c, &w.canon2, W * d.canon_taps))) return rc;
      sm->missing.insert(p + "canon2");
      for (int e = 0; e < l.experts; e++)
        for (const char* n : {".gate", ".up", ".down"}) sm->missing.insert(p + "mlp.e" + std::to_string(e) + n);
      sm->max_top = std::max(sm->max_top, l.top); sm->max_ff = std::max(sm->max_ff, l.ff); sm->max_E = std::max(sm->max_E, l.experts);
    }
    sm->max_in = std::max(sm->max_in, (int)(qd + R + vd)); sm->max_hr = std::max(sm->max_hr, (int)(H * R)); sm->max_hv = std::max(sm->max_hv, (int)vd);
    sm->max_rank = std::max(sm->max_rank, l.kv_rank);
  }
  return TGX_OK;
}

int stack_upload(tgx_ctx* c, const char* name, const void* host, const int64_t* shape, int nd, int src_dtype) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  const int64_t W = d.width;
  auto bad_shape = [&]() { return set_err(c, TGX_ERR_SHAPE, "shape not equal for tensor: %s", name); };
  auto is = [&](int64_t a, int64_t b) { return b < 0 ? (nd == 1 && shape[0] == a) : (nd == 2 && shape[0] == a && shape[1] == b); };
  const bool probe = nd < 0;      // name lookup only (include/tgx.h): every tensor this model knows is a parameter it needs
  auto done = [&](int rc) { if (!rc) sm->missing.erase(name); return rc; };
  if (src_dtype != TGX_BF16 && src_dtype != TGX_F32 && src_dtype != TGX_F16) return set_err(c, TGX_ERR_INVALID, "unknown source dtype %d", src_dtype);
  if (sm->sandwich) return upload_sandwich(c, name, host, shape, nd, src_dtype);
  if (sm->joint) return upload_joint(c, name, host, shape, nd, src_dtype);
  if (sm->affine) return upload_affine(c, name, host, shape, nd, src_dtype);
  if (!strcmp(name, "embed")) { if (probe) return TGX_ERR_SHAPE; if (!is(d.vocab, W)) return bad_shape(); return done(upload_param_ext(c, c->embed, host, d.vocab * W, src_dtype)); }
  if (!strcmp(name, "final.norm")) { if (probe) return TGX_ERR_SHAPE; if (!is(W, -1)) return bad_shape(); return done(upload_f32(c, sm->final_norm, host, W, src_dtype)); }
  int li = -1;
  char rest[128] = {0};
  if (sscanf(name, "l%d.%127s", &li, rest) != 2 || li < 0 || li >= d.layers) return set_err(c, TGX_ERR_NAME, "Unexpected key: %s", name);
  StackLayerW& w = sm->L[(size_t)li];
  const tgx_layer_desc& l = w.d;
  const int64_t H = l.heads, qd = H * l.dim, R = l.kv_rank, vd = H * l.vdim, E = l.experts, F = l.ff;
  struct F32Slot { const char* n; float* dst; int64_t a, b; };
  const F32Slot fs[] = {{"norm1", w.norm1, W, -1}, {"norm2", w.norm2, W, -1}, {"canon1", w.canon1, W, d.canon_taps}, {"canon2", w.canon2, W, d.canon_taps},
                        {"dwa", w.dwa, li + 2, -1}, {"mix.dkv.norm", w.lat_norm, R, -1}, {"mix.sink", w.sink, H, -1},
                        {"mlp.router", w.w_router, E, W}, {"mlp.router.b", w.b_router, E, -1}};
  for (const F32Slot& s : fs)
    if (!strcmp(rest, s.n)) {
      if (!s.dst) break;
      if (probe) return TGX_ERR_SHAPE;
      if (!is(s.a, s.b)) return bad_shape();
      return done(upload_f32(c, s.dst, host, s.b < 0 ? s.a : s.a * s.b, src_dtype));
    }
  struct MatSlot { const char* n; ebyte* dst; int64_t row0, rows, cols; };
  const MatSlot ms[] = {{"mix.q", w.w_in, 0, qd, W}, {"mix.dkv", w.w_in, qd, R, W}, {"mix.g", w.w_in, qd + R, vd, W}, {"mix.uv", w.w_uv, 0, vd, R}, {"mix.o", w.w_o, 0, W, vd}};
  for (const MatSlot& s : ms)
    if (!strcmp(rest, s.n)) {
      if (probe) return TGX_ERR_SHAPE;
      if (!is(s.rows, s.cols)) return bad_shape();
      return done(upload_param_ext(c, s.dst + (size_t)(s.row0 * s.cols) * c->esz, host, s.rows * s.cols, src_dtype));
    }
  if (!strcmp(rest, "mix.uk")) {      // [heads * dim][rank] -> per head [rank][dim]
    if (probe) return TGX_ERR_SHAPE;
    if (!is(qd, R)) return bad_shape();
    const size_t es = esize(src_dtype);
    std::vector<unsigned char> t((size_t)(qd * R) * es);
    const unsigned char* src = (const unsigned char*)host;
    for (int64_t h = 0; h < H; h++)
      for (int64_t dd = 0; dd < l.dim; dd++)
        for (int64_t r = 0; r < R; r++) memcpy(&t[(size_t)((h * R + r) * l.dim + dd) * es], src + (size_t)((h * l.dim + dd) * R + r) * es, es);
    return done(upload_param_ext(c, w.w_ukT, t.data(), qd * R, src_dtype));
  }
  int e = -1;
  char leaf[32] = {0};
  if (l.mlp == TGX_MLP_MOE && sscanf(rest, "mlp.e%d.%31s", &e, leaf) == 2 && e >= 0 && e < E) {
    if (probe) return TGX_ERR_SHAPE;
    if (!strcmp(leaf, "gate") || !strcmp(leaf, "up")) {
      if (!is(F, W)) return bad_shape();
      return done(upload_param_ext(c, (leaf[0] == 'g' ? w.w_gate : w.w_up) + (size_t)(e * F * W) * c->esz, host, F * W, src_dtype));
    }
    if (!strcmp(leaf, "down")) {
      if (!is(W, F)) return bad_shape();
      return done(upload_param_ext(c, w.w_down + (size_t)(e * W * F) * c->esz, host, W * F, src_dtype));
    }
  }
  return set_err(c, TGX_ERR_NAME, "Unexpected key: %s", name);
}

int stack_finalize(tgx_ctx* c) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  if (!sm->missing.empty()) return set_err(c, TGX_ERR_STATE, "Missing key: %s", sm->missing.begin()->c_str());
  if (c->finalized) return TGX_OK;
  HIP_OK(c, hipSetDevice(c->device));
  const size_t W = (size_t)d.width, B = (size_t)d.max_seqs, V = (size_t)d.vocab;
  int rc;
  // angles of the position vector: pos * base^(-2i / width), the factor rounded to fp32 once
  if (!sm->sandwich && !sm->joint && !sm->affine) {
    std::vector<float> fq(W / 2 + 1);
    for (size_t i = 0; i < fq.size(); i++) fq[i] = (float)pow(10000.0, -2.0 * (double)i / (double)W);
    if ((rc = dev_alloc(c, &sm->freq, fq.size()))) return rc;
    HIP_OK(c, hipMemcpy(sm->freq, fq.data(), fq.size() * 4, hipMemcpyHostToDevice));
  }
  // the latent pool and its page tables
  const long long budget = d.budget_tokens > 0 ? d.budget_tokens : (long long)d.max_seqs * d.max_ctx;
  sm->n_pages = (int)((budget + sm->page - 1) / sm->page);
  sm->tbl_stride = (d.max_ctx + sm->page - 1) / sm->page;
  if ((rc = dev_alloc(c, &sm->tbl_dev, B * (size_t)sm->tbl_stride))) return rc;
  HIP_OK(c, hipMemset(sm->tbl_dev, 0, B * (size_t)sm->tbl_stride * 4));
  HIP_OK(c, hipHostMalloc((void**)&sm->tbl_host, B * (size_t)sm->tbl_stride * 4, hipHostMallocDefault));
  memset(sm->tbl_host, 0, B * (size_t)sm->tbl_stride * 4);
  sm->row_pages.assign(B, 0); sm->row_par.assign(B, 0); sm->row_dirty.assign(B, 0);
  for (int p = sm->n_pages - 1; p >= 0; p--) sm->free_pages.push_back(p);
  const size_t nb = sm->sandwich || sm->joint || sm->affine ? 0 : (size_t)d.canon_taps - 1;
  for (auto& r : sm->rot) {      // angle of (position, pair i) = position * base^(-2i / dims), evaluated in double, stored as fp32 cosine and sine
    const size_t half = (size_t)r.dims / 2;
    std::vector<float> cs((size_t)d.max_ctx * half * 2);
    for (size_t i = 0; i < half; i++) {
      const double f = pow((double)r.base, -2.0 * (double)i / (double)r.dims) / (double)r.factor;
      for (size_t p = 0; p < (size_t)d.max_ctx; p++) { cs[(p * half + i) * 2] = (float)cos((double)p * f); cs[(p * half + i) * 2 + 1] = (float)sin((double)p * f); }
    }
    if ((rc = dev_alloc(c, &r.cs, cs.size()))) return rc;
    HIP_OK(c, hipMemcpy(r.cs, cs.data(), cs.size() * 4, hipMemcpyHostToDevice));
  }
  for (auto& run : sm->runs) {      // layer-norm designs: every run of a layer has its own cache
    const tgx_layer_desc& l = sm->L[(size_t)run.layer].d;
    const size_t rows = (size_t)sm->n_pages * sm->page;
    if (l.mixer == TGX_MIXER_ATTENTION) {
      const size_t ke = rows * (size_t)l.kv_heads * l.dim * c->esz, ve = rows * (size_t)l.kv_heads * l.vdim * c->esz;
      if ((rc = dev_alloc(c, &run.pool, ke)) || (rc = dev_alloc(c, &run.poolV, ve))) return rc;
      HIP_OK(c, hipMemset(run.pool, 0, ke));
      HIP_OK(c, hipMemset(run.poolV, 0, ve));
      if (layer_mix_mfma(c, l)) {
        if ((rc = dev_alloc(c, &run.poolT, ve))) return rc;
        HIP_OK(c, hipMemset(run.poolT, 0, ve));
      }
    } else {
      const size_t pe = rows * (size_t)(l.kv_rank + l.rot_dim) * c->esz;
      if ((rc = dev_alloc(c, &run.pool, pe))) return rc;
      HIP_OK(c, hipMemset(run.pool, 0, pe));
      tgx_layer_desc row = l; row.kv_rank = l.kv_rank + l.rot_dim;      // the matrix-core kernel sees the cached row, latent and rotated part, as one latent
      if (layer_attn_mfma(c, row)) {
        if ((rc = dev_alloc(c, &run.poolT, pe))) return rc;
        HIP_OK(c, hipMemset(run.poolT, 0, pe));
      }
    }
  }
  for (auto& w : sm->L) {
    if (sm->affine) break;
    if (sm->joint) {
      const tgx_layer_desc& l = w.d;
      if (l.mixer != TGX_MIXER_WKV && w.kv_src < 0) {      // keys and values of an attention layer / a parallel mixer's attention half (a sharing layer borrows below)
        const size_t ke = (size_t)sm->n_pages * sm->page * (size_t)l.kv_heads * l.dim * c->esz, ve = (size_t)sm->n_pages * sm->page * (size_t)l.kv_heads * l.vdim * c->esz;
        if ((rc = dev_alloc(c, &w.pool, ke)) || (rc = dev_alloc(c, &w.poolV, ve))) return rc;
        HIP_OK(c, hipMemset(w.pool, 0, ke));
        HIP_OK(c, hipMemset(w.poolV, 0, ve));
        // every layer that reads this pool must be able to take the matrix-core kernel's query rows (their strides differ)
        bool mfma = true;
        for (auto& r : sm->L) {
          if (&r != &w && !(r.kv_src >= 0 && &sm->L[(size_t)r.kv_src] == &w)) continue;
          const tgx_layer_desc& q = r.d;
          long long ldq = (long long)q.heads * q.dim + (r.kv_src >= 0 ? 0 : (long long)q.kv_heads * (q.dim + q.vdim));
          if (q.mixer == TGX_MIXER_PARALLEL) ldq += 2LL * q.d_kv_heads * q.d_dim + 2LL * q.d_heads * q.d_vdim + 2LL * q.d_heads;
          mfma = mfma && gqa_mfma_shapes_ok(c->dt, q.dim, q.vdim, sm->page_shift, ldq);
        }
        if (mfma) {
          if ((rc = dev_alloc(c, &w.poolVT, ve))) return rc;
          HIP_OK(c, hipMemset(w.poolVT, 0, ve));
        }
      }
      if (l.mixer == TGX_MIXER_WKV) {
        const size_t se = B * (size_t)l.heads * l.dim * l.dim;
        if ((rc = dev_alloc(c, &w.mS, se)) || (rc = dev_alloc(c, &w.shift, 2 * B * W))) return rc;
        HIP_OK(c, hipMemset(w.mS, 0, se * 4));
        HIP_OK(c, hipMemset(w.shift, 0, 2 * B * W * 4));
        if (l.decay_rank <= 0) return set_err(c, TGX_ERR_STATE, "a wkv layer's decay product has no inner size");
      } else if (l.mixer == TGX_MIXER_PARALLEL) {
        const size_t se = B * (size_t)l.d_heads * l.d_dim * l.d_vdim, rC = 2 * (size_t)l.d_kv_heads * l.d_dim + (size_t)l.d_heads * l.d_vdim, ce = 2 * B * (size_t)(l.conv_taps - 1) * rC;
        if ((rc = dev_alloc(c, &w.mS, se))) return rc;
        HIP_OK(c, hipMemset(w.mS, 0, se * 4));
        if (ce > 0) {
          if ((rc = dev_alloc(c, &w.conv_state, ce))) return rc;
          HIP_OK(c, hipMemset(w.conv_state, 0, ce * 4));
        }
      }
      continue;
    }
    if (sm->sandwich) {
      if (w.d.mixer == TGX_MIXER_ATTENTION) {      // keys and values of the layer, one page table for both
        const size_t ke = (size_t)sm->n_pages * sm->page * (size_t)w.d.kv_heads * w.d.dim * c->esz, ve = (size_t)sm->n_pages * sm->page * (size_t)w.d.kv_heads * w.d.vdim * c->esz;
        if ((rc = dev_alloc(c, &w.pool, ke)) || (rc = dev_alloc(c, &w.poolV, ve))) return rc;
        HIP_OK(c, hipMemset(w.pool, 0, ke));
        HIP_OK(c, hipMemset(w.poolV, 0, ve));
        const long long nin = (long long)w.d.heads * (w.d.dim + w.d.vdim) + (long long)w.d.kv_heads * (w.d.dim + w.d.vdim);
        if (gqa_mfma_shapes_ok(c->dt, w.d.dim, w.d.vdim, sm->page_shift, nin)) {
          if ((rc = dev_alloc(c, &w.poolVT, ve))) return rc;
          HIP_OK(c, hipMemset(w.poolVT, 0, ve));
        }
      } else {                                     // the recurrent state of every slot (a sequence's first token starts from zero whatever the slot held)
        const size_t hs = B * (size_t)w.d.heads;
        if ((rc = dev_alloc(c, &w.mS, hs * w.d.dim * w.d.vdim)) || (rc = dev_alloc(c, &w.mn, 2 * hs * w.d.dim)) || (rc = dev_alloc(c, &w.mm, 2 * hs))) return rc;
        HIP_OK(c, hipMemset(w.mS, 0, hs * w.d.dim * w.d.vdim * 4));
        HIP_OK(c, hipMemset(w.mn, 0, 2 * hs * w.d.dim * 4));
        HIP_OK(c, hipMemset(w.mm, 0, 2 * hs * 4));
      }
      continue;
    }
    const size_t pe = (size_t)sm->n_pages * sm->page * (size_t)w.d.kv_rank * c->esz;
    if ((rc = dev_alloc(c, &w.pool, pe))) return rc;
    HIP_OK(c, hipMemset(w.pool, 0, pe));
    if (layer_attn_mfma(c, w.d)) {
      if ((rc = dev_alloc(c, &w.poolT, pe))) return rc;
      HIP_OK(c, hipMemset(w.poolT, 0, pe));
    }
    if (nb > 0) {
      const size_t se = 4 * B * nb * W;
      if ((rc = dev_alloc(c, &w.conv_state, se))) return rc;
      HIP_OK(c, hipMemset(w.conv_state, 0, se * 4));
    }
  }
  for (auto& w : sm->L)      // layers that read another layer's keys and values borrow its pools
    if (w.kv_src >= 0) { const StackLayerW& o = sm->L[(size_t)w.kv_src]; w.pool = o.pool; w.poolV = o.poolV; w.poolVT = o.poolVT; }
  if ((rc = dev_alloc(c, &sm->moe_off, (size_t)sm->max_E + 2)) || (rc = dev_alloc(c, &sm->n_tiles, 1))) return rc;
  HIP_OK(c, hipEventCreateWithFlags(&sm->meta_ev, hipEventDisableTiming));
  // the rows of the shared sampler (logits, argmax partials, current token) and the token rings
  c->lm_grid = gemv_grid(c, (int)(V + 1) / 2, 1, c->tune[TGX_KERNEL_LMHEAD].bpc);
  c->rows.resize(B);
  if ((rc = dev_alloc(c, &c->slab_x, B * W)) || (rc = dev_alloc(c, &c->slab_logits, B * V)) || (rc = dev_alloc(c, &c->slab_probs, B * V)) ||
      (rc = dev_alloc(c, &c->slab_part_val, B * c->lm_grid)) || (rc = dev_alloc(c, &c->slab_part_idx, B * c->lm_grid)) || (rc = dev_alloc(c, &c->slab_tok, B)) ||
      (rc = dev_alloc(c, &c->slab_pos, B))) return rc;
  HIP_OK(c, hipMemset(c->slab_tok, 0, B * 4));
  HIP_OK(c, hipMemset(c->slab_pos, 0, B * 4));
  HIP_OK(c, hipMemset(c->slab_part_val, 0, B * c->lm_grid * 4));      // a slot that never held logits still rides through the sampler: it picks token 0
  HIP_OK(c, hipMemset(c->slab_part_idx, 0, B * c->lm_grid * 4));
  HIP_OK(c, hipMemset(c->slab_logits, 0, B * V * 4));
  for (size_t b = 0; b < B; b++) {
    RowState& r = c->rows[b];
    r.x = c->slab_x + b * W; r.logits = c->slab_logits + b * V; r.probs = c->slab_probs + b * V;
    r.part_val = c->slab_part_val + b * c->lm_grid; r.part_idx = c->slab_part_idx + b * c->lm_grid; r.tok = c->slab_tok + b; r.pos = c->slab_pos + b;
  }
  c->log_cap = d.max_ctx > 1024 ? d.max_ctx : 1024;
  if ((rc = dev_alloc(c, &c->step, 1)) || (rc = dev_alloc(c, &c->step_done, 1)) || (rc = dev_alloc(c, &c->seed_dev, 1)) || (rc = sampler_alloc(c)) ||
      (rc = dev_alloc(c, &c->tok_log, (size_t)c->log_cap * B))) return rc;
  HIP_OK(c, hipMemset(c->step, 0, 4));
  HIP_OK(c, hipMemset(c->step_done, 0, 4));
  HIP_OK(c, hipHostMalloc((void**)&c->host_ring, (size_t)HOST_RING * B * 4, hipHostMallocMapped));
  HIP_OK(c, hipHostGetDevicePointer((void**)&c->host_ring_dev, c->host_ring, 0));
  for (int i = 0; i < MAX_TICKET_EVENTS; i++) HIP_OK(c, hipEventCreateWithFlags(&c->ticket_ev[i], hipEventDisableTiming));
  c->past = 0;
  c->row_past.assign(B, 0); c->row_tok.assign(B, 0); c->row_idle.assign(B, 0);
  c->row_probs_cfg.resize(B); c->row_probs_ok.assign(B, 0);
  c->finalized = true;
  return TGX_OK;
}

void stack_destroy(tgx_ctx* c) {
  StackModel* sm = c->stack;
  if (!sm) return;
  auto fr = [](void* p) { if (p) (void)hipFree(p); };
  for (auto& w : sm->L) {
    if (w.kv_src >= 0) w.pool = w.poolV = w.poolVT = nullptr;      // borrowed
    fr(w.w_o2); fr(w.w_w1); fr(w.w_w2); fr(w.mu); fr(w.w0); fr(w.ubonus); fr(w.conv_w); fr(w.a_log); fr(w.dt_bias); fr(w.shift);
    fr(w.norm1); fr(w.norm2); fr(w.canon1); fr(w.canon2); fr(w.dwa); fr(w.w_in); fr(w.w_ukT); fr(w.w_uv); fr(w.w_o); fr(w.lat_norm); fr(w.sink);
    fr(w.w_gate); fr(w.w_up); fr(w.w_down); fr(w.w_router); fr(w.b_router); fr(w.pool); fr(w.poolT); fr(w.conv_state);
    fr(w.b_in); fr(w.poolV); fr(w.poolVT); fr(w.vmix); fr(w.head_w); fr(w.mS); fr(w.mn); fr(w.mm); fr(w.act); fr(w.ws_gate); fr(w.ws_up); fr(w.ws_down);
  }
  for (auto& r : sm->rot) fr(r.cs);
  for (auto& r : sm->runs) { fr(r.pool); fr(r.poolV); fr(r.poolT); }
  for (auto& w : sm->L) { fr(w.ln); fr(w.talk); fr(w.pb); }
  fr(sm->w_loop); fr(sm->xcat); fr(sm->qplanes);
  fr(sm->mixed); fr(sm->lora); fr(sm->rec_in);
  fr(sm->head); fr(sm->norm_g); fr(sm->a2); fr(sm->ytmp); fr(sm->ysh); fr(sm->sgw); fr(sm->vfirst); fr(sm->hs);
  fr(sm->final_norm); fr(sm->freq); fr(sm->tbl_dev); fr(sm->meta_dev); fr(sm->x); fr(sm->xs); fr(sm->a); fr(sm->proj); fr(sm->ql); fr(sm->lat); fr(sm->o); fr(sm->selw);
  fr(sm->yh); fr(sm->yd); fr(sm->xn); fr(sm->lg); fr(sm->part); fr(sm->zr); fr(sm->sel); fr(sm->moe_off); fr(sm->perm); fr(sm->ptok); fr(sm->tile_e); fr(sm->tile_m0); fr(sm->n_tiles);
  if (sm->tbl_host) (void)hipHostFree(sm->tbl_host);
  if (sm->meta_host) (void)hipHostFree(sm->meta_host);
  if (sm->meta_ev) (void)hipEventDestroy(sm->meta_ev);
  delete sm;
  c->stack = nullptr;
}

int stack_free_tokens(const tgx_ctx* c) { return (int)std::min<long long>(INT32_MAX, (long long)c->stack->free_pages.size() * c->stack->page); }

int stack_reset_row(tgx_ctx* c, int row) {
  StackModel* sm = c->stack;
  HIP_OK(c, hipStreamSynchronize(c->stream));      // nothing in flight reads the slot's pages or its table any more
  int& have = sm->row_pages[(size_t)row];
  for (int b = 0; b < have; b++) sm->free_pages.push_back(sm->tbl_host[(size_t)row * sm->tbl_stride + b]);
  have = 0;
  c->row_past[(size_t)row] = 0; c->row_tok[(size_t)row] = 0;
  c->row_idle[(size_t)row] = row < c->batch;
  while (c->batch > 0 && c->row_idle[(size_t)c->batch - 1]) { c->row_idle[(size_t)c->batch - 1] = 0; c->batch--; }      // trailing free slots leave the batch
  refresh_rows(c);
  return TGX_OK;
}

int stack_step(tgx_ctx* c, int S, const int32_t* rows, const int32_t* counts, const int64_t* ids, int n_want, const int32_t* want, float* out_logits) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  if (S < 1 || S > d.max_seqs || !rows || !counts || !ids || n_want < 0 || (n_want > 0 && (!want || !out_logits))) return set_err(c, TGX_ERR_INVALID, "step: bad argument");
  long long T = 0, need_pages = 0;
  int max_keys = 0, max_count = 0;
  std::vector<char> seen((size_t)d.max_seqs, 0);
  for (int e = 0; e < S; e++) {
    const int r = rows[e];
    if (r < 0 || r >= d.max_seqs || seen[(size_t)r]) return set_err(c, TGX_ERR_INVALID, "step: slot %d out of range [0,%d) or listed twice", r, d.max_seqs);
    seen[(size_t)r] = 1;
    if (counts[e] < 1) return set_err(c, TGX_ERR_INVALID, "step: entry %d brings no token", e);
    const long long after = c->row_past[(size_t)r] + counts[e];
    if (after > d.max_ctx) return set_err(c, TGX_ERR_CONTEXT, "context size exceeded: slot %d would hold %lld tokens (contextSize %d)", r, after, d.max_ctx);
    need_pages += std::max<long long>(0, (after + sm->page - 1) / sm->page - sm->row_pages[(size_t)r]);
    max_keys = std::max<int>(max_keys, (int)after);
    max_count = std::max<int>(max_count, counts[e]);
    T += counts[e];
  }
  if (T > (1 << 24)) return set_err(c, TGX_ERR_INVALID, "step: %lld tokens", T);
  for (long long i = 0; i < T; i++) if (ids[i] < 0 || ids[i] >= d.vocab) return set_err(c, TGX_ERR_INVALID, "token id out of range");
  for (int i = 0; i < n_want; i++) if (want[i] < 0 || want[i] >= T) return set_err(c, TGX_ERR_INVALID, "step: wanted index %d outside the step's %lld tokens", want[i], T);
  if (need_pages > (long long)sm->free_pages.size())
    return set_err(c, TGX_ERR_CONTEXT, "latent pool exhausted: the step needs %lld more pages of %d tokens, %zu free of %d", need_pages, sm->page, sm->free_pages.size(), sm->n_pages);
  HIP_OK(c, hipSetDevice(c->device));
  int rc;
  if ((rc = ensure_ws(c, (int)std::max<long long>(T, n_want)))) return rc;
  if ((rc = meta_host_free(c))) return rc;
  const MetaPtrs hp = meta_layout(sm->meta_host, (int)T, S, n_want), dp = meta_layout(sm->meta_dev, (int)T, S, n_want);
  std::vector<int> last_want((size_t)S, -1);
  int t = 0;
  for (int e = 0; e < S; e++) {
    const int r = rows[e];
    assign_pages(sm, r, c->row_past[(size_t)r] + counts[e]);
    hp.ent_row[e] = r; hp.ent_start[e] = t; hp.ent_count[e] = counts[e]; hp.ent_par[e] = sm->row_par[(size_t)r];
    for (int i = 0; i < counts[e]; i++, t++) {
      hp.tok_id[t] = (int)ids[t]; hp.tok_pos[t] = (int)c->row_past[(size_t)r] + i; hp.tok_ent[t] = e;
      hp.tok_row[t] = r; hp.tok_idx[t] = i; hp.tok_cnt[t] = counts[e]; hp.tok_par[t] = sm->row_par[(size_t)r];
    }
  }
  for (int i = 0; i < n_want; i++) {
    hp.want[i] = want[i]; hp.want_row[i] = 0;
    for (int e = 0; e < S; e++) if (want[i] == hp.ent_start[e] + counts[e] - 1) last_want[(size_t)e] = i;
  }
  if ((rc = push_tables(c)) || (rc = push_meta(c, hp.n))) return rc;
  if ((rc = run_layers(c, dp, (int)T, S, max_keys, max_count))) return rc;
  if (n_want > 0) {
    run_logits(c, dp.want, n_want, sm->lg, nullptr);
    HIP_OK(c, hipMemcpyAsync(out_logits, sm->lg, (size_t)n_want * d.vocab * 4, hipMemcpyDeviceToHost, c->stream));
  }
  for (int e = 0; e < S; e++) {
    const int r = rows[e];
    if (last_want[(size_t)e] >= 0) {      // the slot's current logits: what tgx_sample_row / tgx_read_logits see
      HIP_OK(c, hipMemcpyAsync(c->rows[(size_t)r].logits, sm->lg + (size_t)last_want[(size_t)e] * d.vocab, (size_t)d.vocab * 4, hipMemcpyDeviceToDevice, c->stream));
      launch_argmax_partials(c, c->rows[(size_t)r].logits, d.vocab, c->rows[(size_t)r].part_val, c->rows[(size_t)r].part_idx);
      c->have_logits = true;
    }
  }
  HIP_OK(c, hipGetLastError());
  HIP_OK(c, hipStreamSynchronize(c->stream));
  LAUNCH_OK(c);
  for (int e = 0; e < S; e++) {
    const int r = rows[e];
    c->row_past[(size_t)r] += counts[e];
    sm->row_par[(size_t)r] ^= 1;
    c->row_tok[(size_t)r] = 0; c->row_idle[(size_t)r] = 0;
    c->batch = std::max(c->batch, r + 1);
    if ((size_t)r < c->row_probs_ok.size()) c->row_probs_ok[(size_t)r] = 0;
  }
  for (int b = 0; b < c->batch; b++) if (!seen[(size_t)b] && c->row_past[(size_t)b] == 0 && !c->row_idle[(size_t)b]) c->row_idle[(size_t)b] = 1;      // slots below a newly admitted one that hold nothing
  refresh_rows(c);
  return TGX_OK;
}

// n decode steps of every live slot: its device-resident current token in, logits into its row, the shared sampler picks the next token
int stack_decode(tgx_ctx* c, const tgx_sampler_cfg& cfg, uint64_t seed, int n) {
  StackModel* sm = c->stack;
  const tgx_stack_desc& d = sm->d;
  if (n <= 0) return TGX_OK;
  std::vector<int> live;
  long long need_pages = 0;
  int max_keys = 0;
  for (int b = 0; b < c->batch; b++) {
    if (c->row_idle[(size_t)b]) continue;
    live.push_back(b);
    const long long after = c->row_past[(size_t)b] + n;
    need_pages += std::max<long long>(0, (after + sm->page - 1) / sm->page - sm->row_pages[(size_t)b]);
    max_keys = std::max<int>(max_keys, (int)c->row_past[(size_t)b]);
  }
  if (live.empty()) return set_err(c, TGX_ERR_STATE, "decode: every slot is retired");
  if (need_pages > (long long)sm->free_pages.size())
    return set_err(c, TGX_ERR_CONTEXT, "latent pool exhausted: %d decode steps need %lld more pages of %d tokens, %zu free", n, need_pages, sm->page, sm->free_pages.size());
  if (!is_greedy(&cfg) && (!c->seed_valid || c->seed_on_dev != (unsigned long long)seed)) {
    HIP_OK(c, hipStreamSynchronize(c->stream));
    const unsigned long long s = seed;
    HIP_OK(c, hipMemcpy(c->seed_dev, &s, 8, hipMemcpyHostToDevice));
    c->seed_on_dev = s; c->seed_valid = true;
  }
  const int S = (int)live.size();
  int rc;
  if ((rc = ensure_ws(c, S)) || (rc = meta_host_free(c))) return rc;
  const MetaPtrs hp = meta_layout(sm->meta_host, S, S, S), dp = meta_layout(sm->meta_dev, S, S, S);
  for (int e = 0; e < S; e++) {
    const int r = live[(size_t)e];
    assign_pages(sm, r, c->row_past[(size_t)r] + n);
    hp.ent_row[e] = r; hp.ent_start[e] = e; hp.ent_count[e] = 1; hp.ent_par[e] = sm->row_par[(size_t)r];
    hp.tok_id[e] = 0; hp.tok_pos[e] = (int)c->row_past[(size_t)r]; hp.tok_ent[e] = e; hp.want[e] = e; hp.want_row[e] = r;
    hp.tok_row[e] = r; hp.tok_idx[e] = 0; hp.tok_cnt[e] = 1; hp.tok_par[e] = sm->row_par[(size_t)r];
  }
  if ((rc = push_tables(c)) || (rc = push_meta(c, hp.n))) return rc;
  for (int b = 0; b < c->batch; b++) { c->row_probs_cfg[(size_t)b] = cfg; c->row_probs_ok[(size_t)b] = is_greedy(&cfg) ? 0 : 1; }
  c->have_probs = !is_greedy(&cfg);
  for (int s = 0; s < n; s++) {
    hipLaunchKernelGGL(tgx::stack_gather_tok_kernel, dim3((S + 63) / 64), dim3(64), 0, c->stream, dp.tok_id, dp.ent_row, c->slab_tok, S);
    if ((rc = run_layers(c, dp, S, S, max_keys + s + 1, 1))) return rc;
    run_logits(c, dp.want, S, c->slab_logits, dp.want_row);
    for (int r : live) launch_argmax_partials(c, c->rows[(size_t)r].logits, d.vocab, c->rows[(size_t)r].part_val, c->rows[(size_t)r].part_idx);
    launch_sample(c, 0, c->batch, cfg, /*advance_pos=*/true, /*log_step=*/true);
    hipLaunchKernelGGL(tgx::stack_advance_kernel, dim3((S + 63) / 64), dim3(64), 0, c->stream, dp.tok_pos, dp.ent_par, dp.tok_par, S);
    c->steps_issued++;
  }
  HIP_OK(c, hipGetLastError());
  for (int r : live) { c->row_past[(size_t)r] += n; if (n & 1) sm->row_par[(size_t)r] ^= 1; }
  refresh_rows(c);
  c->have_logits = true;
  return TGX_OK;
}

// the cached latents of (slot, layer) as fp32 [past][kv_rank] — test / diagnostic use
int stack_read_latent(tgx_ctx* c, int row, int layer, float* out) {
  StackModel* sm = c->stack;
  if (row < 0 || row >= sm->d.max_seqs || layer < 0 || layer >= sm->d.layers || !out) return set_err(c, TGX_ERR_INVALID, "read_kv: row / layer out of range");
  HIP_OK(c, hipStreamSynchronize(c->stream));
  const StackLayerW& w = sm->L[(size_t)layer];
  if ((sm->sandwich && w.d.mixer != TGX_MIXER_ATTENTION) || (sm->joint && !w.pool)) return set_err(c, TGX_ERR_UNSUPPORTED, "read_kv: layer %d caches no rows (its state is recurrent)", layer);
  const ebyte* pool = w.pool;
  size_t R = sm->sandwich || sm->joint ? (size_t)w.d.kv_heads * w.d.dim : (size_t)w.d.kv_rank;      // an attention layer's cached keys, all key heads of a token in a row
  if (sm->affine) {      // the cache of the layer's first run: an attention layer's keys, a latent layer's rows [latent | rotated key part]
    for (const StackRun& r : sm->runs) if (r.layer == layer) { pool = r.pool; break; }
    R = w.d.mixer == TGX_MIXER_ATTENTION ? (size_t)w.d.kv_heads * w.d.dim : (size_t)(w.d.kv_rank + w.d.rot_dim);
  }
  std::vector<unsigned char> buf(R * c->esz);
  for (int64_t t = 0; t < c->row_past[(size_t)row]; t++) {
    const size_t page = (size_t)sm->tbl_host[(size_t)row * sm->tbl_stride + (size_t)(t >> sm->page_shift)];
    HIP_OK(c, hipMemcpy(buf.data(), pool + ((page << sm->page_shift) + (size_t)(t & (sm->page - 1))) * R * c->esz, R * c->esz, hipMemcpyDeviceToHost));
    const std::vector<float> f = to_f32(buf.data(), (int64_t)R, c->d.compute_dtype);
    memcpy(out + (size_t)t * R, f.data(), R * 4);
  }
  return TGX_OK;
}

// HBM bytes one decoded token streams at context T: every matrix the step touches (the chosen experts only) and the cached latents
int64_t stack_bytes_per_token(const tgx_ctx* c, int64_t T) {
  const StackModel* sm = c->stack;
  const int64_t W = sm->d.width, es = (int64_t)c->esz;
  int64_t b = (int64_t)sm->d.vocab * W * es;
  if (sm->sandwich || sm->joint) b *= 2;      // embedding row aside, the head is a matrix of its own
  if (sm->affine) {      // per run of a layer: its matrices (the chosen experts only) and the rows of its cache inside the mask's span
    if (sm->w_loop) b += (int64_t)sm->d.loop_times * 2 * W * W * es;
    for (const StackRun& r : sm->runs) {
      const tgx_layer_desc& l = sm->L[(size_t)r.layer].d;
      const int64_t H = l.heads, vd = H * l.vdim, keys = l.mask_kind ? std::min<int64_t>(T, l.mask_size) : T;
      if (l.mixer == TGX_MIXER_ATTENTION) b += ((H * l.dim + (int64_t)l.kv_heads * (l.dim + l.vdim) + vd) * W + W * vd) * es + keys * l.kv_heads * (l.dim + l.vdim) * es;
      else b += ((H * (l.dim + l.rot_dim) + l.kv_rank + l.rot_dim + H) * W + (H * l.dim + vd) * l.kv_rank + W * vd) * es + keys * (l.kv_rank + l.rot_dim) * es;
      if (l.mlp == TGX_MLP_DENSE) b += 2 * (int64_t)l.ff * W * es;
      if (l.mlp == TGX_MLP_MOE) b += (int64_t)l.experts * W * 4 + (int64_t)l.top * 3 * l.ff * W * es + (int64_t)3 * l.shared_ff * W * es;
    }
    return b;
  }
  for (const auto& w : sm->L) {
    const tgx_layer_desc& l = w.d;
    const int64_t H = l.heads, qd = H * l.dim, R = l.kv_rank, vd = H * l.vdim;
    if (sm->joint) {      // an attention layer reads at most its mask's span of keys; a recurrent state is read and written
      const int64_t keys = l.mask_kind ? std::min<int64_t>(T, l.mask_size) : T, kvw = (int64_t)l.kv_heads * (l.dim + l.vdim);
      if (l.mixer == TGX_MIXER_ATTENTION) b += ((qd + (w.kv_src >= 0 ? 0 : kvw)) * W + W * vd) * es + keys * kvw * es;
      else if (l.mixer == TGX_MIXER_WKV) b += (5 * qd * W + (int64_t)l.decay_rank * (W + qd)) * es + 2 * qd * l.dim * 4;
      else {
        const int64_t rvd = (int64_t)l.d_heads * l.d_vdim, rgd = (int64_t)l.d_kv_heads * l.d_dim;
        b += ((qd + kvw + 2 * rgd + 2 * rvd + 2 * l.d_heads) * W + W * (vd + rvd)) * es + keys * kvw * es + 2 * rvd * l.d_dim * 4;
      }
      if (l.mlp == TGX_MLP_DENSE) b += 3 * (int64_t)l.ff * W * es;
      continue;
    }
    if (sm->sandwich) {
      if (l.mixer == TGX_MIXER_ATTENTION) b += ((qd + (int64_t)l.kv_heads * (l.dim + l.vdim) + vd) * W + W * vd) * es + T * l.kv_heads * (l.dim + l.vdim) * es;
      else b += ((2 * qd + 2 * vd + 2 * H) * W + W * vd) * es + 2 * H * (int64_t)l.dim * l.vdim * 4;      // the state is read and written
      if (l.mlp == TGX_MLP_DENSE) b += 2 * (int64_t)l.ff * W * es;
      if (l.mlp == TGX_MLP_MOE) b += (int64_t)(l.experts + l.identity + 1) * W * 4 + (int64_t)std::min(l.top, l.experts) * 3 * l.ff * W * es + (int64_t)3 * l.shared_ff * W * es;
      continue;
    }
    b += ((qd + R + vd) * W + qd * R + vd * R + W * vd) * es + T * R * es;
    if (l.mlp == TGX_MLP_MOE) b += (int64_t)l.experts * W * 4 + (int64_t)l.top * 3 * l.ff * W * es;
  }
  return b;
}
