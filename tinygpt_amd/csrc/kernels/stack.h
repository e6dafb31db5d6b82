// stack.h — the row-wise kernels of layered models (include/tgx.h tgx_stack_desc): every kernel works on the T tokens of one ragged engine step.
// A step's tokens are the concatenated entries of its batch; StepMeta says which sequence slot and position each token belongs to.
//   sinusoid_embed_kernel   embedding row + interleaved sin / cos position vector
//   norm_conv_kernel        grouped RMS norm, the sublayer's causal short convolution over the normed rows, and the slot's convolution state
//   latent_append_kernel    RMS norm of the down-projected latent and its store into the paged pool
//   latent_attn_kernel      queries (already multiplied into latent space) against the pool: softmax with a sink, output in latent space
//   latent_attn_kernel<.., SPLIT> + latent_attn_merge_kernel   the same with a sequence's keys divided between workgroups (few tokens, long contexts)
//   router_topk_kernel      bias, top-k and softmax over the chosen on the router's fp32 products (stack_gemm.h)
//   moe_plan_kernel         (token, choice) pairs grouped by expert: offsets, permutation, tile list of the grouped products
//   combine_depth_kernel    residual + weighted expert outputs, then the learned average over the embedding output and all layer results
//   final_norm_rows_kernel  grouped RMS norm of the rows whose logits are asked for
// All arithmetic here is fp32; reductions run in a fixed order.
#pragma once
#include "common.h"
#include "stack_meta.h"

namespace tgx {


// ---- x[t] = embed[id] + pe(pos): entry 2i = sin(pos * f_i), 2i + 1 = cos(pos * f_i); f (fp32) comes from the host.  Writes the stream and layer-result slot 0.
template <int DT>
__global__ __launch_bounds__(256) void sinusoid_embed_kernel(StepMeta m, const elem_t<DT>* embed, const float* freq, float* x, float* x0, int W) {
  const int t = blockIdx.x;
  const size_t id = (size_t)m.tok_id[t];
  const float p = (float)m.tok_pos[t];
  for (int c = threadIdx.x; c < W; c += 256) {
    const float ang = p * freq[c >> 1];
    const float pe = (c & 1) ? cosf(ang) : sinf(ang);
    const float v = elem_to_f32<DT>(embed[id * W + c]) + pe;
    x[(size_t)t * W + c] = v;
    x0[(size_t)t * W + c] = v;
  }
}

// ---- grouped RMS norm + input convolution.  One workgroup per token.  hn_r = x_r / rms_group(x_r) * w for the token and its taps - 1 predecessors
// (rows of this step where the entry holds them, the slot's state otherwise, zero before the sequence's start);
// out = hn_t + sum_j cw[:, j] * hn_(t - taps + 1 + j).  The state (the last taps - 1 normed rows of the slot) is double-buffered per slot: this
// step reads buffer `par` and writes buffer `par ^ 1`, so no workgroup can overwrite what another still reads.
constexpr int CONV_MAX_TAPS = 8, NORM_MAX_GROUPS = 64;
struct NormConvArgs {
  const float* x;        // [T][W]
  const float* nw;       // [W] norm weight
  const float* cw;       // [W][taps] convolution weight (nullptr: the norm alone)
  float* out;            // [T][W]
  float* state;          // [2][slots][taps - 1][W] for this layer and sublayer (nullptr when taps == 1)
  size_t state_buf;      // elements between the two buffers
  int W, groups, taps;
  float eps;
};
__global__ __launch_bounds__(256) void norm_conv_kernel(StepMeta m, NormConvArgs a) {
  __shared__ float s_rinv[CONV_MAX_TAPS][NORM_MAX_GROUPS];
  const int t = blockIdx.x, i = m.tok_idx[t], cnt = m.tok_cnt[t], pos = m.tok_pos[t];
  const int row = m.tok_row[t], par = m.tok_par[t];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int gw = a.W / a.groups, nb = a.taps - 1;
  // 1 / rms of every (row back, group) pair that lives in this step: one wave per pair, lanes over the group's channels
  for (int it = wv; it < a.taps * a.groups; it += 4) {
    const int d = it / a.groups, g = it - d * a.groups;
    if (d > i) continue;                                  // wave-uniform: that row comes from the state (already normed) or lies before the start
    const float* xr = a.x + (size_t)(t - d) * a.W + (size_t)g * gw;
    float ss = 0.f;
    if ((a.W & 3) == 0 && (gw & 3) == 0)
      for (int c = 4 * lane; c < gw; c += 256) { const f32x4 v = *reinterpret_cast<const f32x4*>(xr + c); ss = fmaf(v[0], v[0], ss); ss = fmaf(v[1], v[1], ss); ss = fmaf(v[2], v[2], ss); ss = fmaf(v[3], v[3], ss); }
    else
      for (int c = lane; c < gw; c += 64) ss = fmaf(xr[c], xr[c], ss);
    ss = wave_sum(ss);
    if (lane == 0) s_rinv[d][g] = 1.0f / sqrtf(ss / (float)gw + a.eps);
  }
  __syncthreads();
  // (the two state buffers, the stream and the output never overlap: without the qualifiers every state store would order the loads behind it)
  const float* __restrict__ st_old = a.state ? a.state + (size_t)par * a.state_buf + (size_t)row * nb * a.W : nullptr;
  float* __restrict__ st_new = a.state ? a.state + (size_t)(par ^ 1) * a.state_buf + (size_t)row * nb * a.W : nullptr;
  const float* __restrict__ xin = a.x;
  float* __restrict__ outp = a.out;
  // channel c of the token: the normed row, the filter over it and its predecessors, the new state
  auto channel = [&](int c, float xv, float w, const float* cw) -> float {
    const int g = c / gw;
    const float h0 = xv * s_rinv[0][g] * w;
    float acc = h0;
    if (cw) {
      acc = fmaf(cw[nb], h0, acc);
      for (int d = 1; d <= nb; d++) {                      // the row d steps back
        float hv = 0.f;
        if (d <= i) hv = xin[(size_t)(t - d) * a.W + c] * s_rinv[d][g] * w;
        else if (pos - d >= 0) hv = st_old[(size_t)(nb - (d - i)) * a.W + c];       // state slot s holds position past - nb + s, past = pos - i
        acc = fmaf(cw[nb - d], hv, acc);
      }
      // the slot's new state = the last nb normed rows after this step: row i of cnt lands in slot nb - (cnt - i) ...
      const int s = nb - (cnt - i);
      if (s >= 0) st_new[(size_t)s * a.W + c] = h0;
      // ... and an entry shorter than the state keeps the tail of the old one (written by the entry's first token)
      if (i == 0)
        for (int k = 0; k + cnt < nb; k++) st_new[(size_t)k * a.W + c] = (pos - (nb - cnt - k) >= 0) ? st_old[(size_t)(k + cnt) * a.W + c] : 0.f;
    }
    return acc;
  };
  if ((a.W & 3) == 0 && (gw & 3) == 0) {
    // four channels per thread.  Every load is issued unconditionally (where the row back comes from — this step, the state, nowhere — is uniform over the
    // workgroup and only selects the address): one memory round trip instead of one per tap
#pragma unroll 2
    for (int c = 4 * threadIdx.x; c < a.W; c += 1024) {
      const int g = c / gw;
      const f32x4 xv = *reinterpret_cast<const f32x4*>(xin + (size_t)t * a.W + c), wv4 = *reinterpret_cast<const f32x4*>(a.nw + c);
      f32x4 hv[CONV_MAX_TAPS];
      float cwv[4][CONV_MAX_TAPS];
#pragma unroll
      for (int d = 1; d < CONV_MAX_TAPS; d++) {
        if (d > nb) continue;
        const bool inrow = d <= i, ok = inrow || pos - d >= 0;
        const float* p = inrow ? xin + (size_t)(t - d) * a.W + c : (ok ? st_old + (size_t)(nb - (d - i)) * a.W + c : xin + (size_t)t * a.W + c);
        const f32x4 v = *reinterpret_cast<const f32x4*>(p);
        const float sc = inrow ? s_rinv[d][g] : (ok ? 1.f : 0.f);
#pragma unroll
        for (int k = 0; k < 4; k++) hv[d][k] = inrow ? v[k] * sc * wv4[k] : v[k] * sc;
      }
      if (a.cw) {
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
          for (int j = 0; j < CONV_MAX_TAPS; j++) cwv[k][j] = j < a.taps ? a.cw[(size_t)(c + k) * a.taps + j] : 0.f;
      }
      f32x4 o;
#pragma unroll
      for (int k = 0; k < 4; k++) { hv[0][k] = xv[k] * s_rinv[0][g] * wv4[k]; o[k] = hv[0][k]; }
      if (a.cw) {
#pragma unroll
        for (int d = 0; d < CONV_MAX_TAPS; d++) {
          if (d > nb) continue;
#pragma unroll
          for (int k = 0; k < 4; k++) {
            float wsel = 0.f;                                // filter tap nb - d of channel c + k
#pragma unroll
            for (int j = 0; j < CONV_MAX_TAPS; j++) wsel = (j == nb - d) ? cwv[k][j] : wsel;
            o[k] = fmaf(wsel, hv[d][k], o[k]);
          }
        }
        const int sl = nb - (cnt - i);
        if (sl >= 0) *reinterpret_cast<f32x4*>(st_new + (size_t)sl * a.W + c) = hv[0];
        if (i == 0) {
#pragma unroll
          for (int d = 1; d < CONV_MAX_TAPS; d++) {          // an entry shorter than the state keeps the tail of the old one: old row d back -> slot nb - cnt - d
            if (d > nb) continue;
            const int kk = nb - cnt - d;
            if (kk >= 0) *reinterpret_cast<f32x4*>(st_new + (size_t)kk * a.W + c) = hv[d];
          }
        }
      }
      *reinterpret_cast<f32x4*>(outp + (size_t)t * a.W + c) = o;
    }
  } else {
    for (int c = threadIdx.x; c < a.W; c += 256) outp[(size_t)t * a.W + c] = channel(c, xin[(size_t)t * a.W + c], a.nw[c], a.cw ? a.cw + (size_t)c * a.taps : nullptr);
  }
}

// ---- latent: c = rms_norm(down-projected row) * w, stored at the token's place in the pool (storage dtype).  One wave per token.
struct LatentAppendArgs {
  const float* src; long long lds; int col0;     // the projection output [T][lds], latent columns from col0
  const float* nw;                               // [rank]
  void* pool;                                    // [pages][page][rank]
  void* poolT;                                   // [pages][rank][page]: the same latents, token-contiguous per channel (nullptr: not kept)
  int rank; float eps;
  // a rotated key part all heads share (rot_dim > 0): the rot_dim columns behind the latent, not normed, turned by the token's position (rotate-half
  // pairing over the first rot_dims of them, cosine / sine from a host-made table), are stored behind the normed latent: a pool row is [rank + rot_dim].
  // The rotated part of every head's query (q columns [h * qstride + qoff, + rot_dim)) is turned the same way, multiplied by qscale and written behind
  // the head's latent-space query: ql[t][h * (rank + rot_dim) + rank + i]
  int rot_dim, rot_dims; const float* cs;        // cs [positions][rot_dims / 2][2]
  const float* q; int heads, qstride, qoff; float qscale;
  float* ql;
};
template <int DT>
__global__ __launch_bounds__(256) void latent_append_kernel(StepMeta m, LatentAppendArgs a) {
  // one wave, or several (each sums the squares for itself, the stores are dealt to all threads)
  const int t = blockIdx.x, lane = threadIdx.x & 63, pos = m.tok_pos[t], nth = blockDim.x;
  const float* s = a.src + (size_t)t * a.lds + a.col0;
  float ss = 0.f;
  for (int c = lane; c < a.rank; c += 64) ss = fmaf(s[c], s[c], ss);
  ss = wave_sum(ss);
  const float rinv = 1.0f / sqrtf(ss / (float)a.rank + a.eps);
  const int page = m.tbl[(size_t)m.tok_row[t] * m.tbl_stride + (pos >> m.page_shift)];
  const int row_w = a.rank + a.rot_dim;
  elem_t<DT>* dst = reinterpret_cast<elem_t<DT>*>(a.pool) + (((size_t)page << m.page_shift) + (size_t)(pos & ((1 << m.page_shift) - 1))) * row_w;
  elem_t<DT>* dstT = a.poolT ? reinterpret_cast<elem_t<DT>*>(a.poolT) + (((size_t)page * row_w) << m.page_shift) + (size_t)(pos & ((1 << m.page_shift) - 1)) : nullptr;
  for (int c = threadIdx.x; c < a.rank; c += nth) {
    const elem_t<DT> v = f32_to_elem<DT>(s[c] * rinv * a.nw[c]);
    dst[c] = v;
    if (dstT) dstT[(size_t)c << m.page_shift] = v;
  }
  if (a.rot_dim <= 0) return;
  const int half = a.rot_dims >> 1;
  // vector 0 is the shared key part, vectors 1 .. heads the queries' rotated parts; element i of a vector: a rotated pair member or a channel that passes
  for (int i = threadIdx.x; i < (a.heads + 1) * a.rot_dim; i += nth) {
    const int vec = i / a.rot_dim, ch = i - vec * a.rot_dim;
    const float* src = vec == 0 ? s + a.rank : a.q + (size_t)t * a.lds + (size_t)(vec - 1) * a.qstride + a.qoff;
    float v = src[ch];
    if (ch < 2 * half) {
      const int pr = ch < half ? ch : ch - half;
      const float c = a.cs[((size_t)pos * half + pr) * 2], sn = a.cs[((size_t)pos * half + pr) * 2 + 1];
      v = ch < half ? __fsub_rn(__fmul_rn(v, c), __fmul_rn(src[ch + half], sn)) : __fadd_rn(__fmul_rn(v, c), __fmul_rn(src[ch - half], sn));
    }
    if (vec == 0) {
      const elem_t<DT> e = f32_to_elem<DT>(v);
      dst[a.rank + ch] = e;
      if (dstT) dstT[(size_t)(a.rank + ch) << m.page_shift] = e;
    } else a.ql[(size_t)t * a.heads * row_w + (size_t)(vec - 1) * row_w + a.rank + ch] = v * a.qscale;
  }
}

// ---- latent attention, one workgroup per (token, head): the four waves take every fourth key, lanes hold rank / 64 latent channels each.
// Scores are fp32 dot products of the latent-space query (score scale folded in) with the cached latents; the softmax denominator also holds
// exp(sink[head]) — a term without key or value that counts once.  The output stays in latent space (the value up-projection follows as a product).
constexpr int LAT_MAX_RPL = 32;       // latent channels per lane: rank <= 2048
struct LatentAttnArgs {
  const float* q; long long ldq;      // [T][heads * rank]
  const void* pool;
  const float* sink;                  // [heads] (nullptr: the softmax has no sink)
  float* out; long long ldo;          // [T][heads * rank]
  int rank, heads;
  int mask_kind, mask_size;           // MASK_*: the query at position i sees the keys [first_key(i), i] (stack_meta.h)
  // split form: keys [split * keys_per, ...) of every token's range; partial records (m, l, acc[rank]) per (token, head, split)
  float* part; int nsplit, keys_per;
};
template <int DT, int RPL>
__device__ __forceinline__ void latent_scan(const StepMeta& m, const LatentAttnArgs& a, int row, int j0, int j1, int jstep, const float* qv, float& mx, float& l, float* acc) {
  const int lane = threadIdx.x & 63;
  const elem_t<DT>* pool = reinterpret_cast<const elem_t<DT>*>(a.pool);
  const int pmask = (1 << m.page_shift) - 1;
  for (int j = j0; j < j1; j += jstep) {
    const int page = m.tbl[(size_t)row * m.tbl_stride + (j >> m.page_shift)];
    const elem_t<DT>* cr = pool + (((size_t)page << m.page_shift) + (size_t)(j & pmask)) * a.rank;
    float cv[RPL];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < RPL; k++) {
      const int c = lane + 64 * k;
      cv[k] = c < a.rank ? elem_to_f32<DT>(cr[c]) : 0.f;
      s = fmaf(qv[k], cv[k], s);
    }
    s = wave_sum(s);
    const float mn = fmaxf(mx, s);
    const float corr = expf(mx - mn), p = expf(s - mn);      // mx = -inf on a wave's first key: corr = 0
    l = fmaf(l, corr, p);
#pragma unroll
    for (int k = 0; k < RPL; k++) acc[k] = fmaf(acc[k], corr, p * cv[k]);
    mx = mn;
  }
}
template <int DT, int RPL, bool SPLIT>
__global__ __launch_bounds__(256) void latent_attn_kernel(StepMeta m, LatentAttnArgs a) {
  __shared__ float s_m[4], s_l[4];
  extern __shared__ float s_acc[];      // [4][rank]
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int row = m.tok_row[t], nkeys = m.tok_pos[t] + 1;
  int k0 = first_key(nkeys - 1, a.mask_kind, a.mask_size), k1 = nkeys;
  if (SPLIT) { k0 = min(nkeys, k0 + (int)blockIdx.z * a.keys_per); k1 = min(nkeys, k0 + a.keys_per); }
  const float* q = a.q + (size_t)t * a.ldq + (size_t)h * a.rank;
  float qv[RPL], acc[RPL];
#pragma unroll
  for (int k = 0; k < RPL; k++) { const int c = lane + 64 * k; qv[k] = c < a.rank ? q[c] : 0.f; acc[k] = 0.f; }
  // the sink enters once: as the starting state of wave 0 (of split 0)
  const bool has_sink = a.sink && wv == 0 && (!SPLIT || blockIdx.z == 0);
  float mx = has_sink ? a.sink[h] : -INFINITY, l = has_sink ? 1.f : 0.f;
  latent_scan<DT, RPL>(m, a, row, k0 + wv, k1, 4, qv, mx, l, acc);
  if (lane == 0) { s_m[wv] = mx; s_l[wv] = l; }
#pragma unroll
  for (int k = 0; k < RPL; k++) { const int c = lane + 64 * k; if (c < a.rank) s_acc[wv * a.rank + c] = acc[k]; }
  __syncthreads();
  const float M = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
  float f[4], L = 0.f;
#pragma unroll
  for (int w = 0; w < 4; w++) { f[w] = s_m[w] == -INFINITY ? 0.f : expf(s_m[w] - M); L = fmaf(s_l[w], f[w], L); }
  if (SPLIT) {
    float* rec = a.part + (((size_t)t * a.heads + h) * a.nsplit + blockIdx.z) * (size_t)(a.rank + 2);
    if (threadIdx.x == 0) { rec[0] = M; rec[1] = L; }
    for (int c = threadIdx.x; c < a.rank; c += 256) rec[2 + c] = s_acc[c] * f[0] + s_acc[a.rank + c] * f[1] + s_acc[2 * a.rank + c] * f[2] + s_acc[3 * a.rank + c] * f[3];
  } else {
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    float* o = a.out + (size_t)t * a.ldo + (size_t)h * a.rank;
    for (int c = threadIdx.x; c < a.rank; c += 256) o[c] = (s_acc[c] * f[0] + s_acc[a.rank + c] * f[1] + s_acc[2 * a.rank + c] * f[2] + s_acc[3 * a.rank + c] * f[3]) * inv;
  }
}
// merges the split records of one (token, head) in split order
__global__ __launch_bounds__(256) void latent_attn_merge_kernel(LatentAttnArgs a) {
  __shared__ float s_f[64];
  __shared__ float s_inv;
  const int t = blockIdx.x, h = blockIdx.y;
  const size_t rs = (size_t)(a.rank + 2);
  const float* rec = a.part + ((size_t)t * a.heads + h) * a.nsplit * rs;
  if (threadIdx.x < 64) {      // one wave: every split's weight exp(m_s - M) and the merged denominator
    const int s = threadIdx.x;
    const float ms = s < a.nsplit ? rec[(size_t)s * rs] : -INFINITY;
    const float M = group_max<64>(ms);
    const float f = ms == -INFINITY ? 0.f : expf(ms - M);
    float lf = s < a.nsplit ? rec[(size_t)s * rs + 1] * f : 0.f;
    for (int o = 1; o < 64; o <<= 1) { const float other = __shfl_up(lf, o, 64); if (s >= o) lf += other; }      // prefix sums: lane 63 holds the total in split order
    s_f[s] = f;
    if (s == 63) s_inv = lf > 0.f ? 1.0f / lf : 0.f;
  }
  __syncthreads();
  const float inv = s_inv;
  float* o = a.out + (size_t)t * a.ldo + (size_t)h * a.rank;
  for (int c = threadIdx.x; c < a.rank; c += 256) {
    float v = 0.f;
    for (int s = 0; s < a.nsplit; s++) v = fmaf(rec[(size_t)s * rs + 2 + c], s_f[s], v);
    o[c] = v * inv;
  }
}

// ---- router: the `top` largest of z + b (z = Wr h, an fp32 product of fp32 weights; ties: the lower index), weights = softmax over them.  One wave per token.
struct RouterArgs {
  const float* z;        // [T][E] router products
  const float* br;       // [E]
  int* sel;              // [T][top]
  float* selw;           // [T][top]
  int E, top;
};
constexpr int ROUTER_MAX_E = 1024, ROUTER_MAX_TOP = 64;
__global__ __launch_bounds__(64) void router_topk_kernel(RouterArgs a) {
  __shared__ float s_z[ROUTER_MAX_E];
  __shared__ float s_v[ROUTER_MAX_TOP];
  __shared__ int s_i[ROUTER_MAX_TOP];
  const int t = blockIdx.x, lane = threadIdx.x;
  // every lane owns the logits e = lane, lane + 64, ...: it alone writes, reads and retires them, so the loop needs no barrier; the butterfly leaves each
  // pick in all lanes, lane 0 keeps the list
  for (int e = lane; e < a.E; e += 64) s_z[e] = a.z[(size_t)t * a.E + e] + a.br[e];
  for (int k = 0; k < a.top; k++) {
    float bv = -INFINITY; int bi = 0x7fffffff;
    for (int e = lane; e < a.E; e += 64) { const float v = s_z[e]; if (v > bv) { bv = v; bi = e; } }
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64); const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi < a.E && (bi & 63) == lane) s_z[bi] = -INFINITY;
    if (lane == 0) { s_v[k] = bv; s_i[k] = bi < a.E ? bi : 0; }
  }
  if (lane == 0) {
    const float mx = s_v[0];            // the first pick is the largest
    float den = 0.f;
    for (int k = 0; k < a.top; k++) den += expf(s_v[k] - mx);
    for (int k = 0; k < a.top; k++) { a.sel[(size_t)t * a.top + k] = s_i[k]; a.selw[(size_t)t * a.top + k] = expf(s_v[k] - mx) / den; }
  }
}

// ---- plan of the grouped expert products: pairs i = t * top + k grouped by expert.  One workgroup.
//   off[E + 1]   first grouped row of every expert;  perm[n]  the pair at grouped row n;  tok[n] = perm[n] / top (the row of the activations)
//   tiles: (expert, first row) of every tile of tile_m rows, n_tiles of them
struct MoePlanArgs {
  const int* sel; int n_pairs, E, top, tile_m;
  int *off, *perm, *tok, *tile_e, *tile_m0, *n_tiles;
  int E_tiles;               // tiles are made for the first E_tiles experts (0: all); the others' pairs need no product (identity outputs)
};
__global__ __launch_bounds__(1024) void moe_plan_kernel(MoePlanArgs a) {
  __shared__ int s_cnt[ROUTER_MAX_E], s_off[ROUTER_MAX_E + 1], s_cur[ROUTER_MAX_E];
  for (int e = threadIdx.x; e < a.E; e += 1024) { s_cnt[e] = 0; s_cur[e] = 0; }
  __syncthreads();
  for (int i = threadIdx.x; i < a.n_pairs; i += 1024) atomicAdd(&s_cnt[a.sel[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int o = 0, nt = 0;
    for (int e = 0; e < a.E; e++) {
      s_off[e] = o; a.off[e] = o;
      if (a.E_tiles <= 0 || e < a.E_tiles)
        for (int m0 = 0; m0 < s_cnt[e]; m0 += a.tile_m) { a.tile_e[nt] = e; a.tile_m0[nt] = o + m0; nt++; }
      o += s_cnt[e];
    }
    s_off[a.E] = o; a.off[a.E] = o;
    *a.n_tiles = nt;
  }
  __syncthreads();
  // rows of an expert in any order: every pair's result lands in its own output row, so the order changes no value
  for (int i = threadIdx.x; i < a.n_pairs; i += 1024) {
    const int e = a.sel[i];
    const int n = s_off[e] + atomicAdd(&s_cur[e], 1);
    a.perm[n] = i; a.tok[n] = i / a.top;
  }
}

// ---- x_new = x + sum_k y[t * top + k] (router weights already applied), stored as the layer's result X_(i+1); the stream handed on is
// sum_j dw[j] X_j over the embedding output and all results so far.
struct CombineDepthArgs {
  float* x;              // [T][W] in: the stream after the mixer; out: the next layer's input
  const float* y;        // [T * top][W] expert outputs (nullptr / top 0: no feed-forward)
  float* xs;             // [n_res][slot_stride] layer results; this layer writes slot n_res - 1
  size_t slot_stride;
  const float* dw;       // [n_res]
  int W, top, n_res;
};
__global__ __launch_bounds__(256) void combine_depth_kernel(CombineDepthArgs a) {
  const size_t t = blockIdx.x;
  if ((a.W & 3) == 0) {
    for (int c = 4 * threadIdx.x; c < a.W; c += 1024) {
      f32x4 v = *reinterpret_cast<const f32x4*>(a.x + t * a.W + c);
      for (int k = 0; k < a.top; k++) v += *reinterpret_cast<const f32x4*>(a.y + (t * a.top + k) * a.W + c);
      *reinterpret_cast<f32x4*>(a.xs + (size_t)(a.n_res - 1) * a.slot_stride + t * a.W + c) = v;
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
      for (int j = 0; j < a.n_res - 1; j++) {
        const f32x4 r = *reinterpret_cast<const f32x4*>(a.xs + (size_t)j * a.slot_stride + t * a.W + c);
        const float dj = a.dw[j];
#pragma unroll
        for (int k = 0; k < 4; k++) s[k] = fmaf(dj, r[k], s[k]);
      }
      const float dl = a.dw[a.n_res - 1];
#pragma unroll
      for (int k = 0; k < 4; k++) s[k] = fmaf(dl, v[k], s[k]);
      *reinterpret_cast<f32x4*>(a.x + t * a.W + c) = s;
    }
    return;
  }
  for (int c = threadIdx.x; c < a.W; c += 256) {
    float v = a.x[t * a.W + c];
    for (int k = 0; k < a.top; k++) v += a.y[(t * a.top + k) * a.W + c];
    a.xs[(size_t)(a.n_res - 1) * a.slot_stride + t * a.W + c] = v;
    float s = 0.f;
    for (int j = 0; j < a.n_res - 1; j++) s = fmaf(a.dw[j], a.xs[(size_t)j * a.slot_stride + t * a.W + c], s);
    a.x[t * a.W + c] = fmaf(a.dw[a.n_res - 1], v, s);
  }
}

// ---- out[i] = grouped RMS norm of x[rows[i]] * w
__global__ __launch_bounds__(256) void final_norm_rows_kernel(const float* x, const int* rows, const float* nw, float* out, int W, int groups, float eps) {
  __shared__ float s_rinv[NORM_MAX_GROUPS];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, gw = W / groups;
  const float* xr = x + (size_t)rows[blockIdx.x] * W;
  for (int g = wv; g < groups; g += 4) {
    float ss = 0.f;
    for (int c = lane; c < gw; c += 64) ss = fmaf(xr[(size_t)g * gw + c], xr[(size_t)g * gw + c], ss);
    ss = wave_sum(ss);
    if (lane == 0) s_rinv[g] = 1.0f / sqrtf(ss / (float)gw + eps);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < W; c += 256) out[(size_t)blockIdx.x * W + c] = xr[c] * s_rinv[c / gw] * nw[c];
}

// decode steps: the tokens come from the slots' device-resident current tokens, and positions advance on the device
__global__ void stack_gather_tok_kernel(int* tok_id, const int* ent_row, const int* slab_tok, int S) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < S) tok_id[i] = slab_tok[ent_row[i]];
}
__global__ void stack_advance_kernel(int* tok_pos, int* ent_par, int* tok_par, int S) {      // one token per entry: token i is entry i
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < S) { tok_pos[i] += 1; ent_par[i] ^= 1; tok_par[i] ^= 1; }
}

}  // namespace tgx
