// stack.h — host-side state of a layered model (include/tgx.h tgx_stack_desc): per-layer weights, the paged cache pool (latents, or keys and values)
// with its page tables, the slots' convolution / recurrent state and the workspace of one ragged step.  Owned by tgx_ctx::stack; the launch code
// lives in stack.hip.
#pragma once
#include <set>
#include <string>
#include <vector>

#include "ctx.h"

struct StackLayerW {
  tgx_layer_desc d{};
  float *norm1 = nullptr, *norm2 = nullptr, *canon1 = nullptr, *canon2 = nullptr, *dwa = nullptr;      // fp32
  // mixer (latent attention)
  ebyte* w_in = nullptr;        // [heads * dim | kv_rank | heads * vdim][width]: query, latent and gate projections in one product
  ebyte* w_ukT = nullptr;       // [heads][kv_rank][dim]: the key up-projection, transposed per head (queries are multiplied into latent space)
  ebyte* w_uv = nullptr;        // [heads * vdim][kv_rank]
  ebyte* w_o = nullptr;         // [width][heads * vdim]
  float *lat_norm = nullptr, *sink = nullptr;
  // feed-forward (mixture of experts)
  ebyte *w_gate = nullptr, *w_up = nullptr, *w_down = nullptr;      // [experts][ff][width] x 2, [experts][width][ff]
  float *w_router = nullptr, *b_router = nullptr;                   // fp32 [experts][width], [experts]
  ebyte* pool = nullptr;        // latent cache of this layer: [pages][page_tokens][kv_rank]
  ebyte* poolT = nullptr;       // ... and its transposed copy [pages][kv_rank][page_tokens] for the matrix-core attention (layers that take it)
  float* conv_state = nullptr;  // [2 sublayers][2 buffers][slots][taps - 1][width]
  // sandwich-norm designs: the four norm numbers of the layer live in StackModel::norm_g at 4 * layer (norm1, norm1b, norm2, norm2b)
  // grouped-query attention: w_in = [q | k | v | gate] rows, bias b_in over the same rows; mLSTM: w_in = [q | k | v | gate | zi | zf]
  float* b_in = nullptr;        // fp32 [rows of w_in]
  ebyte* poolV = nullptr;       // attention: values [pages][page_tokens][kv_heads * vdim] (`pool` holds the keys [..][kv_heads * dim])
  ebyte* poolVT = nullptr;      // ... and their transposed copy [pages][kv_heads * vdim][page_tokens] for the matrix-core attention (layers that take it)
  float* vmix = nullptr;        // attention: the value-mixing number
  int vmode = 0;                // 0: no value mixing, 1: the first mixing layer (its values are handed on), 2: mixes
  int rot = -1;                 // index of the layer's rotation table (StackModel::rot)
  float* head_w = nullptr;      // mLSTM: [heads * vdim] scale after the per-head norm
  float *mS = nullptr, *mn = nullptr, *mm = nullptr;      // mLSTM state: [slots][heads][dim][vdim], [2][slots][heads][dim], [2][slots][heads]
  // dense feed-forward: w_up [ff][width], w_down [width][ff] (the expert fields), act = PolyNorm's four numbers
  float* act = nullptr;
  // grouped-choice experts: w_router holds experts + identity rows and, with a shared expert, its gate row last; b_router is the correction
  ebyte *ws_gate = nullptr, *ws_up = nullptr, *ws_down = nullptr;      // shared expert
  // parallel-sublayer designs (Vitudra).  norm1 holds the layer's norm weight (its distance from one); the gated feed-forward uses w_gate / w_up / w_down.
  //   attention: w_in = [q | k | v] rows (q alone when the layer reads another layer's pool: kv_src, whose pool pointers it borrows)
  //   wkv:       w_in = [r | k | v | g] (one product batched over the four token-shift mixes), w_w1 / w_w2 / w0 the decay's low-rank product, mu the five
  //              mixing vectors, ubonus the current token's bonus, head_w the scale behind the per-head norm; mS the state, shift the slot's last row
  //   parallel:  w_in = [left q | k | v | right q | k | v | b | a | g], w_o the left and w_o2 the right output projection; conv_w the right half's filters,
  //              conv_state the tails of its raw projections, mS its state, head_w the weight all heads share
  int kv_src = -1;
  ebyte *w_o2 = nullptr, *w_w1 = nullptr, *w_w2 = nullptr;
  float *mu = nullptr, *w0 = nullptr, *ubonus = nullptr, *conv_w = nullptr, *a_log = nullptr, *dt_bias = nullptr;
  float* shift = nullptr;       // [2][slots][width]
  // layer-norm designs (Zaluvik).  ln holds the layer's eight norm vectors [norm1 w | b | norm1b w | b | norm2 w | b | norm2b w | b][width].
  //   attention:        w_in = [q | k | v | gate] rows (gate per output channel), talk the head-mixing matrix [heads][heads], pb the per-head score bias
  //   latent attention: w_in = [q (heads * (dim + rot_dim)) | latent + rotated key part (kv_rank + rot_dim) | gate (heads)], w_ukT / w_uv / lat_norm as above
  //   dense: w_up / w_down; experts: w_router (fp32), w_gate / w_up / w_down stacked, ws_* the shared expert
  // The caches of these layers belong to their RUNS (StackModel::runs): a layer inside the loop has one per pass.
  float *ln = nullptr, *talk = nullptr, *pb = nullptr;
};

// one run of a layer (layer-norm designs): which layer's weights, whether the loop's input product comes first, and the run's own cache
struct StackRun {
  int layer = 0;
  bool inject = false;          // x <- W_loop [x; x0] in front of this run (the first layer of a pass of the loop)
  ebyte* pool = nullptr;        // attention: keys [pages][page_tokens][kv_heads * dim]; latent attention: [pages][page_tokens][kv_rank + rot_dim]
  ebyte* poolV = nullptr;       // attention: values [pages][page_tokens][kv_heads * vdim]
  ebyte* poolT = nullptr;       // the transposed copy for the matrix-core kernels (runs that take them): a latent run's rows [pages][kv_rank + rot_dim][page_tokens],
                                // an attention run's values [pages][kv_heads * vdim][page_tokens]
};

struct RotTable { int dims; float base; float factor; float* cs; };      // cos / sin of (position, pair) [max_ctx][dims / 2][2], angle = position * base^(-2 pair / dims) / factor, made on the host in double precision

struct StackModel {
  tgx_stack_desc d{};
  std::vector<StackLayerW> L;
  std::set<std::string> missing;       // checkpoint names not uploaded yet
  float *final_norm = nullptr, *freq = nullptr;
  // what the family fixes (stack_create): the kind of norm and of layer wiring
  bool sandwich = false;               // scalar RMS norms before and after every sublayer, no convolutions, no depth average, no position vector, a separate head
  bool joint = false;                  // one offset-weight RMS norm per layer; mixer and feed-forward read it side by side; x += residual_mult * (their sum); a separate head
  bool affine = false;                 // layer norms (weight and bias) before and after every sublayer, x += residual_mult * norm(sublayer(norm(x))); a looped span; logits against the embedding table
  std::vector<StackRun> runs;          // affine designs: the layers in the order they run
  ebyte* w_loop = nullptr;             // [width][2 width]: the loop's input product on [x; x0]
  float* xcat = nullptr;               // step workspace [T][2 width]: the stream beside the embedding output
  unsigned short* qplanes = nullptr;   // step workspace [2][T][max_qd]: an attention layer's queries as two 16-bit terms (matrix-core score products)
  int max_qd = 0;
  float *mixed = nullptr, *lora = nullptr, *rec_in = nullptr;      // joint designs' step workspace: the token-shift mixes, the decay's inner product, the delta rule's inputs
  int max_shift = 0, max_lora = 0, max_rec = 0;
  ebyte* head = nullptr;               // [vocab][width] (sandwich and joint designs; the others multiply by the embedding table)
  float* norm_g = nullptr;             // [4 * layers + 1] norm numbers, the final norm's last
  std::vector<RotTable> rot;
  float *a2 = nullptr, *ytmp = nullptr, *ysh = nullptr, *sgw = nullptr, *vfirst = nullptr, *hs = nullptr;      // more step workspace
  int max_kvv = 0, max_sff = 0;
  // pages
  int page = 64, page_shift = 6, n_pages = 0, tbl_stride = 0;
  int* tbl_dev = nullptr;
  int* tbl_host = nullptr;             // pinned mirror [slots][tbl_stride]
  std::vector<int> free_pages, row_pages, row_par;
  std::vector<char> row_dirty;
  // step workspace, grown to the largest step seen
  int cap_tokens = 0, cap_want = 0;
  int* meta_dev = nullptr; int* meta_host = nullptr; size_t meta_cap = 0;      // one block of ints: the StepMeta arrays + the wanted rows
  hipEvent_t meta_ev = nullptr; bool meta_pending = false;
  float *x = nullptr, *xs = nullptr, *a = nullptr, *proj = nullptr, *ql = nullptr, *lat = nullptr, *o = nullptr;
  float* zr = nullptr;                 // [T][experts] router products
  float *selw = nullptr, *yh = nullptr, *yd = nullptr, *xn = nullptr, *lg = nullptr, *part = nullptr;
  size_t part_elems = 0;
  int *sel = nullptr, *moe_off = nullptr, *perm = nullptr, *ptok = nullptr, *tile_e = nullptr, *tile_m0 = nullptr, *n_tiles = nullptr;
  int max_in = 0, max_hr = 0, max_hv = 0, max_top = 0, max_ff = 0, max_E = 0, max_rank = 0;
  int attn_split_min_keys = 2048;      // option attn.split_min: steps of few tokens split a sequence's keys between workgroups from this context on
  int gqa_split_min_keys = 1024;       // option attn.gqa_split_min: the same threshold for the grouped-query kernels, counted in keys a workgroup would walk (a mask's span); attn.split_min sets both
  int attn_mfma = 1;                   // option attn.mfma: 0 keeps every layer on the lane-per-channel attention kernels
  int gemv = 1;                        // option stack.gemv: 0 sends products of few rows through the matrix-core tiles as well
  int mlstm_narrow = -1;               // option mlstm.narrow: the matrix-memory scan's columns per wave (1: eight, 0: sixteen, -1: by the step's entries and heads)
  int mix_groups = 0;                  // option attn.mix_groups: key / value heads per workgroup of the matrix-core sigmoid attention: 1; 2 where their accumulators fit, whatever the grid; 0: 2 while the halved grid fills the chip
  int gemm_wt = 0;                     // option stack.gemm_wt: force the product's tile (1: 64 x 64, 2: 128 x 128); 0 = by the number of tiles
};

// stack_gqa.hip
namespace tgx { struct StepMeta; struct GqaMfmaArgs; struct MixMfmaArgs; }
bool gqa_mfma_shapes_ok(int dt, int dim, int vdim, int page_shift, long long ldq);
void launch_gqa_mfma(tgx_ctx* c, const tgx::StepMeta& m, const tgx::GqaMfmaArgs& a, dim3 grid, bool split);
void launch_mix_mfma(tgx_ctx* c, const tgx::StepMeta& m, const tgx::MixMfmaArgs& a, dim3 grid);      // kernels/stack_mix_mfma.h
size_t mix_mfma_wg_lds(int heads, int kv_heads);      // LDS bytes of one of its workgroups

int stack_create(const tgx_stack_desc* desc, const tgx_layer_desc* layers, int device_ordinal, tgx_ctx** out_ctx);
int stack_upload(tgx_ctx* c, const char* name, const void* host, const int64_t* shape, int nd, int src_dtype);
int stack_finalize(tgx_ctx* c);
void stack_destroy(tgx_ctx* c);
int stack_step(tgx_ctx* c, int n_entries, const int32_t* rows, const int32_t* counts, const int64_t* ids, int n_want, const int32_t* want, float* out_logits);
int stack_decode(tgx_ctx* c, const tgx_sampler_cfg& cfg, uint64_t seed, int n_steps);
int stack_reset_row(tgx_ctx* c, int row);
int stack_free_tokens(const tgx_ctx* c);
int stack_read_latent(tgx_ctx* c, int row, int layer, float* out);
int64_t stack_bytes_per_token(const tgx_ctx* c, int64_t T);
