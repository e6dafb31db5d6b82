/*
 * tgx.h — the drop-in boundary of the MI355X decode path (C ABI, no C++/torch types).
 *
 * TinyGPT has no FFI of its own: the device is a tinytorch::Device value threaded through
 * GPTConfig -> ModelLoader::load -> every nn::Module (reference: src/engine/GPTEngine.h:25-32,
 * src/huggingface/ModelLoader.cpp:25-89) and CPU-vs-CUDA dispatch happens inside TinyTorch.
 * This header defines the boundary at the seams the reference does expose — the virtual
 * GPTModel interface (src/model/GPTModel.h:80-106), KVCacheManager (src/engine/CacheManager.h:18-55),
 * Sampler::sample (src/engine/Sampler.h:30, Sampler.cpp:23-79) and the AsyncTokenPipeline hook
 * (src/engine/GPTEngine.cpp:17-35).  Each entry point names the reference interface it replaces.
 *
 * Conventions (mirroring the reference's: bool returns + LOGE, exceptions disabled,
 * src/CMakeLists.txt:63-67; single engine thread, server/HttpServer.cpp:118-163):
 *   - every function returns a tgx_status (0 = ok) and never throws across the ABI;
 *   - one opaque context per GPU; all calls on a context come from one host thread;
 *   - the caller owns host buffers; the library owns device memory and one HIP stream;
 *   - host buffers may be pageable; ids are int64 like the reference's token tensors.
 */
#ifndef TGX_H
#define TGX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 3 (round 5): per-row sequence lifecycle (tgx_reset_row / tgx_forward_row / tgx_sample_row / tgx_past_length_row); tgx_get_option added and
 * tgx_engine_read_stats + the options engine.*, pf.*, attn.fold_*, lmhead.fuse_finalize removed since 2. */
#define TGX_ABI_VERSION 7   /* 4: layered models (tgx_create_stack, tgx_step_ragged); 5: Modepel (more mixers / feed-forward kinds in tgx_layer_desc);
                             * 6: Vitudra (masks, score bias and cap, shared key / value layers, two recurrent mixers, parallel sublayers);
                             * 7: Zaluvik (layer norms around every sublayer, a looped span of layers, un-normalised sigmoid attention with mixed heads,
                             *    windowed latent attention with a shared rotated key part, sigmoid group-limited router) */

#if defined(__GNUC__)
#define TGX_API __attribute__((visibility("default")))
#else
#define TGX_API
#endif

typedef struct tgx_ctx tgx_ctx;

typedef enum tgx_status {
  TGX_OK = 0,
  TGX_ERR_INVALID = 1,     /* bad argument (null pointer, batch/seq out of range, ...)        */
  TGX_ERR_UNSUPPORTED = 2, /* family / dtype / head_dim this backend does not implement       */
  TGX_ERR_DEVICE = 3,      /* a HIP call failed; tgx_last_error() has the HIP error string     */
  TGX_ERR_STATE = 4,       /* call order violated (forward before finalize, missing tensors)  */
  TGX_ERR_NOMEM = 5,       /* host or device allocation failed                                */
  TGX_ERR_NAME = 6,        /* tensor name not part of this model ("Unexpected key")           */
  TGX_ERR_SHAPE = 7,       /* "shape not equal for tensor" (SafeTensors.cpp:187-193)          */
  TGX_ERR_CONTEXT = 8      /* pastLength + seq would exceed contextSize()                     */
} tgx_status;

/* GPTModelType (src/model/GPTModel.h:71-78) */
typedef enum tgx_family {
  TGX_FAMILY_GPT2 = 1,
  TGX_FAMILY_LLAMA = 2,
  TGX_FAMILY_QWEN2 = 3,
  TGX_FAMILY_QWEN3 = 4,
  TGX_FAMILY_MISTRAL = 5,
  TGX_FAMILY_ZAKUSUN = 6,  /* a layered model (tgx_stack_desc below), no counterpart in the reference */
  TGX_FAMILY_MODEPEL = 7,  /* a layered model: rotary grouped-query attention and matrix-memory (mLSTM) layers, sandwich norms */
  TGX_FAMILY_VITUDRA = 8,  /* a layered model: one norm per layer in front of a mixer and a gated feed-forward that run side by side; windowed and chunked
                            * attention, shared key / value layers, decaying matrix states (token-shift "wkv" and gated delta rule) */
  TGX_FAMILY_ZALUVIK = 9   /* a layered model: layer norms (weight and bias) before and after every sublayer, a span of layers run several times with the
                            * embedding output fed back in, windowed sigmoid attention whose weights are mixed across heads, windowed latent attention
                            * with a rotated key part all heads share, erf-gelu feed-forwards and sigmoid-routed experts; logits against the embedding table */
} tgx_family;

/* tinytorch::DType values the CLI accepts (examples/inference/main.cpp:82-88) */
typedef enum tgx_dtype { TGX_F32 = 0, TGX_BF16 = 1, TGX_F16 = 2 } tgx_dtype;

/*
 * What the family factories derive from config.json (src/huggingface/ModelConfig.cpp:63-122,
 * src/model/ModelLlama.h:21-53, ModelQwen2.h:23-45, ModelMistral.h:23-40, ModelGPT2.h:226-230).
 */
typedef struct tgx_model_desc {
  int32_t family;         /* tgx_family                                                          */
  int32_t hidden;         /* hidden_size / n_embd                                                */
  int32_t layers;         /* num_hidden_layers / n_layer                                         */
  int32_t heads;          /* num_attention_heads / n_head                                        */
  int32_t kv_heads;       /* num_key_value_heads (must divide heads, Attention.h:38)             */
  int32_t head_dim;       /* hidden/heads for llama/qwen2/mistral (ModelLlama.h:37)              */
  int32_t inter;          /* intermediate_size (4*n_embd for GPT-2, ModelGPT2.h:96)              */
  int32_t vocab;          /* vocab_size                                                          */
  int32_t max_ctx;        /* GPTModel::contextSize(): KV capacity and RoPE table length          */
  int32_t qkv_bias;       /* 1 for Qwen2 (ModelQwen2.h:26-31) and GPT-2                          */
  int32_t tied;           /* tie_word_embeddings: lm_head aliases embed_tokens (GPTModel.h:39-41)*/
  int32_t compute_dtype;  /* tgx_dtype the model is cast to after load (ModelLoader.cpp:84)      */
  float norm_eps;         /* rms_norm_eps / layer_norm_epsilon                                   */
  float rope_theta;       /* rope_theta                                                          */
  float rope_factor;      /* llama3 RopeScalingConfig.factor; 0 = std::nullopt (no scaling)      */
  float rope_low_freq;    /* .lowFreqFactor                                                      */
  float rope_high_freq;   /* .highFreqFactor                                                     */
  int32_t rope_orig_ctx;  /* .originalMaxPositionEmbeddings                                      */
  int32_t n_positions;    /* GPT-2 wpe rows; 0 otherwise                                         */
  int32_t max_batch;      /* rows of independent KV state to allocate (>= 1)                     */
  int32_t qk_norm;        /* 1: per-head RMSNorm on q and k before RoPE (AttentionWithQKNorm,    */
                          /*    src/layer/Attention.h:128-167; Qwen3, ModelQwen3.h:23-40)        */
} tgx_model_desc;

/* ---- layered models (ABI 4) ----------------------------------------------------------------
 * A model whose config.json lists its layers one by one, each with its own mixer and feed-forward sizes, does not fit the flat
 * tgx_model_desc: it is described by one tgx_stack_desc and an array of tgx_layer_desc, created by tgx_create_stack, and served by the
 * same calls as the other families (tgx_upload by checkpoint name, tgx_finalize, tgx_forward / tgx_forward_row, tgx_sample*, tgx_decode,
 * tgx_step_async, tgx_reset_row / tgx_reset_cache, tgx_read_logits) plus tgx_step_ragged.  Its rows are sequence slots: a slot holds the
 * short-convolution inputs of every sublayer and a table of pages of the shared latent cache pool.
 * Mechanisms (each a parameterised building block of csrc/kernels/stack*.h):
 *   grouped RMS norm          the vector in norm_groups equal parts, each divided by its own sqrt(mean(part^2) + norm_eps), times a weight
 *   input convolution         every sublayer reads h + conv(h), conv a causal depth-wise filter of canon_taps taps over the normed inputs
 *   latent attention          queries per head against a shared low-rank latent (the only cached quantity), softmax with a learned per-head
 *                             sink in the denominator, sigmoid output gate
 *   mixture of experts        top-k of a 32-bit router (+ bias), weights = softmax over the chosen logits, clamped gated experts
 *   depth average             the stream handed to layer i + 1 is a learned weighting of the embedding output and all layer results so far
 *   sinusoidal positions      added to the embedding rows (interleaved sin / cos, base 10000)
 * and, for TGX_FAMILY_MODEPEL (whose slots hold pages of a key / value pool and one recurrent state per mLSTM layer):
 *   scalar RMS norm           x / sqrt(mean(x^2) + norm_eps) times ONE learned number, before and after every sublayer ("sandwich"):
 *                             x <- x + norm_b(sublayer(norm_a(x)))
 *   grouped-query attention   heads query heads over kv_heads cached key / value heads, biases on q / k / v, rotary positions on the first rot_dims
 *                             dimensions of every head (rotate-half pairing, base rot_base), score scale `scale`, a sink of score 0 without a value
 *                             in the softmax denominator, values mixed with the first such layer's values of the same token (v_mix), sigmoid output gate
 *   mLSTM                     matrix memory per head with exponential input gate, sigmoid forget gate (both soft-capped by gate_cap), a running
 *                             maximum that starts at 0, fp32 state per slot; per-head RMS norm, learned scale, sigmoid output gate
 *   dense feed-forward        down(PolyNorm(up(h))): a N(z) + b N(z^2) + c N(z^3) + e over a token's ff values
 *   grouped-choice experts    softmax router over experts + identity outputs; the choice adds a correction and is limited to the best groups_keep of
 *                             `groups` neighbour groups; weights = scores * router_scale; identity outputs hand the input through; gated-silu
 *                             experts; a shared expert of width shared_ff with a per-token sigmoid gate
 * and, for TGX_FAMILY_VITUDRA (x <- x + residual_mult * (mixer(h) + ff(h)), h = x / sqrt(mean(x^2) + norm_eps) * (1 + w); slots hold pages of the
 * attention layers' key / value pools, one matrix state per recurrent head, the token-shift row and the convolution tails):
 *   attention masks           mask_kind 1: a sliding window (position i sees j with 0 <= i - j < mask_size); 2: chunks (i sees j <= i of its own block of
 *                             mask_size positions, counted from the start of the sequence); 0: every j <= i
 *   score shaping             score = q . k * scale; then softcap * tanh(score / softcap) (softcap > 0); then minus slope_h * (i - j), slope_h =
 *                             2^(-8 (h + 1) / heads) (dist_bias); queries times 1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1) at position p
 *   rotary variants           rot_pairs 1 turns neighbours (2i, 2i + 1) instead of (i, i + rot_dims / 2); every angle is divided by rot_factor (> 0)
 *   shared keys and values    kv_share = 1 + j: the layer has no key / value projections and reads layer j's pool with its own queries and mask
 *   wkv                       token shift (every projection reads h + (h_before - h) * mu of its own), a decay per key channel from a low-rank product
 *                             (decay_rank), S <- diag(w) S + k v^T read with a bonus u for the current token, per-head unit norm, silu gate
 *   gated delta rule          causal depth-wise convolutions of conv_taps taps and silu on q, k, v; unit q and k; S <- g S; S += k (beta (v - S^T k))^T;
 *                             o = S^T q; per-head unit norm, a weight shared by the heads, silu gate
 *   parallel mixer            left_scale * attention + right_scale * gated delta rule on the same input (the d_* fields size the right half)
 *   dense gated feed-forward  down(silu(gate h) * (up h))
 * and, for TGX_FAMILY_ZALUVIK (x <- x + residual_mult * LN_b(sublayer(LN_a(x))), LN(v) = (v - mean) / sqrt(var + norm_eps) * w + b; slots hold pages of one
 * key / value pool (attention) or latent pool (latent attention) per layer RUN, so a layer inside the loop keeps one cache per pass):
 *   embedding scale           x = embed[token] * embed_scale
 *   loop                      layers loop_start .. loop_stop - 1 run loop_times times in a row with the same weights; in front of the first layer of every
 *                             pass x <- W_loop [x; x0], x0 the embedding output ("loop.in" [width][2 width])
 *   unit queries and keys     qk_norm 1: every query and key head is divided by sqrt(mean(head^2) + norm_eps) (no weight)
 *   sigmoid attention         score_fn 1: the weight of a visible key is sigmoid(q . k * scale + pb[head]); weights are not normalised over the keys
 *   mixed heads               head_mix 1: weight_h(i, j) <- sum_g talk[h][g] weight_g(i, j) before the values are summed (head h keeps its own value head)
 *   output gates              gate_kind 1: per output channel, sigmoid(W_g h) [heads * vdim]; 2: per head, sigmoid(W_g h) [heads]
 *   latent attention, rotated latent attention with rot_dim further query / key dimensions per head: the projection "dkv" has kv_rank + rot_dim rows, the last
 *                             rot_dim of which (not normed, rotated by position, rotate-half pairing over rot_dims = rot_dim) are a key part all heads
 *                             share; score = (q_plain . W_uk c + q_rot . k_rot) * scale; softmax without sink; mask_kind / mask_size as above
 *   erf-gelu feed-forward     ff_act 1: down(gelu(up h)), gelu(z) = z (1 + erf(z / sqrt 2)) / 2
 *   sigmoid router            router_fn 1: scores = sigmoid(W_r h) (32-bit), no correction; group_score 1: a group counts as the sum of its two largest
 *                             scores; router_norm 1: weights = chosen scores / (their sum + 1e-20); a shared expert (shared_ff) without a gate of its own */
typedef enum tgx_mixer { TGX_MIXER_LATENT_ATTENTION = 1, TGX_MIXER_ATTENTION = 2, TGX_MIXER_MLSTM = 3, TGX_MIXER_WKV = 4, TGX_MIXER_PARALLEL = 5 } tgx_mixer;
typedef enum tgx_mlp { TGX_MLP_NONE = 0, TGX_MLP_MOE = 1, TGX_MLP_DENSE = 2 } tgx_mlp;
typedef enum tgx_mask { TGX_MASK_CAUSAL = 0, TGX_MASK_WINDOW = 1, TGX_MASK_CHUNK = 2 } tgx_mask;

typedef struct tgx_layer_desc {
  int32_t mixer;     /* tgx_mixer                                                                 */
  int32_t heads;     /* query heads                                                               */
  int32_t dim;       /* query / key dimensions per head                                           */
  int32_t vdim;      /* value dimensions per head                                                 */
  int32_t kv_rank;   /* width of the cached latent                                                */
  float scale;       /* score scale                                                               */
  int32_t mlp;       /* tgx_mlp                                                                   */
  int32_t experts;   /* experts of the layer                                                      */
  int32_t top;       /* experts per token                                                         */
  int32_t ff;        /* expert width                                                              */
  float limit;       /* clamp of the expert's gate (from above) and up (both sides) projections   */
  /* ABI 5 (zero for the mixers / feed-forward kinds that do not read them) */
  int32_t kv_heads;  /* attention: key / value heads (query head h reads head h / (heads / kv_heads)) */
  int32_t rot_dims;  /* attention: rotated dimensions per head (even, <= dim; 0: none)            */
  float rot_base;    /* attention: dimension pair i turns by position * rot_base^(-2i / rot_dims) */
  int32_t v_mix;     /* attention: 1 = values are mixed with the first such layer's values        */
  float gate_cap;    /* mLSTM: soft cap of the gate pre-activations, cap * tanh(z / cap)          */
  int32_t identity;  /* experts: router outputs beyond `experts` that hand the input through      */
  int32_t groups;    /* experts: neighbour groups of router outputs (<= 1: no group limit)        */
  int32_t groups_keep; /* experts: groups whose members may be chosen                             */
  float router_scale;  /* experts: weights = scores * router_scale                                */
  int32_t shared_ff; /* experts: width of the shared expert (0: none)                             */
  /* ABI 6 (zero for the kinds that do not read them) */
  int32_t mask_kind; /* attention: tgx_mask                                                       */
  int32_t mask_size; /* attention: window / chunk length in positions                             */
  float softcap;     /* attention: soft cap of the scaled score (<= 0: none)                      */
  int32_t dist_bias; /* attention: 1 = minus 2^(-8 (h + 1) / heads) * (i - j)                     */
  float q_temp_coef; /* attention: query temperature (0: none) ...                                */
  int32_t q_temp_every; /*         ... and its period in positions                               */
  int32_t rot_pairs; /* attention: 1 = rotate neighbours (2i, 2i + 1)                             */
  float rot_factor;  /* attention: angles are divided by this (<= 0: 1)                           */
  int32_t kv_share;  /* attention: 1 + the layer whose keys and values this one reads (0: its own) */
  int32_t decay_rank; /* wkv: inner size of the decay's low-rank product (0: from the tensors)    */
  int32_t d_heads;   /* parallel: the gated delta rule's value heads ...                          */
  int32_t d_kv_heads; /*          ... its query / key heads                                      */
  int32_t d_dim;     /*           ... their size                                                 */
  int32_t d_vdim;    /*           ... the value size per head                                    */
  int32_t conv_taps; /*           ... taps of its input convolutions                             */
  float left_scale;  /* parallel: weight of the attention half                                    */
  float right_scale; /* parallel: weight of the gated delta rule                                  */
  /* ABI 7 (zero for the kinds that do not read them) */
  int32_t qk_norm;   /* attention: 1 = unit-RMS queries and keys per head                         */
  int32_t score_fn;  /* attention: 0 = softmax over the visible keys, 1 = sigmoid(score + per-head bias), not normalised */
  int32_t head_mix;  /* attention: 1 = weights mixed across heads by a [heads][heads] matrix      */
  int32_t gate_kind; /* output gate: 0 = the family's own, 1 = per channel, 2 = per head          */
  int32_t rot_dim;   /* latent attention: rotated query / key dimensions per head beside `dim` (0: none) */
  int32_t ff_act;    /* dense feed-forward: 0 = the family's own, 1 = erf gelu without a gate     */
  int32_t router_fn; /* experts: 0 = softmax scores + correction, 1 = sigmoid scores              */
  int32_t group_score; /* experts: a group counts as 0 = its largest, 1 = the sum of its two largest scores */
  int32_t router_norm; /* experts: 1 = weights divided by their sum + 1e-20                       */
} tgx_layer_desc;

typedef struct tgx_stack_desc {
  int32_t family;         /* tgx_family (TGX_FAMILY_ZAKUSUN, TGX_FAMILY_MODEPEL, TGX_FAMILY_VITUDRA, TGX_FAMILY_ZALUVIK) */
  int32_t width;          /* residual width                                                        */
  int32_t layers;         /* entries of the tgx_layer_desc array                                   */
  int32_t vocab;
  int32_t compute_dtype;  /* tgx_dtype of the stored matrices and of the latent cache              */
  int32_t max_seqs;       /* sequence slots (rows)                                                 */
  int32_t max_ctx;        /* longest sequence a slot may hold                                      */
  int32_t budget_tokens;  /* tokens of the latent cache pool all slots share (<= 0: max_seqs * max_ctx) */
  int32_t page_tokens;    /* tokens per page of that pool, a power of two (<= 0: 64)               */
  int32_t norm_groups;
  float norm_eps;
  int32_t canon_taps;     /* taps of the input convolution (>= 1)                                  */
  float logit_scale;      /* logits = embed . norm(x) * logit_scale                                */
  float residual_mult;    /* ABI 6, TGX_FAMILY_VITUDRA / ZALUVIK: the factor on what a sublayer adds to the stream */
  /* ABI 7, TGX_FAMILY_ZALUVIK */
  float embed_scale;      /* x = embed[token] * embed_scale                                         */
  int32_t loop_start;     /* layers loop_start .. loop_stop - 1 run loop_times times (an empty span: no loop) */
  int32_t loop_stop;
  int32_t loop_times;
} tgx_stack_desc;

/* SamplerConfig (src/engine/Sampler.h:13-22).  Greedy iff temperature<=0 && top_k<=0 &&
 * top_p>=1 && min_p<=0 (Sampler.cpp:15-21). */
typedef struct tgx_sampler_cfg {
  float temperature;
  int64_t top_k;
  float top_p;
  float min_p;
} tgx_sampler_cfg;

/* ---- lifetime ---------------------------------------------------------------------------- */

/* Number of visible MI355X devices (the `--device mi355x` probe; reference branch:
 * examples/inference/main.cpp:76-80). */
TGX_API int tgx_device_count(int* out_count);

/* == Model{Llama,Qwen2,Mistral}::Model*(config, device) (e.g. src/model/ModelLlama.h:57-65):
 * validates the description, binds the GPU, allocates parameter storage in compute_dtype. */
TGX_API int tgx_create(const tgx_model_desc* desc, int device_ordinal, tgx_ctx** out_ctx);

/* The layered counterpart of tgx_create: `layers` holds desc->layers entries.  Checkpoint names (tgx_upload): "embed", "final.norm",
 * "l<i>.norm1|norm2|canon1|canon2|dwa", "l<i>.mix.q|dkv|dkv.norm|uk|uv|sink|g|o", "l<i>.mlp.router|router.b", "l<i>.mlp.e<j>.gate|up|down".
 * TGX_FAMILY_MODEPEL: "embed", "head", "final.norm", "l<i>.norm1|norm1b|norm2|norm2b", attention "l<i>.mix.q|k|v(.b)|vmix|g|o", mLSTM
 * "l<i>.mix.q|k|v|g|o|norm|i(.b)|f(.b)", dense "l<i>.mlp.up|down|act", experts "l<i>.mlp.router|correction|e<j>.gate|up|down|shared.gate|up|down|sg".
 * TGX_FAMILY_VITUDRA: "embed", "head", "final.norm", "l<i>.norm1", "l<i>.mlp.gate|up|down", attention "l<i>.mix.q|k|v|o" (no k, v with kv_share), wkv
 * "l<i>.mix.mu.r|k|v|g|w", "l<i>.mix.r|k|v|g|w1|w2|w0|u|norm|o", parallel "l<i>.mix.left.q|k|v|o", "l<i>.mix.right.q|k|v(.conv)|b|a|A_log|dt_bias|g|norm|o".
 * TGX_FAMILY_ZALUVIK: "embed", "loop.in" (with a loop), "final.norm(.b)", "l<i>.norm1|norm1b|norm2|norm2b(.b)", attention "l<i>.mix.q|k|v|talk|pb|g|o", latent
 * attention "l<i>.mix.q|dkv|dkv.norm|uk|uv|g|o", dense "l<i>.mlp.up|down", experts "l<i>.mlp.router|e<j>.gate|up|down|shared.gate|up|down". */
TGX_API int tgx_create_stack(const tgx_stack_desc* desc, const tgx_layer_desc* layers, int device_ordinal, tgx_ctx** out_ctx);

/* == SafeTensors::loadInternal -> Storage::copyOnDevice for ONE named tensor
 * (src/util/SafeTensors.cpp:157-215).  `hf_name` is the checkpoint key; q/k/v and gate/up land in
 * the row slices of the merged weights exactly like MergedLinear's LinearRef views
 * (src/layer/Linear.h:64-79).  Shape must match (TGX_ERR_SHAPE); an unknown key is TGX_ERR_NAME
 * (the reference warns "Unexpected key" and continues — callers may ignore that status).
 * ndim < 0 is a name probe: nothing is copied; TGX_ERR_NAME = unknown key, TGX_OK = a key this path knows and
 * ignores, TGX_ERR_SHAPE = a parameter the model needs (the loader uses it for tensors whose file dtype it cannot convert).
 * `src_dtype` is the dtype of `host`; conversion to compute_dtype happens on upload
 * (bf16->fp32 exact, fp32->bf16 round-to-nearest-even), == model().to(dtype), ModelLoader.cpp:84. */
TGX_API int tgx_upload(tgx_ctx* ctx, const char* hf_name, const void* host, const int64_t* shape, int ndim,
               int src_dtype);

/* == model().eval() + GPTModel::init(): checks every tensor arrived (TGX_ERR_STATE names the
 * first missing key in tgx_last_error), builds the RoPE tables (nn::RoPE ctor, ModelLlama.h:41-42),
 * allocates the KV cache for max_batch x max_ctx tokens and instantiates the decode graph. */
TGX_API int tgx_finalize(tgx_ctx* ctx);

TGX_API void tgx_destroy(tgx_ctx* ctx);

/* ---- the hot path ------------------------------------------------------------------------ */

/* == GPTModel::forward(inputIds[B,S]) + narrow-to-last-position (src/model/GPTModel.h:86,
 * src/engine/GPTEngine.cpp:96-97).  `ids` is a row-major host array [batch][seq] (left-padded by
 * the caller, no mask — GPTEngine.cpp:95).  Appends seq positions to every row's KV cache
 * (KVCacheManager::append, CacheManager.h:24-42) and leaves the last-position logits [batch][vocab]
 * on the device for tgx_sample / tgx_read_logits.  seq>1 with pastLength>0 is rejected with
 * TGX_ERR_INVALID (the reference would run it non-causally, Attention.h:108; its engine never does). */
TGX_API int tgx_forward(tgx_ctx* ctx, const int64_t* ids, int batch, int seq);

/* Copies the logits of the last tgx_forward / decode step to `out` [batch*vocab] as fp32.
 * rounded=1: values as the reference's logits tensor holds them (rounded to compute_dtype);
 * rounded=0: the fp32 accumulators before that rounding (for tolerance checks). */
TGX_API int tgx_read_logits(tgx_ctx* ctx, float* out, int rounded);

/* == Sampler::sample(logits[B,V]) (src/engine/Sampler.cpp:23-79) on the current logits.
 * The sampled ids become the device-resident "next token" of every row; if out_ids != NULL they
 * are also copied to the host ([batch], int64).  `seed` drives the multinomial draw (the
 * reference's RNG stream is not reproducible; greedy ignores it). */
TGX_API int tgx_sample(tgx_ctx* ctx, const tgx_sampler_cfg* cfg, uint64_t seed, int64_t* out_ids);

/* == the decode loop body of GPTEngine::generateSync (src/engine/GPTEngine.cpp:165-168), n_steps
 * times: nextToken = sample(forward(nextToken)).  Token ids and positions stay on the GPU between
 * steps; out_ids (may be NULL) receives [n_steps][batch] int64. */
TGX_API int tgx_decode(tgx_ctx* ctx, const tgx_sampler_cfg* cfg, uint64_t seed, int n_steps, int64_t* out_ids);

/* == AsyncTokenPipeline (src/engine/GPTEngine.cpp:17-35) for generateAsync's one-step lookahead
 * (GPTEngine.cpp:196-217), batch row 0.  tgx_step_async enqueues one decode step and returns
 * immediately with a ticket; tgx_fetch_token blocks until the step with that ticket has sampled
 * and returns its id.  Ticket 0 refers to the token produced by the last tgx_sample. */
TGX_API int tgx_step_async(tgx_ctx* ctx, const tgx_sampler_cfg* cfg, uint64_t seed, int64_t* out_ticket);
TGX_API int tgx_fetch_token(tgx_ctx* ctx, int64_t ticket, int32_t* out_id);

/* == GPTModel::resetCache() (src/model/GPTModel.h:91-94): pastLength back to 0 for all rows. */
TGX_API int tgx_reset_cache(tgx_ctx* ctx);

/* == KVCacheManager::pastLength (src/engine/CacheManager.h:44-51).  With rows of different lengths (see the per-row calls below): the LONGEST
 * row of the batch — the length every capacity check uses. */
TGX_API int64_t tgx_past_length(const tgx_ctx* ctx);

/* ---- per-row sequence lifecycle (ABI 3) ---------------------------------------------------
 * The kernel-contract half of the reference's continuous-batching TODO (README.md:33-34): the reference's KVCacheManager holds ONE pastLength for
 * the whole batch (src/engine/CacheManager.h:44-51) and its engine rebuilds the batch per request (src/engine/GPTEngine.cpp:67-84,180-232), so a
 * finished sequence blocks its slot until the longest one ends.  Here every row owns its cache slab and its device-resident position, and the
 * step kernels read the position per row: a row can be retired and another prompt prefilled into it while the other rows keep their state.
 * What a row keeps is the semantics of a solo sequence (Attention.h:71-112 over its own keys [0, pastLength_row]): its logits equal those of the
 * same prompt run alone up to the summation-order differences between kernel paths (tests/test_hip_rows.py).
 *
 * tgx_reset_row      == resetCache() for ONE row: its pastLength back to 0; the other rows and the batch size are untouched.  The row is now
 *                       RETIRED: tgx_decode / tgx_step_async keep stepping the live rows without waiting for it (a finished sequence with no queued
 *                       prompt stalls nobody).  It still rides in the steps (it decodes from position 0 on its stale token; its ids and logits in
 *                       tgx_decode's output / tgx_read_logits are meaningless and harmless) and counts for neither tgx_past_length nor the context
 *                       check; tgx_past_length_row reports 0 for it.  With every row retired there is nothing to step: tgx_decode refuses.
 * tgx_forward_row    == GPTModel::forward(inputIds[1,S]) for ONE row of the live batch: a retired `row` < batch (refill) or `row` == batch (the
 *                       batch grows by one row, up to max_batch); a live row must be retired first (tgx_reset_row).  Leaves the row's last-position
 *                       logits in its slot of tgx_read_logits; the row is live again but has no current token until tgx_sample_row (or tgx_sample)
 *                       ran — tgx_decode refuses until then.
 * tgx_sample_row     == Sampler::sample on ONE row's logits; the id becomes that row's device-resident next token.
 * tgx_past_length_row   the row's own pastLength. */
TGX_API int tgx_reset_row(tgx_ctx* ctx, int row);
TGX_API int tgx_forward_row(tgx_ctx* ctx, int row, const int64_t* ids, int seq);
TGX_API int tgx_sample_row(tgx_ctx* ctx, int row, const tgx_sampler_cfg* cfg, uint64_t seed, int64_t* out_id);
TGX_API int64_t tgx_past_length_row(const tgx_ctx* ctx, int row);

/* One engine step over a RAGGED batch (layered models; the continuous-batching step the reference's README.md:33-34 leaves as a TODO): entry e
 * brings counts[e] new tokens of slot rows[e] (distinct slots), all entries' ids concatenated in `ids`; each token attends its slot's cache
 * and the tokens before it in the entry — portions of prompts and single decoded tokens share the pass.  A slot is admitted by its first
 * entry (tgx_reset_row frees it) and may sit out any number of steps.  `want` lists n_want indices into the concatenated tokens whose logits are
 * written to out_logits [n_want][vocab] (fp32, host).  When an entry's LAST token is wanted, its logits also become the slot's current logits
 * (tgx_sample_row / tgx_read_logits).  Pages of the pool are assigned before anything is enqueued: TGX_ERR_CONTEXT leaves every slot as it was. */
TGX_API int tgx_step_ragged(tgx_ctx* ctx, int n_entries, const int32_t* rows, const int32_t* counts, const int64_t* ids, int n_want,
                            const int32_t* want, float* out_logits);

/* == GPTModel::contextSize() / numLayers() (src/model/GPTModel.h:97-98). */
TGX_API int64_t tgx_context_size(const tgx_ctx* ctx);
TGX_API int32_t tgx_num_layers(const tgx_ctx* ctx);

/* ---- diagnostics ------------------------------------------------------------------------- */

/* Last error text for this context (or for tgx_create when ctx == NULL). */
TGX_API const char* tgx_last_error(const tgx_ctx* ctx);

/* Blocks until all work enqueued on the context's stream has finished. */
TGX_API int tgx_synchronize(tgx_ctx* ctx);

/* Reads back the KV cache of (row, layer) as fp32 into k_out/v_out, each [pastLength of that row][kv_heads][head_dim]
 * (the BSHD view KVCacheManager::append returns, Attention.h:106).  Test/diagnostic use. */
TGX_API int tgx_read_kv(tgx_ctx* ctx, int row, int layer, float* k_out, float* v_out);

/* The inverse of tgx_read_kv: overwrites cache rows [0, n_rows) of (row, layer), n_rows <= pastLength, from fp32 k_in / v_in
 * [n_rows][kv_heads][head_dim] (either may be NULL), rounded once to the cache's storage dtype.  Test/diagnostic use: with the CPU path's
 * cache rows injected, a decode step is compared free of the bf16 KV-rounding floor (the reference's KVCacheManager holds the tensors
 * it was given, CacheManager.h:24-51 — there is nothing to overwrite there). */
TGX_API int tgx_write_kv(tgx_ctx* ctx, int row, int layer, const float* k_in, const float* v_in, int64_t n_rows);

/* Per-kernel-class timing with HIP events on the context's stream (bench.py's roofline leg).  For each
 * class (TGX_KERNEL_*) the kernels of ALL layers are launched back-to-back between two events, n_reps times,
 * at the current context length; returns launch counts and summed milliseconds.  Every launch streams a
 * different layer's weights (nothing repeats out of the Infinity Cache); residual outputs go to a scratch
 * vector so pastLength, the KV cache and the current token are unchanged (the logits buffer is consumed). */
#define TGX_KERNEL_QKV 0
#define TGX_KERNEL_ATTN 1
#define TGX_KERNEL_OPROJ 2
#define TGX_KERNEL_GATEUP 3
#define TGX_KERNEL_DOWN 4
#define TGX_KERNEL_LMHEAD 5
#define TGX_KERNEL_COUNT 6
TGX_API int tgx_profile_decode(tgx_ctx* ctx, int n_reps, int64_t* launches /*[TGX_KERNEL_COUNT]*/,
                       double* total_ms /*[TGX_KERNEL_COUNT]*/);

/* Final probability vector(s) [batch*vocab] of the last non-greedy tgx_sample / decode step: what the
 * reference passes to multinomial (Sampler.cpp:77) — zero where top-k/top-p/min-p removed a token.  A step
 * does not materialise the vector (the draw needs per-tile sums only): this call evaluates it from what the
 * step left on the device — valid until the next tgx_forward / tgx_forward_row / tgx_set_logits replaces the
 * logits (TGX_ERR_STATE then); rows whose last step was greedy read as zeros. */
TGX_API int tgx_read_probs(tgx_ctx* ctx, float* out);

/* Injects logits [batch][vocab] as if a forward had produced them, so that Sampler::sample can be
 * exercised on its own (the reference's Sampler takes any [B,V] tensor, Sampler.h:30). */
TGX_API int tgx_set_logits(tgx_ctx* ctx, const float* logits, int batch);

/* Launch-geometry knobs for tuning sweeps (results stay within the parity tolerances; summation order may change):
 *   "<class>.ks"   waves sharing a row pair's K range (1/2/4), class in {qkv,oproj,gateup,down,lmhead}
 *   "<class>.bpc"  grid cap in workgroups per CU ("lmhead.bpc" only before tgx_finalize)
 *   "attn.nsplit"  KV splits per kv head (<= 32, before tgx_finalize); "attn.gmax" query heads per attention workgroup
 *   "attn.direct_max"  contexts up to this many keys run attention as one workgroup per head group, without the combine launch (default 768 at head_dim 64, 384 at 128; 0 = never)
 *   "graph" 0/1    hipGraph replay vs eager launches; "graph.steps" decode steps per graph for long tgx_decode calls
 *   "prefill.min_rows"  prompts shorter than this take passes through the decode kernels instead of the batched prefill (default 7)
 *   "prefill.splitk" 0/1  split K over workgroups when a prompt gives the GEMMs few row tiles (default 1)
 *   "prefill.mfma" 0/1  batched matrix-core prefill vs passes through the decode kernels; "prefill.gemm_tm" 64/128 row tile
 *   "act.round16" 0/1  (default 0) numerics contract: 1 = the input of every Linear is rounded to the storage dtype (round-to-nearest-even) before the
 *                  product — what a module constructed in config.torch_dtype sees (ModelLlama.h:62) — instead of entering in fp32.  The matrix-core
 *                  products of the prefill and of batched steps then take one 16-bit term per activation instead of two or three;
 *                  fp32 storage: no effect.  Set it before the first tgx_forward of a sequence: the cache of a sequence must be filled under one contract
 *   "kv.budget_tokens"  (default 0; set BEFORE tgx_finalize, which sizes the caches; 16-bit storage dtypes) PAGED KV — the kernel contract of the reference's
 *                  "Paged Attention" TODO (README.md:32-34).  0: every row owns a max_ctx slab ([layer][kv_head][max_ctx][hd], max_batch x max_ctx tokens of
 *                  cache whatever the rows hold).  N > 0: the caches are pools of 128-token blocks worth N tokens in all, shared by the rows; a row's blocks are
 *                  assigned as its sequence grows (a device-resident block table per row, read by the attention and cache-append kernels) and returned by
 *                  tgx_reset_row / tgx_reset_cache; max_ctx stays the per-row limit.  A call that would need a block when none is free returns TGX_ERR_CONTEXT and
 *                  changes nothing (retire a row, retry).  Results are those of the unpaged cache, bit for bit on the same kernels (tests/test_hip_paged.py);
 *                  tgx_get_option "kv.free_tokens" = the unassigned blocks' worth of tokens (-1 when unpaged)
 *   "attn.split_min", "attn.gqa_split_min", "attn.mfma", "stack.gemv", "stack.gemm_wt", "mlstm.narrow", "attn.mix_groups"  (layered models) keys a workgroup walks from which a step of few
 *                  tokens divides them between workgroups (the first sets both thresholds, the second the grouped-query kernels' alone, counted in a mask's span);
 *                  0 = lane attention kernels only; 0 = few-row products on the matrix-core tiles too; forced product tile; the mLSTM scan's column split;
 *                  key / value heads per workgroup of the matrix-core sigmoid attention (1; 2 = two where their accumulators fit; 0 = two while the halved grid fills the chip)
 *   "debug.*"      experiment switches (tools/gemv_dissect.py, tools/attn_dissect.py; live only in a -DTGX_DISSECT=1 build) */
TGX_API int tgx_set_option(tgx_ctx* ctx, const char* key, int value);

/* Reads back what the library would do for the CURRENT batch size (no reference counterpart; callers that time a decode region use it to keep the
 * region on one attention form instead of mirroring the defaults):
 *   "attn.direct_limit"  decode steps at contexts up to this many keys run the direct attention form (batch-1 steps at head_dim 64: with the
 *                        o_proj product in the same launch), beyond it the split form
 *   "attn.nw4_limit"     ... and up to this many keys its four-wave variant (0 = never)
 *   "graph.steps"        decode steps per captured multi-step graph */
TGX_API int tgx_get_option(const tgx_ctx* ctx, const char* key, int* out_value);

/* Algorithmic HBM bytes one decoded token streams at context length T (SURVEY.md §8d formula). */
TGX_API int64_t tgx_bytes_per_token(const tgx_ctx* ctx, int64_t T);

TGX_API int tgx_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* TGX_H */
