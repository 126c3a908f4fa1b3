/*
 * inferflow_amd.h -- C ABI of the MI355X-native quantized decode path.
 *
 * This is the drop-in boundary for the lower surface that Inferflow's
 * GpuInferenceWorker calls:
 *   TensorOpr::*      src/tensor/tensor_opr.h:33-131
 *   TensorMul::*      src/tensor/tensor_mul.h:14-57
 *   CublasEngine      src/tensor/cublas_engine.h:31-33
 *   LayerKVCache      src/transformer/kv_cache.h:13-34
 *   CudaUtil          src/common/cuda_util.h:40-61
 * and, one level up, for the per-step work of GpuInferenceWorker::Run
 * (src/transformer/inference_worker.cc:234-340) behind InferenceEngine
 * (src/transformer/inference_engine.h:32-129).
 *
 * Conventions
 *  - extern "C", plain pointers and sizes, no C++/torch types.
 *  - Every function returns 0 on success or a negative IFA_ERR_* code;
 *    ifa_last_error() returns the message of the last failure on this thread
 *    (the reference ops return false + LogError; never throw).
 *  - All data pointers are DEVICE pointers unless the name says host.
 *  - `stream` is a hipStream_t passed as void* (NULL = default stream).  No op
 *    synchronises; the reference's "synchronous on return" behaviour is
 *    obtained by calling ifa_stream_sync() after the op.
 *  - dtype ids are the reference's ElementType enum values
 *    (src/tensor/tensor_common.h:15-42).
 *  - Tensors are row-major with ne0 (columns) contiguous, like DeviceTensor
 *    (src/tensor/device_tensor.h:85-153).  Quantized rows hold
 *    cols/capacity blocks in the reference's byte layout
 *    (src/common/quant_types.h:11-174).
 */
#ifndef INFERFLOW_AMD_H_
#define INFERFLOW_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    IFA_F32 = 0, IFA_F16 = 1, IFA_BF16 = 2,
    IFA_Q8_B32T1 = 7, IFA_Q8_B32T2 = 8, IFA_Q6_B64T1 = 9, IFA_Q5_B64T1 = 10, IFA_Q5_B32T1 = 11,
    IFA_Q4_B16 = 12, IFA_Q4_B32T1A = 13, IFA_Q4_B32T1B = 14, IFA_Q4_B64T1 = 17, IFA_Q3H_B64T1 = 18,
    IFA_Q3_B32T1A = 19, IFA_Q3_B32T1B = 20, IFA_Q2_B32T1A = 21, IFA_Q2_B32T1B = 22
} ifa_dtype;

enum {
    IFA_OK = 0,
    IFA_ERR_ARG = -1,      /* bad shape / null pointer / misaligned size */
    IFA_ERR_DTYPE = -2,    /* dtype not supported by this op */
    IFA_ERR_HIP = -3,      /* HIP runtime error */
    IFA_ERR_STATE = -4,    /* object not initialised / wrong phase */
    IFA_ERR_NOMEM = -5
};

typedef void *ifa_stream;

/* ---- library ------------------------------------------------------------ */
const char *ifa_version(void);
const char *ifa_last_error(void);
/* number of visible HIP devices (0 if none); never fails */
int ifa_device_count(void);

/* ---- CudaUtil counterparts (src/common/cuda_util.h:40-61) --------------- */
int ifa_set_device(int device);
int ifa_malloc(void **dptr, size_t bytes);
int ifa_free(void *dptr);
int ifa_memcpy_h2d(void *dst, const void *src_host, size_t bytes, ifa_stream stream);
int ifa_memcpy_d2h(void *dst_host, const void *src, size_t bytes, ifa_stream stream);
int ifa_memcpy_d2d(void *dst, const void *src, size_t bytes, ifa_stream stream);
int ifa_memset(void *dst, int value, size_t bytes, ifa_stream stream);
int ifa_stream_create(ifa_stream *out);
int ifa_stream_destroy(ifa_stream s);
int ifa_stream_sync(ifa_stream s);

/* ---- type registry (src/tensor/tensor_common.cc:6-234) ------------------ */
int ifa_block_capacity(int dtype);               /* 0 if unknown */
int ifa_block_bytes(int dtype);
size_t ifa_row_bytes(int dtype, size_t cols);    /* TensorCommon::ByteCount per row */
/* "q4" -> IFA_Q4_B32T1A etc.; returns -1 if unknown (InitElementTypeMap :171-205) */
int ifa_dtype_from_name(const char *name);

/* ---- TensorOpr::Quantize / Dequantize (src/tensor/tensor_opr.cu:1623, :2229) */
/* src F16 [rows][cols] -> packed reference-layout blocks.  Q8_B32T2 uses the
 * device alg-2 quantizer (src/kernels/tensor_quant.h:44-82) like the reference. */
int ifa_quantize(int dtype, const void *src_f16, size_t rows, size_t cols, void *dst, ifa_stream stream);
int ifa_quantize_f32(int dtype, const void *src_f32, size_t rows, size_t cols, void *dst, ifa_stream stream);
int ifa_dequantize(int dtype, const void *src, size_t rows, size_t cols, void *dst_f16, ifa_stream stream);
/* activation / KV-row quantizer: F16 [rows][cols] -> Q8_B32T2, cols may be ragged */
int ifa_quantize_act_q8(const void *src_f16, size_t rows, size_t cols, void *dst, ifa_stream stream);

/* ---- TensorMul::Gemv_AX (src/tensor/tensor_mul.h:27, tensor_mul.cu:766-846) */
/* y[rows] (F16) = W[rows][cols] . x (+bias).  x_dtype is IFA_Q8_B32T2 (the
 * int8 x intN path, gemv.h:1499-1709; W must be one of the 7 eligible types)
 * or IFA_F16 (gemv.h:469-1497; any W type incl. IFA_F16).  bias may be NULL. */
int ifa_gemv(int w_dtype, const void *W, size_t rows, size_t cols,
             int x_dtype, const void *x, const void *bias_f16, void *y_f16, ifa_stream stream);

/* ---- prefill / batched linear layer (MatrixMultiplication's T>1 branch,
 * src/transformer/inference_worker.cc:2374-2415: TensorOpr::Dequantize + CublasEngine::GemmEx
 * F16xF16->F16 with fp32 accumulate + Transpose).  Y[tokens][rows] (F16) = X[tokens][cols] (F16)
 * . W[rows][cols]^T (+bias); W in any block format (reference layout) or F16.  No F16 copy of W exists: up to 128 tokens
 * every lane dequantises the blocks it needs into its MFMA operand registers (split-K kernels, weight-stream bound);
 * above 128 tokens (formats with blocks of <= 32 values) a workgroup dequantises its weight tile once per K step into
 * LDS and 256 x 256 / 128 x 256 / 128 x 128 output tiles are multiplied from there (v_mfma_f32_32x32x16_f16).
 * Every T runs these in-tree kernels: the library neither links nor loads a vendor GEMM. */
int ifa_gemm(int w_dtype, const void *W, size_t rows, size_t cols, const void *x_f16, size_t tokens,
             const void *bias_f16, void *y_f16, ifa_stream stream);
/* the large-tile kernel for tokens > 128 (default 1; 0: the smaller-tile kernels serve every T).  The tile kernels add the same
 * products in DIFFERENT orders (and the split-K form of the 128 x 128 tiles adds its two halves of K as first + second): results
 * agree within the F16 rounding of one product row, they are not bit-identical.  < 0 only queries; returns the previous setting */
int ifa_gemm_big_tiles(int on);

/* ---- launches that wait for sibling workgroups inside the launch (the fused QKV + attention step, the split-K halves of the
 * large-tile GEMM, the K parts of the 9..32-row GEMM).  They are chosen only when the whole waiting grid can be resident at once:
 * occupancy of the kernel x the CUs this process may use (ROC_GLOBAL_CU_MASK / HSA_CU_MASK are read; IFA_VISIBLE_CUS overrides).
 * Every wait is bounded (0.2 s); one that gives up leaves a code, the synchronising call (ifa_stream_sync, ifa_model_forward /
 * _decode / _decode_batch) returns IFA_ERR_STATE, and the waiting launches stay off for the rest of the process -- the HIP context
 * survives, the non-waiting kernels serve from there on.  IFA_NO_INLAUNCH_WAITS=1 (environment) starts the process that way;
 * per model: ifa_model_set_option "rows_kparts" / "gemm_splitk" / "fuse_attn" = 0.
 * host-only helpers (no device needed): the residency rule and the CU-mask reader behind that choice. */
int ifa_wait_grid_decision(int blocks_per_cu, int visible_cus, long long grid);      /* 1: the grid fits */
int ifa_visible_cus_from_mask(const char *mask_text, int device, int device_cus);    /* CUs the mask leaves for `device` */
int ifa_inlaunch_waits_enabled(void);
/* frees the scratch the prefill kernels keep for this stream on the current device (call before destroying a stream that ran
 * long-prompt attention; ifa_model_destroy / ifa_model_set_stream do it for the worker's) */
int ifa_gemm_release_stream(ifa_stream stream);

/* Re-tile reference-layout rows into the row-local plane layout the fused
 * decode kernels stream (DESIGN.md "HBM layout"): same bytes per row, row stride
 * padded to a multiple of 16 (ifa_tiled_row_bytes; 0 for types without a tiled
 * layout).  Supported for the AX8-eligible types; src and dst must not alias;
 * dst holds rows * ifa_tiled_row_bytes(dtype, cols) bytes. */
size_t ifa_tiled_row_bytes(int dtype, size_t cols);
int ifa_repack_weights(int dtype, const void *src, size_t rows, size_t cols, void *dst, ifa_stream stream);
/* same GEMV as ifa_gemv(x_dtype = Q8) reading the re-tiled layout */
int ifa_gemv_tiled(int w_dtype, const void *Wt, size_t rows, size_t cols,
                   const void *x_q8, const void *bias_f16, void *y_f16, ifa_stream stream);

/* ---- TensorOpr::LayerNormalization (tensor_opr.cu:458-602) --------------- */
/* kind 0 = RMS (x*rsqrt(mean(x^2)+eps)*(multi_base+w) + b), 1 = STD.  w,b may be NULL. */
int ifa_layernorm(int kind, const void *x_f16, size_t rows, size_t cols, const void *w_f16,
                  const void *b_f16, float multi_base, float eps, void *y_f16, ifa_stream stream);

/* ---- TensorOpr::PositionEmbedding (tensor_opr.cu:693-806) --------------- */
/* x F16 [tokens][heads][head_dim] in place; order 1 = adjacent pairs
 * (PosEmbedding_Rope_Std_Kernel), 2 = (c, c+rope_cols/2) (Rope_Order2). */
int ifa_rope(void *x_f16, int head_dim, int heads, int tokens, int pos0, float theta,
             int order, float partial_rotary_factor, ifa_stream stream);
/* scores F16 [heads][q_tokens][ctx] += col*m_head (PosEmbedding_Alibi_Std_Kernel) */
int ifa_alibi(void *scores_f16, int ctx, int q_tokens, int heads, int base_head, int total_heads,
              ifa_stream stream);

/* ---- TensorOpr::SoftMax (tensor_opr.cu:1189-1225) ------------------------ */
/* s F16 [cz][cy][cx] in place; element xi of row r is masked (-inf) iff
 * prefix_len >= 0 && xi > prefix_len + r; values are multiplied by scale first. */
int ifa_softmax(void *s_f16, int cx, int cy, int cz, int prefix_len, float scale, ifa_stream stream);

/* ---- TensorOpr::Activation / Mul / Add / Scale --------------------------- */
/* kind 0 silu, 1 gelu(tanh), 2 relu; is_glu: input rows are [2*cols], out = act(a)*b */
int ifa_activation(int kind, int is_glu, const void *x_f16, size_t rows, size_t cols, void *y_f16,
                   ifa_stream stream);
int ifa_mul(const void *a_f16, const void *b_f16, size_t n, void *c_f16, ifa_stream stream);
/* c = a + b, b broadcast with period b_period elements (0 = same size) */
int ifa_add(const void *a_f16, const void *b_f16, size_t n, size_t b_period, void *c_f16, ifa_stream stream);
int ifa_scale(const void *a_f16, float s, size_t n, void *c_f16, ifa_stream stream);
/* TensorOpr::AddByRowIndex (tensor_opr.cu:1519-1548, kernel binary_tensor_opr.h:80-125), the MoE scatter-add:
 * B[row_idx[r]][:] = hfma(A[r][:], weights[r], B[row_idx[r]][:]) in half precision (weights may be NULL = 1). */
int ifa_add_by_row_index(void *b_f16, const void *a_f16, size_t rows, size_t cols, const int *row_idx_dev,
                         const void *weights_f16_dev, ifa_stream stream);

/* ---- attention over a KV cache (inference_worker.cc:983-1405, :1639-1724) */
/* q F16 [q_tokens][heads][head_dim]; caches [n_ctx rows][kv_heads*head_dim] in
 * IFA_F16 or IFA_Q8_B32T2 (LayerKVCache, kv_cache.cc:104-249); causal mask with
 * prefix_len; GQA by indexing (no RepeatKV copy); out F16 [q_tokens][heads*head_dim].
 * alibi: 0/1; alibi_base_head/total_heads as in ifa_alibi. */
int ifa_attention(const void *q_f16, const void *kcache, const void *vcache, int kv_dtype,
                  int n_ctx, int q_tokens, int prefix_len, int heads, int kv_heads, int head_dim,
                  float kq_scale, int alibi, int alibi_base_head, int alibi_total_heads,
                  void *out_f16, ifa_stream stream);
/* ---- parity instruments: single-row ops in the SUMMATION ORDER of the reference's CUDA kernels (csrc/ifa_exact.hip) -- the 32-lane walk +
 * xor butterfly of Gemv_AX8_* (src/kernels/gemv.h:1499-1709; F16 activations: the serial fp32 order of the oracle's restatement of :469-1497),
 * Tensor_RmsNorm_Kernel's 128 chunks (unary_tensor_opr.h:216-289), serial fp32 attention dots + the 32-lane softmax (gemm.h:83-178,
 * unary_tensor_opr.h:480-535), SiLU / ReLU (+ gate) with libm's expf.  Results equal the CPU oracle's bit for bit; not timed kernels.
 * Same argument meaning as ifa_layernorm / ifa_gemv / ifa_attention (one query row, no ALiBi) / ifa_activation_mul (gate may be NULL). */
int ifa_exact_rmsnorm(const void *x_f16, size_t rows, size_t cols, const void *w_f16, const void *b_f16, float multi_base, float eps,
                      void *y_f16, ifa_stream stream);
int ifa_exact_gemv(int w_dtype, const void *W, size_t rows, size_t cols, int x_dtype, const void *x, const void *bias_f16, void *y_f16,
                   ifa_stream stream);
int ifa_exact_attention(const void *q_f16, const void *kcache, const void *vcache, int kv_dtype, int n_ctx, int heads, int kv_heads,
                        int head_dim, float kq_scale, void *out_f16, ifa_stream stream);
int ifa_exact_activation_mul(int kind, const void *a_f16, const void *gate_f16, size_t n, void *y_f16, ifa_stream stream);
/* chunks of at least min_tokens queries (default 64; 0 = never, < 0 only queries) take the two-pass kernels: K / V blocks staged
 * once per query tile, scores recomputed in the second pass instead of a [queries x keys] tile; head_dim 64 / 128; same rounding
 * points as the staged 32-query kernel.  Default variant: 64 queries per workgroup, the key blocks split over wave pairs;
 * on contexts of at least min_keys keys (default: never) chunks of >= 128 queries take the 128-query variant instead.
 * Each returns its previous threshold. */
int ifa_attention_two_pass_min(int min_tokens);
int ifa_attention_two_pass_min_keys(int min_keys);

/* ---- greedy argmax over F16 logits (SampleTokens top-1) ------------------ */
/* MoE routing of `tokens` softmaxed router rows [tokens][experts] on the device -- the per-row part of
 * HostTensorOpr::BuildRowsForMoE (src/tensor/host_tensor_opr.cc:190-244): top_k by repeated first maximum, probabilities
 * below 1e-5 dropped, optional renormalisation over the kept ones.  sel_out [tokens][top_k]: expert ids in ascending
 * order (-1 = unused slot), weights_out [tokens][top_k] F16.  (The reference copies the probabilities to the host.) */
int ifa_moe_route_topk(const void *probs_f16, size_t tokens, int experts, int top_k, int norm_top_k_prob, int *sel_out_dev,
                       void *weights_out_f16_dev, ifa_stream stream);
/* LayerKVCache::SetKRows / SetVRows (src/transformer/kv_cache.cc:159-249): `tokens` F16 rows [kv_dim] into rows
 * [first_row, first_row + tokens) of a K or V cache of dtype F16 (copy) or Q8_B32T2 (the Alg2 quantiser) */
int ifa_kv_store(int kv_dtype, const void *rows_f16, size_t tokens, size_t kv_dim, void *cache, size_t first_row, ifa_stream stream);
int ifa_argmax(const void *logits_f16, size_t n, int *out_index_dev, ifa_stream stream);
/* the same over the ALLOWED ids: excluded_dev = {count (<= 3), id, id, id} in device memory (nullable) -- the ids
 * SamplingStrategy::GetSortedTopK never offers to its queue: the vocabulary's unk id and Invalid-type tokens
 * (src/transformer/sampling_strategy.cc:281-297) */
int ifa_argmax_masked(const void *logits_f16, size_t n, const int *excluded_dev, int *out_index_dev, ifa_stream stream);

/* ======================================================================== */
/* Per-device decode worker: counterpart of GpuInferenceWorker                */
/* (src/transformer/inference_worker.h:23-62, inference_worker.cc:234-340)    */
/* for the hyper-parameters of ModelSpec (src/transformer/model.h:72-151).    */
/* ======================================================================== */
typedef struct ifa_model ifa_model;

typedef struct {
    int dim, layers, heads, kv_heads, head_dim, ffn, vocab, max_ctx;
    int norm_kind;       /* 0 rms, 1 std                      (normalization_function) */
    int act_kind;        /* 0 silu, 1 gelu, 2 relu            (activation_function)    */
    int is_glu;          /* informational: w3 present                                   */
    int rope_order;      /* 0 none, 1 adjacent pairs, 2 half-split (qk_column_order)    */
    int use_alibi;       /* position_embedding == alibi                                 */
    int parallel_attn;   /* is_parallel_attn                                            */
    int share_input;     /* mlp_attn_share_input                                        */
    float rope_theta, partial_rotary, kq_scale, eps;
    int kv_dtype;        /* IFA_F16 or IFA_Q8_B32T2 (device_kv_cache_data_type)         */
    int full_quant_gemv; /* enable_full_quant_gemv (inference_engine.cc:57)             */
    int experts, moe_top_k, moe_norm_topk;
    int tp_rank, tp_size;/* tensor-parallel shard of this worker (heads/kv_heads/ffn are per-shard) */
    int device;          /* HIP device ordinal */
    /* RMS weight = base + w (attn_pre_norm_base / ffn_pre_norm_base / output_norm_base: Gemma) and TensorOpr::Scale of
     * the attention output, the FFN output and the last layer's output (attn_out_scale / ffn_out_scale / out_scale:
     * MiniCPM; inference_worker.cc:568-570, 842-843, 928-929).  Scales <= 0 mean 1. */
    float attn_norm_base, ffn_norm_base, out_norm_base, attn_out_scale, ffn_out_scale, out_scale;
    /* TensorOpr::LinearNorm on the decoder input (has_embedding_linear_norm / embedding_linear_scale: Gemma, MiniCPM;
     * inference_worker.cc:447-451, tensor_opr.cu:482-497): every embedding row is multiplied by this scale;
     * 0 = absent, < 0 = the reference's default sqrt(dim). */
    float embd_scale;
} ifa_model_config;

/* tensor ids for ifa_model_set_tensor (StdDeviceNetwork, src/transformer/model.h:168-276) */
enum {
    IFA_T_EMBD = 0, IFA_T_OUT_NORM = 1, IFA_T_OUT_NORM_B = 2, IFA_T_LM_HEAD = 3,
    IFA_T_EMBD_NORM = 4,      /* layer-list models with stem 1: weight of the grouped RMS norm behind the embedding */
    IFA_T_BIGRAM = 5,         /* layer-list models with stem 2 / 3: hashed token-pair embedding [bigram_buckets + 1][width] */
    IFA_T_OUT_NORM_ALPHA = 6, /* layer-list models with stem 3: the scalar of the Dynamic Tanh norm before lm_head (its bias: IFA_T_OUT_NORM_B) */
    IFA_T_LOOP_STEP = 7,      /* layer-list models with a looped layer group: [loop_times][width], row t added before pass t */
    IFA_T_ATTN_NORM = 10, IFA_T_ATTN_NORM_B = 11, IFA_T_WQ = 12, IFA_T_WK = 13, IFA_T_WV = 14, IFA_T_WO = 15,
    IFA_T_FFN_NORM = 16, IFA_T_FFN_NORM_B = 17, IFA_T_W1 = 18, IFA_T_W2 = 19, IFA_T_W3 = 20, IFA_T_MOE_GATE = 21,
    IFA_T_WQ_B = 22, IFA_T_WK_B = 23, IFA_T_WV_B = 24, IFA_T_WO_B = 25, IFA_T_W1_B = 26, IFA_T_W2_B = 27, IFA_T_W3_B = 28,
    /* self_attn.post_norm / feed_forward.post_norm (+ biases): StdDeviceNetwork::AttentionLayer::post_norm, FeedForwardLayer::post_norm
     * (src/transformer/model.h:168-276); applied by ProcessGpuLayer (inference_worker.cc:857-866, 954-965).  Models that carry them take
     * the op-by-op layer (the fused decode / prompt launches decline).  ModelSpec::is_attn_post_as_residual (model.h:113, default
     * true) is the model option "attn_post_as_residual". */
    IFA_T_ATTN_POST_NORM = 29, IFA_T_ATTN_POST_NORM_B = 30, IFA_T_FFN_POST_NORM = 31, IFA_T_FFN_POST_NORM_B = 32
};

int ifa_model_create(const ifa_model_config *cfg, ifa_model **out);
int ifa_model_destroy(ifa_model *m);
/* Copy a tensor that is already in its final dtype (reference block layout or F16)
 * from device memory into the worker; eligible weight matrices are also re-tiled. */
int ifa_model_set_tensor(ifa_model *m, int layer, int tensor_id, int expert, int dtype,
                         const void *dev_src, size_t rows, size_t cols);
/* F16 source quantised on the device to target_dtype first
 * (DeviceTensorBuilder::Build_Quant, src/tensor/device_tensor_builder.cu:383-420). */
int ifa_model_set_tensor_f16(ifa_model *m, int layer, int tensor_id, int expert, int target_dtype,
                             const void *dev_src_f16, size_t rows, size_t cols);
/* allocate KV caches (KVCache::Init, kv_cache.cc:278-319) and scratch */
int ifa_model_finalize(ifa_model *m);
int ifa_model_reset(ifa_model *m);
/* options: "fused" (1), "graph" (1), "rpw_qkv|rpw_wo|rpw_ffn|rpw_w2|rpw_lm" (0 = auto), "batch_fused" (1), "rows_mo" (1: the batched
 * step and short prompts stream MFMA-operand-order copies of the weights, built on first use), "attn_split_ctx" (-1 = by model: 512 keys, 640 with grouped queries, 320 without the fused launch; a decode call that reaches more keys than this runs the attention as scores / P.V / combine launches with a head's keys split over 8 or 16 workgroups; 0: never), "fuse_attn" (1: the attention as the
 * tail of the wq | wk | wv launch), "attn_unload" (1: in the 256-row bucket of that launch the heads' workgroups take no weight rows and request their cache rows at once; 2: in the 128-row bucket too, measured slower), "fuse_ffn" (0; 1 / 2: [Wo ->] W1 | W3 -> W2 as one chained launch, csrc/ifa_decode_chain.h: bit-identical,
 * measured slower than the separate launches on MI355X, kept as the measurement harness of that statement), "prefill_mid" (1),
 * "prefill_mid_max" (768), "prefill_res_mid" (2048: up to this many tokens wo / w2 keep the mid-size kernel above prefill_mid_max), "prefill_big_min" (47), "attn_post_as_residual" (1), "exact_order" (0; 1: every single-token step -- and every row
 * of a prompt, one by one -- runs in the summation order of the reference's CUDA kernels, csrc/ifa_exact.hip: a parity instrument whose
 * logits, ids and int8 codes equal the CPU oracle's bit for bit; fails for models outside that step instead of changing arithmetic),
 * "q3h_native" (0; 1: Q3H_B64T1 Wo / W1 / W3 / W2 streamed at 32 bytes per block, pair codes decoded in the kernel: bit-identical, measured slower),
 * "perf_stat" (0; 1: steps and prompts take the op-by-op layer with a HIP event pair around every phase, see ifa_model_perf_stat) */
/* Independent KV caches inside one worker, one per concurrent query -- the reference keeps a LayerKVCache set
 * per query processor (QueryStateTable, src/transformer/query_state_table.h:19-85; KVCache::Init, kv_cache.cc:278-319).
 * ifa_model_kv_slots grows the number of caches to n_slots (slot 0 exists after finalize); ifa_model_select_kv
 * makes one of them the cache that forward()/decode() read and write (each slot keeps its own captured graph). */
int ifa_model_kv_slots(ifa_model *m, int n_slots);
int ifa_model_select_kv(ifa_model *m, int slot);
int ifa_model_set_option(ifa_model *m, const char *name, int value);
/* up to 3 token ids the worker's greedy argmax (forward / decode / decode_batch) never selects: the unk id and
 * Invalid-type tokens GetSortedTopK skips (sampling_strategy.cc:281-297).  None by default at this level; the engine
 * facade sets the model's unk id. */
int ifa_model_set_excluded_tokens(ifa_model *m, const int *ids_host, int n);
/* Per-phase times in the key space of the reference's InferencePerfStat (GpuInferenceWorker::UpdatePerfStat, inference_worker.cc:2670-2697;
 * keys: (layer + 1) * 10000 + phase -- + 0 the whole layer for layers 0..5 (:318-322); for layer 0, the reference's layer_idx_for_study_:
 * + 10 attention pre-norm, + 30 q / k / v products, + 50 RoPE + cache rows, + 60 scores / softmax / V product, + 90 wo, + 300 the attention
 * part as a whole, + 710 FFN pre-norm, + 730 w1, + 750 w3, + 760 activation * gate, + 780 w2, + 700 the FFN as a whole, + 800 what follows it;
 * 1000009 the output stage (:673-675), 1 the embedding rows (inference_engine.cc:1168-1176)).  With option "perf_stat" = 1 every
 * ifa_model_forward / ifa_model_decode step ADDS the device milliseconds of its spans to the keys (the reference adds host-side launch times);
 * this call drains the stream, copies up to cap (key, ms) pairs in ascending key order, stores the number of keys there are in *n_out and
 * clears the map if clear != 0. */
int ifa_model_perf_stat(ifa_model *m, int *keys_out, float *ms_out, int cap, int *n_out, int clear);
/* 1 if the fused batch-1 decode kernels cover this model, else 0 (+ reason) */
int ifa_model_fused_supported(ifa_model *m, char *why, size_t why_len);
/* One Infer() step for one query: n_tokens new tokens at positions
 * [prefix_len, prefix_len+n_tokens); op-by-op; synchronous.  logits_out_dev (F16
 * [n_tokens][vocab], nullable) mirrors return_output_tensors; *next_token_host is
 * the greedy argmax of the last row. */
int ifa_model_forward(ifa_model *m, const int *tokens_host, int n_tokens, int prefix_len,
                      void *logits_out_dev, int *next_token_host);
/* Greedy batch-1 decode of n_steps tokens starting from first_token at start_pos
 * (its KV rows [0,start_pos) must already be cached).  Fused kernels, one graph
 * replay per token, token fed back on the device.  out_tokens_host[n_steps]
 * receives the generated ids; *elapsed_ms (nullable) the HIP-event time of the
 * n_steps replays on the worker's stream. */
int ifa_model_decode(ifa_model *m, int first_token, int start_pos, int n_steps,
                     int *out_tokens_host, float *elapsed_ms);
/* Everything a decode call of n_steps from start_pos sets up before its first launch (the attention variant of the contexts it
 * reaches, the hand-off arenas, the captured step and its multi-step replay) WITHOUT running a step: a caller that times its
 * first call keeps graph capture / instantiation out of it.  The KV cache and the activations are not touched. */
int ifa_model_decode_prepare(ifa_model *m, int start_pos, int n_steps);
/* Dynamic batching: ONE new token for each of n queries in one step (QueryStateTable + Infer_Std over several queries,
 * src/transformer/inference_engine.cc:1054-1220).  Row r is token tokens[r] at position positions[r] of the query whose
 * KV cache is slot kv_slots[r] (ifa_model_kv_slots; slots must be distinct).  The linear layers run once over the n rows
 * (the weights are streamed once for all queries), attention per row on its own cache.  logits_out: optional [n][vocab] F16. */
int ifa_model_decode_batch(ifa_model *m, int n, const int *tokens_host, const int *positions_host, const int *kv_slots_host,
                           int *next_tokens_host, void *logits_out_dev);
/* debugging taps: "logits", "hidden", "kcache", "vcache" (device pointers) */
int ifa_model_get_buffer(ifa_model *m, const char *name, int layer, void **dptr, size_t *bytes);
void *ifa_model_stream(ifa_model *m);
/* run the worker on a caller-owned stream (e.g. the one the caller's RCCL collectives are ordered on) */
int ifa_model_set_stream(ifa_model *m, ifa_stream stream);

/* ======================================================================== */
/* Collectives of the multi-GPU partitions (RCCL over xGMI; csrc/ifa_comm.hip) */
/* -- what GpuInferenceWorker::DistributeAndMergeTensors / MergeTensors /     */
/* DeviceCopy (src/transformer/inference_worker.cc:2148-2335) and             */
/* GpuInfGlobalData (src/transformer/gpu_inf_global_data.cu:25-199) do with   */
/* host-side spin-waits and serial copies.  Enqueue-only, explicit stream,    */
/* capturable; one communicator per (rank, group).                            */
/* ======================================================================== */
typedef struct ifa_comm ifa_comm;
#define IFA_COMM_ID_BYTES 128
/* one process per GPU: rank 0 makes the id, ships the 128 bytes over any host channel, every rank joins */
int ifa_comm_unique_id(void *id_out_128);
int ifa_comm_init_rank(const void *id_128, int nranks, int rank, int device, ifa_comm **out);
/* one process, one host thread per GPU (the engine facade, like inference_engine.cc:1203-1206): all ranks at once */
int ifa_comm_init_all(const int *device_ids, int n, ifa_comm **comms_out);
/* a device list that names ONE device n times makes an in-process loopback group instead (RCCL refuses two ranks on a
 * device): kernels / copies on that device with a host rendezvous between the rank threads -- host-synchronous, not
 * capturable (ifa_comm_capturable() == 0); for exercising the multi-rank paths on a 1-GPU box */
int ifa_comm_capturable(const ifa_comm *c);
/* identity of the communicator OBJECT (a new one at the same address gets a new serial): what a cached, captured step
 * is keyed on */
unsigned long long ifa_comm_serial(const ifa_comm *c);
/* One-shot all-reduce (csrc/ifa_comm.hip): communicators made by ifa_comm_init_all whose devices can map each other's
 * memory exchange vectors of <= 64 KB directly (push into peer inboxes + epoch flags, sum in rank order in half: the
 * arithmetic of MergeTensors, inference_worker.cc:2197-2260) instead of a ring collective -- one launch per rank, no host
 * rendezvous.  ifa_comm_oneshot: 1 if this communicator does; ifa_comm_set_oneshot(c, 0) keeps RCCL for every size;
 * ifa_comm_status: non-zero if a wait inside a one-shot all-reduce of this rank gave up (2 s). */
int ifa_comm_oneshot(const ifa_comm *c);
/* One process per rank (ifa_comm_init_rank): export allocates this rank's inbox / flags and writes their two IPC handles
 * (IFA_ONESHOT_HANDLE_BYTES); the caller gathers all ranks' handles in rank order over the channel that carried the
 * communicator id; import maps the peers' buffers (hipIpcOpenMemHandle) -- ifa_comm_oneshot(c) is 1 afterwards. */
#define IFA_ONESHOT_HANDLE_BYTES 128
int ifa_comm_oneshot_export(ifa_comm *c, void *handle_out_128);
int ifa_comm_oneshot_import(ifa_comm *c, const void *handles_all_ranks);
int ifa_comm_set_oneshot(ifa_comm *c, int on);
int ifa_comm_status(ifa_comm *c);
/* Wake every rank blocked in (or later entering) a collective of this communicator with an error: called by the rank
 * that failed, or by whoever supervises the ranks (ncclCommAbort, inference_worker.cc has no counterpart: the reference
 * deadlocks its worker threads in this case).  The communicator can only be destroyed afterwards. */
int ifa_comm_abort(ifa_comm *c);
int ifa_comm_destroy(ifa_comm *c);
int ifa_comm_rank(const ifa_comm *c);
int ifa_comm_size(const ifa_comm *c);
/* one host thread issuing the calls of several ranks brackets them with group_start / group_end */
int ifa_comm_group_start(void);
int ifa_comm_group_end(void);
/* BY_TENSOR merge: element-wise sum of the ranks' partial [count] F16 vectors (in place allowed) */
int ifa_allreduce_sum_f16(ifa_comm *c, const void *send_f16, void *recv_f16, size_t count, ifa_stream stream);
/* recv = the ranks' `bytes_per_rank` blocks in rank order (distributed argmax over a vocabulary-sharded lm_head) */
int ifa_allgather(ifa_comm *c, const void *send, void *recv, size_t bytes_per_rank, ifa_stream stream);
int ifa_broadcast(ifa_comm *c, void *buf, size_t bytes, int root, ifa_stream stream);
/* BY_LAYER hand-over of the [T][dim] F16 layer output between device groups (DeviceCopy, :2300-2335) */
int ifa_send(ifa_comm *c, const void *buf, size_t bytes, int peer, ifa_stream stream);
int ifa_recv(ifa_comm *c, void *buf, size_t bytes, int peer, ifa_stream stream);

/* ---- tensor-parallel decode (BY_TENSOR partition, src/transformer/network_builder.cc:1594-1686):
 * the worker holds heads/tp_size heads, kv_heads/tp_size KV heads and ffn/tp_size FFN rows; the
 * caller sums the two partial [dim] F16 vectors per layer over the group exactly where the
 * reference calls DistributeAndMergeTensors (inference_worker.cc:1378-1391, :1882-1895).
 * All calls only enqueue work on the worker's stream.
 *   begin(token,pos)            token < 0 / pos < 0: keep the id / position already in the device state
 *   attn(l, partial)            norm + QKV + attention + Wo product (no bias/residual)
 *   post_attn(l, reduced)       + bias, + residual
 *   ffn(l, partial)             norm + W1/W3 + act + W2 product
 *   post_ffn(l, reduced)        + bias, + residual -> next layer input
 *   logits(shard_out)           final norm + this rank's vocabulary rows of lm_head
 *   set_token(dev_ptr)          next token id from device memory (after the distributed argmax); advances the
 *                               device-side position, so begin(-1,-1) ... set_token() is replayable as a hipGraph */
int ifa_model_tp_begin(ifa_model *m, int token, int pos);
/* BY_LAYER / HYBRID partition (MultiGpuStrategy, src/transformer/model.h:61-66; layer ranges per device group:
 * NetworkBuilder::SplitGpuLayers, network_builder.cc:2094-2118): a worker that holds a layer range only starts its
 * step from the previous group's output instead of an embedding row, and hands its last layer's output on.
 *   begin_hidden(x, pos)   layer input from device memory ([dim] F16); pos < 0 keeps the device-side position
 *   hidden(x_out)          copy of the current layer input/output vector (after the last local layer) */
int ifa_model_tp_begin_hidden(ifa_model *m, const void *x_f16, int pos);
int ifa_model_tp_hidden(ifa_model *m, void *x_out_f16);
int ifa_model_tp_attn(ifa_model *m, int layer, void *partial_out_f16);
int ifa_model_tp_post_attn(ifa_model *m, int layer, const void *reduced_f16);
int ifa_model_tp_ffn(ifa_model *m, int layer, void *partial_out_f16);
int ifa_model_tp_post_ffn(ifa_model *m, int layer, const void *reduced_f16);
int ifa_model_tp_logits(ifa_model *m, void *logits_shard_out_f16);
int ifa_model_tp_set_token(ifa_model *m, const int *token_dev);
/* The whole multi-GPU greedy decode from C: the segments above + the collectives of csrc/ifa_comm.hip on the worker's
 * stream, a distributed argmax over the vocabulary-sharded lm_head, token / position fed back in device memory; the step
 * is captured once as a hipGraph (tensor-parallel groups) and replayed per token.  Every rank calls it with the same
 * arguments (one host thread or process per GPU).  out_tokens_host[n_steps]: the generated ids on every rank. */
typedef struct {
    ifa_comm *tp;          /* this worker's tensor-parallel group (NULL / size 1: nothing to merge) */
    ifa_comm *world;       /* all ranks of the job: hand-over between layer groups + token broadcast (n_stages > 1) */
    int stage, n_stages;   /* BY_LAYER / HYBRID: this worker's device group, number of groups (1 = BY_TENSOR only) */
    int prev_rank, next_rank, token_src;   /* ranks in `world`; -1 = none */
    int vocab_offset;      /* first vocabulary row of this rank's lm_head shard */
    int force_collectives; /* issue the collectives even in a group of one (plumbing check on a 1-GPU box) */
} ifa_tp_topology;
int ifa_model_tp_decode(ifa_model *m, const ifa_tp_topology *topo, int first_token, int start_pos, int n_steps,
                        int *out_tokens_host, float *elapsed_ms);
/* One Infer() step of a query over the partition: n_tokens new tokens at [start_pos, start_pos + n_tokens) fed through
 * the partition: n_tokens > 1 as ONE T > 1 step (row-sliced MFMA GEMMs, [T][dim] merges after wo and w2, [T][dim]
 * hand-over between layer groups), a single token through the decode path; *next_token_host = greedy next token of the
 * last one (every rank).
 * logits_shard_out_dev (nullable; last device group): this rank's lm_head rows of every token, [n_tokens][rows] F16. */
int ifa_model_tp_prefill(ifa_model *m, const ifa_tp_topology *topo, const int *tokens_host, int n_tokens, int start_pos,
                         void *logits_shard_out_dev, int *next_token_host);
/* ifa_model_decode_batch over a tensor-parallel group (one new token for each of n queries; merges over [n][dim], one
 * distributed argmax per row); logits_shard_out_dev: optional [n][this rank's lm_head rows] F16 */
int ifa_model_tp_decode_batch(ifa_model *m, const ifa_tp_topology *topo, int n, const int *tokens_host, const int *positions_host,
                              const int *kv_slots_host, int *next_tokens_host, void *logits_shard_out_dev);
/* reference-layout copy of a loaded tensor (device pointer); returns 1 if the tensor is not set */
int ifa_model_get_tensor(ifa_model *m, int layer, int tensor_id, int *dtype, void **dptr, size_t *rows, size_t *cols);
/* the same for W1 / W2 / W3 of expert `expert` of a mixture-of-experts layer */
int ifa_model_get_expert_tensor(ifa_model *m, int layer, int expert, int tensor_id, int *dtype, void **dptr, size_t *rows, size_t *cols);
/* Average duration (HIP events on the worker's stream) of `iters` back-to-back
 * launches of one fused decode kernel, rotating over the layers' weights:
 * which = 0 qkv, 1 attention, 2 wo, 3 ffn w1/w3, 4 w2, 5 lm_head.  For bench.py's roofline. */
int ifa_model_time_kernel(ifa_model *m, int which, int iters, float *avg_us);


/* ======================================================================== */
/* Ops on 32-bit activations with bfloat16 parameters (csrc/ifa_linear_bf16.hip, ifa_ops_f32.hip, ifa_seqmix.hip,         */
/* ifa_attn_window.hip): the building blocks of the layer-list worker below, usable on their own.  Activations, the         */
/* residual stream, attention scores and every recurrent state are fp32; weights are bfloat16 bit patterns.               */
/* ======================================================================== */
/* C[t][n] (+)= alpha * mul[n] * (sum_k A[t][k] W[n][k] + bias[n]);  W bf16 [rows][cols], A fp32 [tokens][lda], C fp32 [tokens][ldc];
 * bias / mul (bf16 [rows]) nullable; accumulate != 0 adds into C (the residual update of a layer).  ops32 != 0 keeps the operands
 * of the matrix-core product in fp32 (v_mfma_f32_32x32x2_f32) instead of rounding them to bfloat16; up to 8 tokens the product is
 * a weight-streaming fp32 dot either way.  Output columns [silu_col0, silu_col1) pass SiLU right after the bias (empty range: none).
 * fp32 accumulation, no atomics: deterministic. */
int ifa_linear_bf16w(const void *w_bf16, size_t rows, size_t cols, const void *a_f32, size_t lda, size_t tokens, const void *bias_bf16,
                     const void *mul_bf16, float alpha, int accumulate, int ops32, void *c_f32, size_t ldc, int silu_col0, int silu_col1,
                     ifa_stream stream);
/* the same product for at most 8 rows (always the weight-streaming fp32 kernel) with the neighbouring element-wise op folded into the
 * read of the activations: prologue 1 = layer norm without bias, a = (x - mean) / sqrt(var + eps) * norm_w[k]; prologue 2 = gated GELU,
 * the row holds gate | up (lda >= 2 cols), a = gelu_tanh(gate[k]) * up[k]; 0 = none.  Needs cols % 8 == 0 and 16-byte aligned rows. */
int ifa_linear_bf16w_rows(int prologue, const void *norm_w_bf16, float norm_eps, const void *w_bf16, size_t rows, size_t cols, const void *a_f32,
                          size_t lda, size_t tokens, const void *bias_bf16, const void *mul_bf16, float alpha, int accumulate, void *c_f32,
                          size_t ldc, int silu_col0, int silu_col1, ifa_stream stream);
/* Grouped product on the matrix cores: `groups` matrices [rows][cols] back to back in w_bf16; the output rows are sorted by group and cut
 * into tiles of at most 64 rows of ONE group: tile_map_dev[3 i] = {group, first row, rows}, *n_tiles_dev tiles (max_tiles < 65536 bounds
 * the grid).  C[r][n] = row_scale[r] * act(sum_k A[a_rows[r]][k] W_group[n][k]); a_rows_dev / row_scale_f32 nullable; act 0 none, 1 erf-GELU. */
int ifa_linear_bf16w_grouped(const void *w_bf16, size_t rows, size_t cols, int groups, const void *a_f32, size_t lda, const int *a_rows_dev,
                             const int *tile_map_dev, const int *n_tiles_dev, size_t max_tiles, const void *row_scale_f32, int act, int ops32,
                             void *c_f32, size_t ldc, ifa_stream stream);
/* x[t] = embed[token_t] + pe(pos_t), pe[2i] = sin(p base^(-2i/width)), pe[2i+1] = cos(same); angles formed in double */
int ifa_embed_sinpos_f32(const void *embed_bf16, int vocab, int width, const int *tokens_dev, const int *positions_dev, size_t tokens,
                         float base, void *x_f32, ifa_stream stream);
/* kind 0: RMS norm x / sqrt(mean(x^2) + eps) * w; kind 1: layer norm without bias (x - mean) / sqrt(var + eps) * w; w bf16 nullable */
int ifa_layernorm_f32(int kind, const void *x_f32, size_t ldx, size_t rows, size_t cols, const void *w_bf16, float eps, void *y_f32, size_t ldy,
                      ifa_stream stream);
/* out[t][c] = act(gu[t][c]) * gu[t][cols + c]; kind 0 silu, 1 gelu (tanh form), 2 relu */
int ifa_glu_f32(int kind, const void *gate_up_f32, size_t ld, size_t rows, size_t cols, void *out_f32, size_t ldo, ifa_stream stream);
/* greedy argmax per row (lowest index on ties); excluded_dev = {count <= 3, id, id, id} nullable */
int ifa_argmax_rows_f32(const void *logits_f32, size_t n, size_t row_stride, size_t rows, const int *excluded_dev, int *out_dev, ifa_stream stream);
int ifa_convert_f32_f16(const void *src_f32, size_t n, void *dst_f16, ifa_stream stream);

/* A step's rows are described by sequences: rows [row0, row0 + n) are positions [pos0, pos0 + n) of the sequence whose cache and
 * state live in slot `slot`; row_seq_dev[row] = index of the row's sequence.  slot_base_dev[slot] = base pointer (fp32) of the
 * slot's arena; *_off = offset in floats of a layer's part.  A sequence at pos0 == 0 starts from zero state whatever the slot holds. */
typedef struct { int row0, n, pos0, slot; } ifa_seq_desc;
/* short causal convolution per channel (w bf16 [channels][taps], last tap = current token) + SiLU; the last taps - 1 inputs of a
 * sequence are carried in its slot ([taps - 1][channels]; ifa_shortconv_tail_f32 advances them AFTER the step's rows are computed).
 * Then channels [0, norm_cols) become unit vectors in groups of group_dim (x / sqrt(sum x^2 + l2_eps)) and channels [0, scale_cols)
 * are multiplied by scale. */
int ifa_shortconv_silu_f32(const void *x_f32, size_t ldx, int channels, int taps, const void *w_bf16, const void *seqs_dev, const int *row_seq_dev,
                           size_t rows, void *const *slot_base_dev, size_t state_off, int norm_cols, int group_dim, float l2_eps, int scale_cols,
                           float scale, void *y_f32, size_t ldy, ifa_stream stream);
int ifa_shortconv_tail_f32(const void *x_f32, size_t ldx, int channels, int taps, const void *seqs_dev, int n_seqs, void *const *slot_base_dev,
                           size_t state_off, ifa_stream stream);
/* gates of the gated delta rule: beta = sigmoid(b), decay = exp(-exp(A_log[h]) * softplus(a + dt_bias[h])); outputs fp32 [rows][heads] */
int ifa_delta_gates_f32(const void *b_f32, size_t ldb, const void *a_f32, size_t lda, int heads, size_t rows, const void *a_log_bf16,
                        const void *dt_bias_bf16, void *beta_f32, void *decay_f32, ifa_stream stream);
/* per-head matrix state S [dk][dv] (fp32, in the slot: [heads][dk][dv]) advanced token by token;
 * kind 0: S <- d_h S + k v^T, o = S^T q (decay_head_f32 [heads]); kind 1 (gated delta rule): S <- g S; u = beta (v - S^T k);
 * S <- S + k u^T; o = S^T q (decay_row / beta_row fp32 [rows][heads]).  Head h reads q / k head h / (heads / qk_heads).
 * in_act != 0: q, k, v pass SiLU as they are read.  dk <= 256. */
int ifa_state_scan_f32(int kind, int in_act, const void *q_f32, size_t ldq, const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int heads,
                       int qk_heads, int dk, int dv, const void *decay_head_f32, const void *decay_row_f32, const void *beta_row_f32,
                       const void *seqs_dev, int n_seqs, void *const *slot_base_dev, size_t state_off, void *out_f32, size_t ldo, ifa_stream stream);
/* y = o / sqrt(mean_group(o^2) + eps) * w[c % wlen] * act(gate); gate_act 0 sigmoid, 1 silu; groups of `group` channels; y may be o */
int ifa_gated_groupnorm_f32(const void *o_f32, size_t ldo, size_t rows, int channels, int group, const void *w_bf16, int wlen, const void *gate_f32,
                            size_t ldg, int gate_act, float eps, void *y_f32, size_t ldy, ifa_stream stream);
/* rows of a step into the fp32 K / V cache of their sequences ([max_ctx][kv_heads * dim] each): K = k / rms_head(k) if norm_k, V = v */
int ifa_kv_store_f32(const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int kv_heads, int dim, int norm_k, float eps, const void *seqs_dev,
                     const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off, ifa_stream stream);
/* softmax attention of the step's rows over their sequences' caches: query i sees key j iff j <= i and (i - j < window or
 * j < keep_first); q RMS-normed per head if norm_q; score = q.k * scale, soft cap cap * tanh(score / cap) if softcap > 0, + bias
 * rel[bucket_of[i - j]][head] if rel (bf16 [n_buckets][heads], bucket_of_dev: int per distance 0 .. max_ctx - 1); sink_bf16 [heads]
 * (nullable): exp(sink) joins the denominator.  dim <= 1024.  out fp32 [rows][heads * dim].
 * Steps of at least tile_min_rows rows (head sizes 32 / 64 / 96 / 128) take the tiled kernel -- 128 queries of one sequence per workgroup,
 * scores and weighted sums on the fp32 matrix cores -- which needs the step's sequences on the host too (seqs_host [n_seqs], the same
 * values as seqs_dev; NULL / n_seqs 0: always one workgroup per row).  With a workspace (ws_f32, ws_bytes; nullable) and at most 512
 * (row, head) pairs, the keys of a pair are shared out to up to 32 workgroups (64 keys each) and merged by a second launch (decode steps). */
int ifa_attention_window_f32(const void *q_f32, size_t ldq, int heads, int kv_heads, int dim, int norm_q, float eps, float scale, float softcap,
                             int window, int keep_first, const void *rel_bf16, const int *bucket_of_dev, int n_buckets, const void *sink_bf16,
                             const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off,
                             void *out_f32, size_t ldo, const void *seqs_host, int n_seqs, int tile_min_rows, void *ws_f32, size_t ws_bytes, ifa_stream stream);

/* The same attention over caches whose keys have been normed and rotated by ifa_qk_rope_store_f32: key rows [max_ctx][kv_heads * dim]
 * at k_off, value rows [max_ctx][kv_heads * vdim] at v_off (they may be another layer's); window 0: every earlier position; sink != 0:
 * exp(sink_score) joins the denominator of every head; no norm, cap or bias inside.  The tiled kernel takes heads of up to 128
 * dimensions of any size (zero-padded to whole 32s in LDS); max_keys (0: unknown) bounds the keys a row can see, for sharing them out. */
int ifa_attention_kv_f32(const void *q_f32, size_t ldq, int heads, int kv_heads, int dim, int vdim, float scale, int window, int keep_first, int sink,
                         float sink_score, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off,
                         void *out_f32, size_t ldo, const void *seqs_host, int n_seqs, int tile_min_rows, int max_keys, void *ws_f32, size_t ws_bytes,
                         ifa_stream stream);
/* rows of a step: per head RMS norm over dim with a weight (bf16 [dim], shared by the heads; null: no norm), then rotation of the first
 * rot_dims dimensions, dimension i paired with i + rot_dims / 2: (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = pos * freq[i]
 * (freq_f64_dev: double [rot_dims / 2], angles formed in double).  Query heads are rewritten in place; key heads go to the K rows of
 * the sequences' caches, the values as they are to the V rows.  k_f32 null: queries only.  dim <= 1024. */
int ifa_qk_rope_store_f32(void *q_f32, size_t ldq, int heads, const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int kv_heads, int dim, int vdim,
                          const void *q_norm_w_bf16, const void *k_norm_w_bf16, float eps, int rot_dims, const double *freq_f64_dev, const void *seqs_dev,
                          const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off, ifa_stream stream);

/* x[t] = embed[token_t] + pair[(prev_t * mul_prev + token_t * mul_cur) mod buckets] (pair_bf16 [buckets + 1][width]; null: no second
 * term); a sequence's first token (position 0) takes row `buckets`.  prev_t is the row before in the step, or, for the first row of a
 * sequence that continues, the token its slot holds (one int at state_off); the sequence's last token of the step is left there. */
int ifa_embed_pair_f32(const void *embed_bf16, int vocab, int width, const void *pair_bf16, int buckets, int mul_prev, int mul_cur, const int *tokens_dev,
                       const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t state_off, void *x_f32,
                       ifa_stream stream);
/* RMS norm whose stored weight is the offset from w_offset: y (+)= x / sqrt(mean(x^2) + eps) * (w_offset + w[c]); accumulate != 0 adds into y (the
 * residual update behind a sub-layer; y must not be x then) */
int ifa_rmsnorm_offset_f32(const void *x_f32, size_t ldx, size_t rows, size_t cols, const void *w_bf16, float w_offset, float eps, int accumulate,
                           void *y_f32, size_t ldy, ifa_stream stream);
/* both norms between two sub-layers in one launch: x += m / rms(m) * (w_offset + w_after[c]), then (w_before_bf16 not null)
 * h = x / rms(x) * (w_offset + w_before[c]) */
int ifa_norm_add_norm_f32(void *x_f32, size_t ldx, size_t rows, size_t cols, const void *m_f32, size_t ldm, const void *w_after_bf16,
                          const void *w_before_bf16, float w_offset, float eps, void *h_f32, size_t ldh, ifa_stream stream);
/* out[t][c] = f(gu[t][c], gu[t][cols + c]) * (row_gate ? sigmoid(row_gate[t * ldg]) : 1); kind 0 / 1 / 2 as ifa_glu_f32, kind 3:
 * g = min(gate, limit), u = clamp(up, -limit, limit), f = g * sigmoid(1.702 g) * (u + 1) */
int ifa_glu_ex_f32(int kind, float limit, const void *gate_up_f32, size_t ld, size_t rows, size_t cols, const void *row_gate_f32, size_t ldg,
                   void *out_f32, size_t ldo, ifa_stream stream);

/* x[t] = embed[token_t] (bf16 rows) as fp32, no position vector */
int ifa_embed_rows_f32(const void *embed_bf16, int vocab, int width, const int *tokens_dev, size_t tokens, void *x_f32, ifa_stream stream);
/* RMS norm in `groups` equal consecutive parts of a row: y = x / sqrt(mean_part(x^2) + eps) * w[c]; accumulate != 0: y += that (the
 * residual update of a block whose norm sits on the sub-layer's OUTPUT).  cols % groups == 0; y may be x when accumulate == 0. */
int ifa_group_rmsnorm_f32(const void *x_f32, size_t ldx, size_t rows, size_t cols, int groups, const void *w_bf16, float eps, int accumulate,
                          void *y_f32, size_t ldy, ifa_stream stream);
/* y = x + conv(x): causal convolution over time on each channel WITHOUT activation (w bf16 [channels][taps], last tap = current token),
 * the last taps - 1 inputs carried in the slot like ifa_shortconv_silu_f32's (ifa_shortconv_tail_f32 advances them afterwards) */
int ifa_shortconv_residual_f32(const void *x_f32, size_t ldx, int channels, int taps, const void *w_bf16, const void *seqs_dev, const int *row_seq_dev,
                               size_t rows, void *const *slot_base_dev, size_t state_off, void *y_f32, size_t ldy, ifa_stream stream);
/* Steps of a few rows (<= 64; a workgroup per norm part): what lies between two sub-layers of a post-norm block in ONE launch, every part optional:
 * x[t] += group_rms_norm(m[t]) * norm_w (m null: skip); depth average as ifa_depth_average_f32 (stack null: skip); h = x + conv(x) with the
 * carried tail read and then advanced, as ifa_shortconv_residual_f32 + ifa_shortconv_tail_f32 (conv_w null: skip).  x is rows x cols, contiguous. */
int ifa_norm_add_conv_rows_f32(void *x_f32, size_t rows, size_t cols, const void *m_f32, size_t ldm, const void *norm_w_bf16, int groups, float eps,
                               void *stack_f32, size_t plane_stride, int count, const void *depth_w_bf16, const void *conv_w_bf16, int taps,
                               const void *seqs_dev, int n_seqs, const int *row_seq_dev, void *const *slot_base_dev, size_t state_off, void *h_f32,
                               ifa_stream stream);
/* depth average: stack[count - 1] <- x (rows x cols, contiguous), then x <- sum_j w[j] stack[j], j < count; stack planes are
 * plane_stride floats apart; w bf16 [count] */
int ifa_depth_average_f32(void *x_f32, size_t rows, size_t cols, void *stack_f32, size_t plane_stride, int count, const void *w_bf16, ifa_stream stream);
/* x <- cap * tanh(x / cap) over n contiguous values */
int ifa_softcap_f32(void *x_f32, size_t n, float cap, ifa_stream stream);

/* ---- latent attention (csrc/ifa_attn_latent.hip): the cache of a layer holds ONE row per position, [kv_rank latent | rot_dim rotated key
 * part] fp32, shared by all heads; keys and values of a head are linear maps of the latent (w_uk [heads * dim][kv_rank],
 * w_uv [heads * vdim][kv_rank], bf16).  A query head is [dim unrotated | rot_dim rotated]; score = (q_u . W_uk c + q_r . k_r) * scale.
 * Rotation: interleaved pairs (2i, 2i + 1) of the first rot_dims dimensions of the rotated part by angle pos * freq[i]
 * (freq_f64_dev: double [rot_dims / 2], angles formed in double), cos and sin multiplied by rot_mult. */
/* rows of a step: c = rms(kv[:kv_rank]) * c_norm_w and the rotated key part into the cache; the rotated part of every query head in place */
int ifa_latent_prepare_f32(const void *kv_f32, size_t ldkv, int kv_rank, int rot_dim, int rot_dims, const void *c_norm_w_bf16, float eps,
                           void *q_f32, size_t ldq, int heads, int dim, const double *freq_f64_dev, float rot_mult, const void *seqs_dev,
                           const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t cache_off, ifa_stream stream);
/* absorbed query: qa[t][h] = [W_uk[h]^T q_u[t][h] (kv_rank) | q_r[t][h] (rot_dim)]: a query against the cache rows themselves */
int ifa_latent_absorb_q_f32(const void *q_f32, size_t ldq, int heads, int dim, int rot_dim, int kv_rank, const void *w_uk_bf16, size_t rows,
                            void *qa_f32, size_t ldqa, ifa_stream stream);
/* single tokens: softmax attention of the absorbed queries over the cache rows of their sequences (keys: the whole row, values: its first
 * kv_rank floats; causal); four heads share one read of the keys; the keys of a row are shared out to up to 64 workgroups per head group
 * (max_keys = the longest sequence the cache holds sizes the shares) whose partial results go through ws_f32 (rows * heads * shares *
 * (kv_rank + 2) floats at most).  kv_rank <= 1024.  out fp32 [rows][heads * kv_rank]. */
int ifa_attention_latent_rows_f32(const void *qa_f32, size_t ldqa, int heads, int kv_rank, int rot_dim, float scale, const void *seqs_dev,
                                  const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t cache_off, int max_keys, void *ws_f32,
                                  size_t ws_bytes, void *out_f32, size_t ldo, ifa_stream stream);
/* asks ahead for the LDS the single-token kernel needs for this row shape (beyond 48 KB it has to be granted once per kernel): call it
 * before a step that may be captured into a graph, where the grant cannot be asked for */
int ifa_attention_latent_rows_reserve(int kv_rank, int rot_dim);
/* out[t][h * vdim + e] = gate[t][h] * sum_r w_uv[h * vdim + e][r] * ol[t][h * ld_head + r]; gate = sigmoid(g[t][h]) or 1 (g null) */
int ifa_latent_expand_out_f32(const void *ol_f32, size_t ldol, int ld_head, int heads, int vdim, int kv_rank, const void *w_uv_bf16,
                              const void *g_f32, size_t ldg, size_t rows, void *out_f32, size_t ldo, ifa_stream stream);
/* prompts: causal softmax attention of the step's rows with per-head keys [kx (dim, expanded: kx_f32 [ctx rows][heads * dim]) | rotated
 * part from the cache rows] and values vx_f32 [ctx rows][heads * vdim]; ctx0_dev[s] / seqs_host: first expanded row of sequence s (its
 * position 0).  128 queries of one sequence per workgroup on the fp32 matrix cores, online softmax in fp32. */
int ifa_attention_latent_tile_f32(const void *q_f32, size_t ldq, int heads, int dim, int rot_dim, int vdim, int kv_rank, float scale,
                                  const void *kx_f32, size_t ldkx, const void *vx_f32, size_t ldvx, const int *ctx0_dev, const void *g_f32, size_t ldg,
                                  const void *seqs_dev, const void *seqs_host, int n_seqs, void *const *slot_base_dev, size_t cache_off,
                                  void *out_f32, size_t ldo, ifa_stream stream);
/* 1 if the tiled kernel serves these head sizes (keys up to 192, values up to 128 dimensions, within the LDS) */
int ifa_attention_latent_tile_fits(int dim, int rot_dim, int vdim);

/* ---- mixture of experts (csrc/ifa_moe_f32.hip): `experts` feed-forward experts down(act(up h)) without biases (up bf16
 * [experts][ff][width], down bf16 [experts][width][ff]) + `identity` experts whose output is h itself.  Router: scores = softmax of the
 * logits over experts + identity; the `top` largest (score + correction) are chosen (lowest index on ties); weights = their scores,
 * not renormalized.  idx_dev / wgt_dev: [rows][top]. */
int ifa_moe_route_f32(const void *logits_f32, size_t ld, size_t rows, int n_all, int top, const void *correction_bf16, int *idx_dev, void *wgt_f32,
                      ifa_stream stream);
/* the same for steps of at most 64 rows with the router's product (router_bf16 [n_all][width], fp32 dots) inside the launch */
int ifa_moe_route_rows_f32(const void *h_f32, size_t ldh, size_t rows, int width, const void *router_bf16, int n_all, int top, const void *correction_bf16,
                           int *idx_dev, void *wgt_f32, ifa_stream stream);
/* y[t] (+)= sum_k wgt[t][k] * expert_{idx[t][k]}(h[t]); act 0: exact (erf) GELU.  Rows are served by expert: few rows stream each chosen
 * expert's weights per row; many rows are sorted by expert and run as grouped matrix-core products (ops32 as in ifa_linear_bf16w).
 * ws: workspace of ifa_moe_workspace_bytes(rows, top, width, ff, experts) bytes.  Deterministic: no atomics on values. */
size_t ifa_moe_workspace_bytes(size_t rows, int top, int width, int ff, int experts);
int ifa_moe_experts_f32(const void *h_f32, size_t ldh, size_t rows, int width, int ff, int experts, int identity, int top, int act,
                        const void *up_bf16, const void *down_bf16, const int *idx_dev, const void *wgt_f32, int ops32, void *ws, size_t ws_bytes,
                        void *y_f32, size_t ldy, int accumulate, ifa_stream stream);

/* Router of the second kind: the `top` largest (logit + bias) are chosen (lowest index on ties; bias bf16 [n_all], nullable) and their
 * weights are the softmax over the chosen values only. */
int ifa_moe_route_top_f32(const void *logits_f32, size_t ld, size_t rows, int n_all, int top, const void *bias_bf16, int *idx_dev, void *wgt_f32,
                          ifa_stream stream);
/* Gated experts: E_e(h) = W_down[e] (silu(W_gate[e] h) * (W_up[e] h)); gate_up bf16 [experts][gate ff | up ff][width], down bf16
 * [experts][width][ff]; otherwise as ifa_moe_experts_f32 (workspace: ifa_moe_workspace_bytes(rows, top, width, 3 * ff, experts)). */
int ifa_moe_experts_gated_f32(const void *h_f32, size_t ldh, size_t rows, int width, int ff, int experts, int top, const void *gate_up_bf16,
                              const void *down_bf16, const int *idx_dev, const void *wgt_f32, int ops32, void *ws, size_t ws_bytes, void *y_f32, size_t ldy,
                              int accumulate, ifa_stream stream);


/* ---- ops of pre-norm blocks with element-wise norms, looped layer groups, rotated values and per-channel recurrences */
/* Dynamic Tanh "norm": y[t][c] = tanh(alpha * x[t][c]) * w[c] + b[c]; alpha_bf16 one value, w / b bf16 [cols]; no mean, no variance */
int ifa_dyt_f32(const void *x_f32, size_t ldx, size_t rows, size_t cols, const void *alpha_bf16, const void *w_bf16, const void *b_bf16, void *y_f32,
                size_t ldy, ifa_stream stream);
/* a residual update (behind a sub-layer, or at the start of a looped pass) and the Dynamic Tanh in front of the next sub-layer in one launch:
 * x[t][c] += m[t][c] + vec[c] (either nullable), then (w not null) h = tanh(alpha x) w + b */
int ifa_add_dyt_f32(void *x_f32, size_t ldx, size_t rows, size_t cols, const void *m_f32, size_t ldm, const void *vec_bf16, const void *alpha_bf16, const void *w_bf16,
                    const void *b_bf16, void *h_f32, size_t ldh, ifa_stream stream);
/* x[t][c] += (add_f32 ? add[t][c] : 0) + (vec_bf16 ? vec[c] : 0): what a pass of a looped layer group starts from */
int ifa_add_rows_vec_f32(void *x_f32, size_t ldx, size_t rows, size_t cols, const void *add_f32, size_t lda, const void *vec_bf16, ifa_stream stream);
/* ifa_embed_pair_f32 with the token embedding multiplied by embed_scale (the pair row is not) and an optional second copy of the result */
int ifa_embed_pair_scaled_f32(const void *embed_bf16, int vocab, int width, float embed_scale, const void *pair_bf16, int buckets, int mul_prev, int mul_cur,
                              const int *tokens_dev, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t state_off,
                              void *x_f32, void *x_copy_f32, ifa_stream stream);
/* ifa_qk_rope_store_f32 whose values are treated too before they enter the V rows: v_norm != 0: each value head is divided by its root
 * mean square (eps, no weight); v_freq_f64_dev != null: the value head of position j then turns by j over ALL vdim dimensions, pair
 * (m, m + vdim / 2) by j * v_freq[m] (double [vdim / 2]; vdim even). */
int ifa_qkv_rope_store_f32(void *q_f32, size_t ldq, int heads, const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int kv_heads, int dim, int vdim,
                           const void *q_norm_w_bf16, const void *k_norm_w_bf16, float eps, int rot_dims, const double *freq_f64_dev, int v_norm,
                           const double *v_freq_f64_dev, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off,
                           size_t v_off, ifa_stream stream);
/* heads of a step's rows turned in place by sign * position: pair (m, m + rot_dims / 2) of the first rot_dims dimensions of every head by
 * sign * pos * freq[m] (angles in double).  sign -1 turns an attention output over rotated values back. */
int ifa_rotate_heads_f32(void *x_f32, size_t ldx, int heads, int dim, int rot_dims, const double *freq_f64_dev, float sign, const void *seqs_dev,
                         const int *row_seq_dev, size_t rows, ifa_stream stream);
/* ifa_attention_kv_f32 with a learned sink per head (sink_bf16 [heads]; null: none): exp(sink_h) joins the denominator */
int ifa_attention_kv_sinks_f32(const void *q_f32, size_t ldq, int heads, int kv_heads, int dim, int vdim, float scale, int window, int keep_first,
                               const void *sink_bf16, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off,
                               size_t v_off, void *out_f32, size_t ldo, const void *seqs_host, int n_seqs, int tile_min_rows, int max_keys, void *ws_f32,
                               size_t ws_bytes, ifa_stream stream);
/* gates of the generalized delta rule, per row and key channel c of heads * dim: decay[c] = exp(-decay_mult * sigmoid(w2[c] . tanh(lr) + w0[c]))
 * (lr fp32 [rows][rank]: the bottleneck's pre-activations; w2 bf16 [heads * dim][rank]; w0 bf16 [heads * dim], nullable), unit key
 * u = k / sqrt(sum_head(k^2) + l2_eps), removal[c] = sigmoid(a[c]) * u[c] (a with its bias already added).  Outputs fp32 [rows][heads * dim], contiguous.
 * rank 0: lr_f32 holds the sigmoid's argument itself, [rows][heads * dim] (w2 / w0 unused): larger steps form it as a matrix product over
 * ifa_tanh_f32 of the bottleneck. */
int ifa_chan_delta_gates_f32(const void *lr_f32, size_t ldl, int rank, const void *w2_bf16, const void *w0_bf16, float decay_mult, const void *a_f32, size_t lda,
                             const void *k_f32, size_t ldk, int heads, int dim, float l2_eps, size_t rows, void *decay_f32, void *unit_f32, void *removal_f32,
                             ifa_stream stream);
/* x[t][c] = tanh(x[t][c]) in place, c < cols */
int ifa_tanh_f32(void *x_f32, size_t ldx, size_t rows, size_t cols, ifa_stream stream);
/* generalized delta rule with a decay and a removal rate per key channel: per head, S [dk][dv] fp32 in the slot,
 * S <- diag(decay_t) S - removal_t (unit_t^T S) + k_t v_t^T (both terms read the old state), o_t = S^T q_t.
 * decay / unit / removal fp32 [rows][heads * dk] (row stride ldg).  dk <= 256. */
int ifa_state_scan_chan_f32(const void *q_f32, size_t ldq, const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int heads, int dk, int dv,
                            const void *decay_f32, const void *unit_f32, const void *removal_f32, size_t ldg, const void *seqs_dev, int n_seqs,
                            void *const *slot_base_dev, size_t state_off, void *out_f32, size_t ldo, ifa_stream stream);
/* Router with a choice of scores: score_kind 0 = softmax over all (ifa_moe_route_f32), 1 = sigmoid of each logit; the `top` largest
 * (score + correction) are chosen (lowest index on ties), weights = their plain scores, not renormalized */
int ifa_moe_route_scores_f32(int score_kind, const void *logits_f32, size_t ld, size_t rows, int n_all, int top, const void *correction_bf16, int *idx_dev,
                             void *wgt_f32, ifa_stream stream);
int ifa_moe_route_rows_scores_f32(int score_kind, const void *h_f32, size_t ldh, size_t rows, int width, const void *router_bf16, int n_all, int top,
                                  const void *correction_bf16, int *idx_dev, void *wgt_f32, ifa_stream stream);
/* the same with the Dynamic Tanh norm in front of the router inside the launch: h[t] = tanh(alpha x[t]) w + b is written (the experts read it), then routed */
int ifa_moe_dyt_route_rows_f32(int score_kind, const void *x_f32, size_t ldx, const void *alpha_bf16, const void *norm_w_bf16, const void *norm_b_bf16, void *h_f32,
                               size_t ldh, size_t rows, int width, const void *router_bf16, int n_all, int top, const void *correction_bf16, int *idx_dev,
                               void *wgt_f32, ifa_stream stream);
/* Gated experts with a choice of the gate: glu_kind 0 = silu(gate) * up (ifa_moe_experts_gated_f32), 3 = the clamped form of ifa_glu_ex_f32
 * (g = min(gate, limit), u = clamp(up, +-limit), g sigmoid(1.702 g) (u + 1)) */
int ifa_moe_experts_glu_f32(int glu_kind, float limit, const void *h_f32, size_t ldh, size_t rows, int width, int ff, int experts, int top,
                            const void *gate_up_bf16, const void *down_bf16, const int *idx_dev, const void *wgt_f32, int ops32, void *ws, size_t ws_bytes,
                            void *y_f32, size_t ldy, int accumulate, ifa_stream stream);

/* ======================================================================== */
/* Layer-list worker: a decoder whose layers are given one by one, each with its own sequence mixer, a 32-bit residual       */
/* stream and bfloat16 weights (csrc/ifa_engine_layered.hip).  It is an ifa_model: finalize / kv_slots / select_kv /        */
/* forward / decode / decode_batch / set_option / set_excluded_tokens / get_buffer / destroy work as above (a "KV slot" holds */
/* the key / value rows AND the recurrent states of one query); the tensor-parallel entry points decline.                   */
/* A layer: h = norm1(x); x <- x + ls1 * mixer(h) + ls2 * ffn(h)  (one norm, both sub-layers read it).                      */
/* ======================================================================== */
enum { IFA_MIX_WINDOW_LINEAR = 1,   /* windowed softmax attention (values = keys as projected) + decayed linear attention, side by side */
       IFA_MIX_GATED_DELTA = 2,     /* gated delta rule behind short convolutions */
       IFA_MIX_LATENT = 3,          /* latent attention: one compressed key / value row per position, a rotated key part shared by all heads */
       IFA_MIX_ROTARY = 4,          /* softmax attention with rotated queries / keys: grouped queries, q | k | v projections with biases, weighted
                                     * RMS norm of q and k per head, rotation of the first a_rot_dims dimensions (pairs i, i + a_rot_dims / 2),
                                     * values of their own size, optional sink (fixed score or learned per head), optional window, keys / values
                                     * of an earlier layer, optionally scaled frequencies, normed values, rotated values */
       IFA_MIX_CHAN_DELTA = 5 };    /* generalized delta rule: decay and removal rate per head and key channel (the decay through a small
                                     * two-matrix bottleneck), unit keys for the removal, per-head RMS norm x weight x sigmoid gate on the output */
/* wiring of a layer.  PARALLEL: h = norm1(x); x <- x + ls1 * mixer(h) + ls2 * ffn(h).  POSTNORM: the sub-layers read x itself (plus a
 * short causal convolution of x when canon_taps > 0) and the grouped RMS norm sits on their OUTPUT: x <- x + norm1(mixer(x'));
 * x <- x + norm2(ffn(x')); with depth_avg the next layer reads sum_j dwa[j] X_j over the embedding output X_0 and every layer result.
 * SANDWICH: an RMS norm with weight (1 + w) before AND after each sub-layer: x <- x + norm1b(mixer(norm1(x))); x <- x + norm2b(ffn(norm2(x))).
 * PRENORM: x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x)) with Dynamic Tanh norms tanh(alpha x) w + b (tensors IFA_LT_NORM1 / _B / _ALPHA). */
enum { IFA_BLOCK_PARALLEL = 0, IFA_BLOCK_POSTNORM = 1, IFA_BLOCK_SANDWICH = 2, IFA_BLOCK_PRENORM = 3 };
enum { IFA_FFN_GATED = 0,           /* gated feed-forward (GELU tanh, biases), width `ffn` */
       IFA_FFN_MOE = 1,             /* mixture of experts: x_experts experts of width x_ff + x_identity identity experts, x_top per token */
       IFA_FFN_CLAMPED = 2 };       /* width `ffn`, no biases: g = min(gate, f_limit), u = clamp(up, +-f_limit), y = down(g sigmoid(1.702 g) (u + 1)) */
typedef struct {
    int mixer;                       /* IFA_MIX_* */
    int ffn;                         /* width of the gated feed-forward (GELU tanh, biases); 0 = none */
    /* windowed attention */
    int a_heads, a_kv_heads, a_dim, a_window, a_keep_first, a_buckets, a_bias_max;
    float a_scale, a_softcap, a_out_scale;
    /* decayed linear attention (decays: tensor IFA_LT_L_DECAY) */
    int l_heads, l_dim, l_vdim;
    float l_out_scale;
    /* gated delta rule */
    int d_heads, d_kv_heads, d_dim, d_vdim, d_conv;
    /* wiring (IFA_BLOCK_*), taps of the input convolution of both sub-layers (0: none), depth average on / off */
    int block, canon_taps, depth_avg;
    /* latent attention: heads of [m_dim unrotated | m_rot_dim rotated] query / key dimensions, values of m_vdim, latent of m_kv_rank;
     * m_q_rank > 0: the queries go through an RMS-normed latent of that size; m_gate: a sigmoid gate per head on the output;
     * the first m_rot_dims dimensions of the rotated part turn with base m_rot_base; m_yarn_factor > 0: YaRN frequency scaling */
    int m_heads, m_dim, m_rot_dim, m_vdim, m_kv_rank, m_q_rank, m_gate, m_rot_dims;
    float m_scale, m_rot_base, m_yarn_factor, m_yarn_original, m_yarn_fast, m_yarn_slow;
    /* feed-forward kind (IFA_FFN_*) and the mixture's sizes */
    int ffn_kind, x_experts, x_identity, x_top, x_ff;
    /* IFA_MIX_ROTARY (with a_heads, a_kv_heads, a_dim, a_scale; a_window 0 = every earlier position, a_keep_first): size of a value head,
     * rotated dimensions (even, <= a_dim) and their base, a_sink 1: a sink of score a_sink_score joins the softmax's denominator,
     * a_kv_layer: 0 = keys and values of its own, j + 1 = the cache rows of layer j (an earlier IFA_MIX_ROTARY layer with projections of
     * its own and the same a_kv_heads / a_dim / a_vdim): then the layer has no k / v tensors */
    int a_vdim, a_rot_dims, a_sink, a_kv_layer;
    float a_rot_base, a_sink_score;
    /* IFA_FFN_CLAMPED: the limit.  Mixture: x_gated 1 = experts down(silu(gate h) * (up h)) (IFA_LT_X_UP holds [gate rows | up rows] per
     * expert); x_route 0 = softmax over all, choice by score + correction, weights = scores; 1 = choice by logit + bias, weights = softmax
     * over the chosen logits; x_shared_ff > 0: a shared gated expert of that width for every row, times sigmoid(w_sg . h) */
    float f_limit;
    int x_gated, x_route, x_shared_ff;
    /* more of IFA_MIX_ROTARY.  a_sink 2: a learned sink per head (tensor IFA_LT_A_SINK).  a_rot_scale_factor > 0: frequencies scaled by
     * wavelength l = 2 pi / f: kept where l < original / high, f / factor where l > original / low, blended linearly in
     * (original / l - low) / (high - low) between.  a_vnorm 1: value heads divided by their root mean square before they are cached.
     * a_vrot 1: the value of position j enters the cache turned by j over all a_vdim dimensions (pairs m, m + a_vdim / 2, frequency
     * a_rot_base^(-2m / a_vdim), never scaled) and the head's output at position i is turned back by -i. */
    float a_rot_scale_factor, a_rot_scale_low, a_rot_scale_high, a_rot_scale_original;
    int a_vnorm, a_vrot;
    /* IFA_MIX_CHAN_DELTA: c_heads heads of c_dim key and value channels, bottleneck of c_rank for the decay; decay = exp(-c_decay_mult *
     * sigmoid(.)); eps inside the root of the unit key */
    int c_heads, c_dim, c_rank;
    float c_decay_mult, c_l2_eps;
    /* mixture: x_score 0 softmax over all, 1 sigmoid per expert (x_route 0); x_glu 0 silu(gate) * up, 3 the clamped form with x_limit (x_gated 1) */
    int x_score, x_glu;
    float x_limit;
} ifa_layer_spec;
typedef struct {
    int width, vocab, max_ctx, n_layers, device;
    int ops32;                       /* 1: matrix products keep fp32 operands (exact mode); 0: operands rounded to bfloat16 */
    float eps, pos_base;             /* eps of every norm of the stack; base of the sinusoidal position vector (10000) */
    int stem;                        /* 0: embedding + sinusoidal position vector, layer norm before lm_head; 1: embedding through a grouped RMS
                                      * norm (IFA_T_EMBD_NORM), grouped RMS norm before lm_head, no position vector */
    int norm_groups;                 /* parts of the grouped RMS norms (stem 1 and POSTNORM layers) */
    float logit_softcap;             /* > 0: logits <- cap * tanh(logits / cap) */
    /* stem 2: embedding + hashed token-pair embedding (IFA_T_BIGRAM row (prev * bigram_mul_prev + token * bigram_mul_cur) mod
     * bigram_buckets; row bigram_buckets for a sequence's first token; bigram_buckets 0: none), no position vector, RMS norm with
     * weight (1 + w) before lm_head.  The previous token of a sequence is kept in its slot. */
    int bigram_buckets, bigram_mul_prev, bigram_mul_cur;
    /* stem 3: stem 2 with the token embedding times embed_scale (0: 1), a Dynamic Tanh norm before lm_head (IFA_T_OUT_NORM / _B / _ALPHA)
     * and logits times logit_scale (0: 1) */
    float embed_scale, logit_scale;
    /* looped layer group: layers [loop_start, loop_stop) run loop_times times in a row with the same weights, each pass on cache rows and
     * states of its own; before every pass but the first the embedding output is added to the residual, and before every pass row t of
     * IFA_T_LOOP_STEP ([loop_times][width]).  loop_times 0: no group. */
    int loop_start, loop_stop, loop_times;
} ifa_layered_config;
/* tensors of a layer-list model (global ones use IFA_T_EMBD / IFA_T_OUT_NORM / IFA_T_LM_HEAD with layer = -1) */
enum {
    IFA_LT_NORM1 = 40, IFA_LT_LS1, IFA_LT_LS2, IFA_LT_FFN_GATE, IFA_LT_FFN_GATE_B, IFA_LT_FFN_UP, IFA_LT_FFN_UP_B, IFA_LT_FFN_DOWN, IFA_LT_FFN_DOWN_B,
    IFA_LT_A_Q, IFA_LT_A_K, IFA_LT_A_REL, IFA_LT_A_SINK, IFA_LT_A_O,
    IFA_LT_L_Q, IFA_LT_L_K, IFA_LT_L_V, IFA_LT_L_G, IFA_LT_L_O, IFA_LT_L_NORM, IFA_LT_L_DECAY /* fp32 [heads] */,
    IFA_LT_D_Q, IFA_LT_D_K, IFA_LT_D_V, IFA_LT_D_QCONV, IFA_LT_D_KCONV, IFA_LT_D_VCONV, IFA_LT_D_B, IFA_LT_D_A, IFA_LT_D_ALOG, IFA_LT_D_DTBIAS,
    IFA_LT_D_G, IFA_LT_D_NORM, IFA_LT_D_O,
    IFA_LT_NORM2, IFA_LT_CANON1, IFA_LT_CANON2, IFA_LT_DWA,
    IFA_LT_M_Q, IFA_LT_M_DQ, IFA_LT_M_DQ_NORM, IFA_LT_M_UQ, IFA_LT_M_DKV, IFA_LT_M_DKV_NORM, IFA_LT_M_UK, IFA_LT_M_UV, IFA_LT_M_G, IFA_LT_M_O,
    IFA_LT_X_ROUTER, IFA_LT_X_CORR, IFA_LT_X_UP /* [experts * ff][width]; gated experts: [experts][gate ff | up ff][width] */, IFA_LT_X_DOWN /* [experts * width][ff] */,
    IFA_LT_NORM1B, IFA_LT_NORM2B,                  /* SANDWICH: the norms behind the sub-layers */
    IFA_LT_A_V, IFA_LT_A_Q_B, IFA_LT_A_K_B, IFA_LT_A_V_B, IFA_LT_A_Q_NORM, IFA_LT_A_K_NORM,      /* IFA_MIX_ROTARY (with IFA_LT_A_Q / _K / _O) */
    IFA_LT_X_ROUTER_B, IFA_LT_X_SH_GATE, IFA_LT_X_SH_UP, IFA_LT_X_SH_DOWN, IFA_LT_X_SH_SG,
    IFA_LT_NORM1_B, IFA_LT_NORM1_ALPHA, IFA_LT_NORM2_B, IFA_LT_NORM2_ALPHA,                       /* PRENORM: bias and scalar of the Dynamic Tanh norms */
    IFA_LT_C_R, IFA_LT_C_K, IFA_LT_C_V, IFA_LT_C_G, IFA_LT_C_A, IFA_LT_C_A_B, IFA_LT_C_W1, IFA_LT_C_W2, IFA_LT_C_W0, IFA_LT_C_NORM, IFA_LT_C_O,      /* IFA_MIX_CHAN_DELTA */
    IFA_LT_END
};
int ifa_model_create_layered(const ifa_layered_config *cfg, const ifa_layer_spec *layers, ifa_model **out);
/* a tensor from HOST memory: dtype IFA_BF16 (bit patterns) or IFA_F32 (IFA_LT_L_DECAY only); shapes are checked against the specs */
int ifa_model_set_tensor_host(ifa_model *m, int layer, int tensor_id, int dtype, const void *host_src, size_t rows, size_t cols);
/* fp32 logits of the most recent forward / decode_batch step (device pointer; rows x cols); the F16 logits_out of those calls
 * is a rounded copy of these */
int ifa_model_logits_f32(ifa_model *m, void **dptr, size_t *rows, size_t *cols);
/* One step over several queries at once, prompts and single tokens mixed: query q brings seq_lens[q] tokens (all queries' tokens
 * concatenated in tokens_host) at positions [seq_pos0[q], ...) on its slot seq_slots[q] (distinct).  all_logits 0: the fp32 logits
 * (ifa_model_logits_f32) hold one row per query, that of its last token; 1: one row per token, in order.  next_tokens_host[q]:
 * greedy token after query q's last row.  A row's result does not depend on what else is in the step. */
int ifa_model_step_seqs(ifa_model *m, int n_seqs, const int *tokens_host, const int *seq_lens, const int *seq_pos0, const int *seq_slots, int all_logits,
                        int *next_tokens_host);
/* 1 for a layer-list model, 0 for the standard network */
int ifa_model_is_layered(const ifa_model *m);

#ifdef __cplusplus
}
#endif
#endif /* INFERFLOW_AMD_H_ */
