/*
 * ttmi.h -- C ABI of libttmi.so, the MI355X (gfx950 / CDNA4) device layer behind the
 * TurboTransformers BERT encoder-layer hot path.
 *
 * Every entry point takes plain pointers, sizes and enums; nothing from HIP, torch or
 * pybind11 appears in a signature, so host C++ (or any FFI) can bind it without HIP
 * headers.  It replaces the `#ifdef TT_WITH_CUDA` device branches of the reference's
 * kernel and core layers; each declaration cites the reference interface it stands in
 * for (paths relative to the reference tree).
 *
 * Conventions
 *   - all tensors are dense row-major unless a leading dimension is given;
 *   - `dtype` selects the storage type of activations/weights (TTMI_F32 / F16 / BF16);
 *     reductions, softmax, LayerNorm and GEMM accumulation are always fp32
 *     (int32 for TTMI_I8 GEMMs);
 *   - `stream` is a `hipStream_t` passed as `void*` (NULL = the legacy default stream);
 *     kernels are enqueued and NOT synchronised;
 *   - every function returns 0 on success or a negative TTMI_E* code, and
 *     ttmi_last_error() then returns a thread-local message.
 */
#ifndef TTMI_H_
#define TTMI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTMI_API __attribute__((visibility("default")))

enum ttmi_dtype { TTMI_F32 = 0, TTMI_F16 = 1, TTMI_BF16 = 2, TTMI_I8 = 3, TTMI_I32 = 4, TTMI_I64 = 5 };
enum ttmi_act { TTMI_ACT_NONE = -1, TTMI_ACT_GELU = 0, TTMI_ACT_TANH = 1, TTMI_ACT_RELU = 2 };
enum ttmi_memcpy_kind { TTMI_H2D = 0, TTMI_D2H = 1, TTMI_D2D = 2 };
enum ttmi_status {
  TTMI_OK = 0,
  TTMI_EINVAL = -1,      /* bad argument / unsupported shape */
  TTMI_EDEVICE = -2,     /* a HIP runtime call failed */
  TTMI_ENOMEM = -3,      /* hipMalloc failed */
  TTMI_EINDEX = -4       /* an embedding id was out of range (reported by ttmi_check_async) */
};

/* Epilogues a GEMM can apply to its fp32 accumulators before the single store to HBM. */
enum ttmi_epilogue {
  TTMI_EPI_NONE = 0,          /* C = alpha*acc + beta*C                                   */
  TTMI_EPI_BIAS = 1,          /* C = acc + bias[n]                                        */
  TTMI_EPI_BIAS_ACT = 2,      /* C = act(acc + bias[n])             (AddBiasAct fused)    */
  TTMI_EPI_BIAS_RESIDUAL = 3, /* C = acc + bias[n] + residual[m,n]  (pre-LayerNorm sum)   */
  TTMI_EPI_QKV_SPLIT = 4,     /* acc + bias -> q,k,v [B,h,S,d]      (SplitAddBiasTranspose fused) */
  TTMI_EPI_QKV_SPLIT_PAD = 5, /* packed rows -> zero-padded q,k,v [B,h,maxS,d]            */
  TTMI_EPI_F32_OUT = 6        /* C_f32 = acc (+ bias[n] if given): c is float* whatever dtype */
};

/* ------------------------------------------------------------------ runtime ---------- */

TTMI_API const char* ttmi_last_error(void);

/* Kernel-selection switches, for A/B timing and for tests that push small or ragged problems through a kernel the
 * launchers would not pick for them.  No counterpart in the reference (cuBLAS and the CUDA kernels have no such
 * knob).  Names and values:
 *   "TTMI_LARGE_TILE"       1 = every eligible 16-bit product on the one-wavefront-per-SIMD GEMM kernel, 0 = none;
 *   "TTMI_WAVE_KERNEL"      0 = products of at most 128 rows stay on the LDS-tiled kernels;
 *   "TTMI_ATTENTION_WAVES"  4 / 8 = wavefronts per workgroup of the one-kernel attention;
 *   "TTMI_STATIC_SCRATCH_LIMIT"  bytes of its buffer ttmi_gemm_bias_layer_norm_static admits (to test its refusal);
 *   "TTMI_W4_A_STAGES"      2 = the one-wavefront-per-SIMD GEMM kernel keeps two LDS stages for the A operand
 *                           where it would take three;
 *   "TTMI_W4_SPLITK"        0 = ttmi_gemm_bias_layer_norm never cuts a product along K on that kernel, n >= 2 = n
 *                           slices for every product that can be cut that way;
 *   -1 = the launcher decides (the default).
 * Each switch starts from the environment variable of the same name, which is read once, at the first launch or
 * the first call of this function; later changes of the environment are not seen. */
TTMI_API int ttmi_set_kernel_switch(const char* name, int value);

/* Device bring-up and properties.  Replaces core::CUDADeviceContext
 * (turbo_transformers/core/cuda_device_context.cpp:23-46). */
TTMI_API int ttmi_device_count(int* count);
TTMI_API int ttmi_set_device(int device);
TTMI_API int ttmi_device_info(char* name, int name_len, int* compute_units, int* clock_khz,
                              int64_t* hbm_bytes, int* lds_bytes_per_cu);
TTMI_API int ttmi_mem_info(int64_t* free_bytes, int64_t* total_bytes);

/* Raw device memory.  Replaces allocator_impl.cpp's cudaMalloc/cudaFree branch
 * (turbo_transformers/core/allocator/allocator_impl.cpp:20-56). */
TTMI_API int ttmi_malloc(void** ptr, size_t bytes);
TTMI_API int ttmi_free(void* ptr);
/* Pinned host memory for staging copies. */
TTMI_API int ttmi_host_malloc(void** ptr, size_t bytes);
TTMI_API int ttmi_host_free(void* ptr);

/* Copies.  `ttmi_memcpy` is synchronous with respect to the host like core::Memcpy
 * (turbo_transformers/core/memory.cpp:34-81): it is enqueued on `stream` and the stream
 * is then synchronised.  `ttmi_memcpy_async` only enqueues. */
TTMI_API int ttmi_memcpy(void* dst, const void* src, size_t bytes, int kind, void* stream);
TTMI_API int ttmi_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream);
TTMI_API int ttmi_memset_zero(void* dst, size_t bytes, void* stream); /* fill kernel, graph-safe */

TTMI_API int ttmi_stream_create(void** stream);
TTMI_API int ttmi_stream_destroy(void* stream);
TTMI_API int ttmi_stream_sync(void* stream);
TTMI_API int ttmi_event_create(void** event);
TTMI_API int ttmi_event_destroy(void* event);
TTMI_API int ttmi_event_record(void* event, void* stream);
TTMI_API int ttmi_event_sync(void* event);
TTMI_API int ttmi_event_elapsed_ms(void* start, void* stop, float* ms);

/* Asynchronous device-side error flag (out-of-range embedding id): returns TTMI_EINDEX
 * once after a kernel has raised it.  The caller must have synchronised the stream.
 * Stands in for the `trap` in gpu_embedding_kernel.cu:32-34 and the throw in
 * embedding.cpp:59. */
TTMI_API int ttmi_check_async(void);

/* ---------------------------------------------------- memory-bound epilogue kernels --- */

/* kernels::LayerNorm  (layers/kernels/layer_norm.cpp:33-91, CPU branch :43-74).
 * In place on out[m,n]: mean = sum/n, var = sumsq/n - mean^2, out = beta + gamma*(x-mean)/sqrt(var+eps). */
TTMI_API int ttmi_layer_norm(void* out, const void* gamma, const void* beta, int64_t m, int64_t n,
                             float eps, int dtype, void* stream);

/* kernels::AddBiasLayerNorm  (layers/kernels/layer_norm.cpp:99-180, CPU branch :130-164).
 * out = LN(out + input + bias), in place on out. */
TTMI_API int ttmi_add_bias_layer_norm(void* out, const void* input, const void* bias, const void* gamma,
                                      const void* beta, int64_t m, int64_t n, float eps, int dtype,
                                      void* stream);

/* AddBiasLayerNorm whose residual stream stays in fp32 while `out` is 16-bit storage:
 *   y = LN(out + residual_f32 + bias);  out = round(y);  out_f32 = y.
 * residual_f32 and out_f32 may be the same buffer.  Used by the layers for bfloat16 models so
 * that only GEMM operands are rounded (no counterpart in the reference, which is fp32-only). */
TTMI_API int ttmi_add_bias_layer_norm_residual32(void* out, const float* residual_f32, const void* bias,
                                                 const void* gamma, const void* beta, float* out_f32, int64_t m,
                                                 int64_t n, float eps, int dtype, void* stream);

/* The same with the product itself in fp32: product_out_f32[m,n] holds a[m,k] . w[n,k]^T as the GEMM accumulated it
 * (ttmi_gemm_fused with TTMI_EPI_F32_OUT) and is overwritten with the unrounded result,
 *   y = LN(product_out_f32 + residual_f32 + bias);  out = round(y);  product_out_f32 = y.
 * product_out_f32 must not alias residual_f32.  No counterpart in the reference (fp32-only, where this is plain
 * AddBiasLayerNorm, layers/kernels/layer_norm.cpp:99-180). */
TTMI_API int ttmi_add_bias_layer_norm_product32(void* out, const float* residual_f32, const void* bias,
                                                const void* gamma, const void* beta, float* product_out_f32,
                                                int64_t m, int64_t n, float eps, int dtype, void* stream);

/* The dense projection and AddBiasLayerNorm that close both halves of an encoder layer, as one call:
 *   out[m,n] = LN(a[m,k] . w[n,k]^T + bias + residual)
 * (BertOutput, layers/bert_output.cpp:41-60; the attention output, layers/multi_headed_attention.cpp:359-371;
 * the reference issues MatMul then AddBiasLayerNorm).  Small problems, where the product is cut along K to
 * fill the chip, normalise inside the kernel that sums the K slices; larger ones run ttmi_gemm followed by
 * ttmi_add_bias_layer_norm.  Either `residual` (same dtype as out) or the pair residual_f32 / out_f32 (the
 * fp32 residual stream of ttmi_add_bias_layer_norm_residual32, which may alias each other) is given; the
 * unused ones are NULL.  With the fp32 pair and out_f32 != residual_f32, 16-bit products of large problems are kept
 * in fp32 between the GEMM and the LayerNorm (in out_f32), as the K-sliced path does for small ones; when the two
 * alias, the product of a large problem passes through `out` in the 16-bit type.  `out` must not alias `residual` or `a` (large problems store the bare product to `out`
 * before the residual is read); a call that passes the same buffer is refused.  a, w, out are densely packed
 * (lda = ldb = k, ldc = n). */
TTMI_API int ttmi_gemm_bias_layer_norm(const void* a, const void* w, void* out, const void* residual,
                                       const float* residual_f32, const void* bias, const void* gamma,
                                       const void* beta, float* out_f32, int64_t m, int64_t n, int64_t k, float eps,
                                       int dtype, void* stream);

/* ttmi_gemm_bias_layer_norm for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * arguments, same kernels and bit-identical results; the fp32 partial tiles of a product that is cut along K
 * live in a buffer of TTMI_STATIC_SCRATCH_BYTES that is part of the library's device image (every GPU the
 * library runs on holds it until the process ends) instead of the per-stream workspace ttmi_gemm_bias_layer_norm
 * allocates on first use.  The call reaches no hipMalloc / hipFree.  A problem whose K slices need more than
 * that buffer (slices * m * n * 4 bytes; the largest the encoder configurations produce is m = 2560, n = 768,
 * k = 3072 in three slices, 23.6 MB) is refused with TTMI_EINVAL; problems large enough to run unsplit need no
 * scratch and are accepted at any size.  One exception to "the same kernels": a product of a few thousand rows that
 * ttmi_gemm_bias_layer_norm cuts in two on its large-tile kernel (an optimisation of a product that also runs whole;
 * 6275 x 768 x 3072 is one) is cut here only if its partial products fit the buffer, and runs whole otherwise, with
 * the 16-bit rounding of the product in front of the LayerNorm that large problems have.  The first call on a device resolves the buffer's address and sets kernel
 * attributes, so make one call outside a graph capture before capturing calls.  Nothing has to be cleared between calls (every partial tile that is read
 * has been written by the same call), but all calls on one GPU share the buffer: calls that overlap in time
 * on one GPU (different streams or threads) race. */
#define TTMI_STATIC_SCRATCH_BYTES (32u << 20)
TTMI_API int ttmi_gemm_bias_layer_norm_static(const void* a, const void* w, void* out, const void* residual,
                                              const float* residual_f32, const void* bias, const void* gamma,
                                              const void* beta, float* out_f32, int64_t m, int64_t n, int64_t k,
                                              float eps, int dtype, void* stream);

/* kernels::AddBiasAct<T, Act>  (layers/kernels/activation.cpp:33-55, 90-119).
 * out[m,n] = act(out[m,n] + bias[n]) in place; gelu is the tanh form. */
TTMI_API int ttmi_add_bias_act(void* out, const void* bias, int64_t m, int64_t n, int act, int dtype,
                               void* stream);

/* kernels::ApplyMaskAndSoftmax  (layers/kernels/softmax.cpp:28-125).
 * In place on score[B,h,F,T]: x = score*scale + mask; p = exp(x-max)/sum over T.
 * `mask` is fp32 or NULL; mask_is_2d != 0 -> mask[B,T] (broadcast over heads and rows),
 * else mask[B,F,T]. */
TTMI_API int ttmi_apply_mask_and_softmax(void* score, const float* mask, int64_t batch, int64_t heads,
                                         int64_t from_len, int64_t to_len, int mask_is_2d, float scale,
                                         int dtype, void* stream);

/* kernels::SplitAddBiasTransposeForScore, 3-output form  (layers/kernels/transpose.cpp:310-406).
 * in[B,S,3,h,d] + bias[3,h,d] -> q,k,v each [B,h,S,d]. */
TTMI_API int ttmi_split_add_bias_transpose_for_score(const void* in, const void* bias, void* q, void* k,
                                                     void* v, int64_t batch, int64_t seq, int64_t heads,
                                                     int64_t head_dim, int dtype, void* stream);

/* kernels::SplitAddBiasTransposeForScorePad  (layers/kernels/transpose.cpp:459-580).
 * Packed in[1,sum(len),3,h,d] -> q,k,v [B,h,max_seq,d]; rows s >= len[b] are zero (no bias).
 * `cu_seqlens` is a DEVICE int32 array [batch+1] of exclusive prefix sums of the lengths
 * (built once per batch by ttmi_build_cu_seqlens instead of a per-call malloc+copy,
 * gpu_transpose_kernel.cu:213-222). */
TTMI_API int ttmi_split_add_bias_transpose_for_score_pad(const void* in, const void* bias, void* q, void* k,
                                                         void* v, const int32_t* cu_seqlens, int64_t batch,
                                                         int64_t max_seq, int64_t heads, int64_t head_dim,
                                                         int dtype, void* stream);

/* kernels::TransposeForScore  (layers/kernels/transpose.cpp:105-125, 158-191): [B,h,S,d] -> [B,S,h,d]. */
TTMI_API int ttmi_transpose_for_score(const void* in, void* out, int64_t batch, int64_t seq, int64_t heads,
                                      int64_t head_dim, int dtype, void* stream);

/* kernels::TransposeForScorePad  (layers/kernels/transpose.cpp:128-156, 589-623):
 * [B,h,max_seq,d] -> packed [1,sum(len),h,d], pad rows dropped. */
TTMI_API int ttmi_transpose_for_score_pad(const void* in, void* out, const int32_t* cu_seqlens, int64_t batch,
                                          int64_t max_seq, int64_t heads, int64_t head_dim, int dtype,
                                          void* stream);

/* Upload host lengths as a device prefix array cu_seqlens[batch+1] (int32) on `stream`.
 * `staging` is pinned host memory of at least (batch+1)*4 bytes owned by the caller. */
TTMI_API int ttmi_build_cu_seqlens(const int64_t* host_lens, int64_t batch, int32_t* staging,
                                   int32_t* cu_seqlens_dev, void* stream);

/* Per-token destination rows of a packed batch: token_rows[t] = b*max_seq + (t - cu_seqlens[b])
 * for cu_seqlens[b] <= t < cu_seqlens[b+1]; `total` = cu_seqlens[batch].  Built once per batch;
 * consumed by the QKV_SPLIT_PAD GEMM epilogue. */
TTMI_API int ttmi_build_token_rows(const int32_t* cu_seqlens, int64_t batch, int64_t max_seq, int64_t total,
                                   int32_t* token_rows, void* stream);

/* kernels::LookupEmbedding<Add>  (layers/kernels/embedding.cpp:28-85).
 * out[i,:] = table[ids[i],:]  (add=0) or out[i,:] += table[ids[i],:] (add=1); ids are int64.
 * An id outside [0,vocab) leaves the row untouched and raises the async error flag. */
TTMI_API int ttmi_lookup_embedding(void* out, const void* table, const int64_t* ids, int64_t num_ids,
                                   int64_t hidden, int64_t vocab, int add, int dtype, void* stream);

/* layers::BERTEmbedding::operator() as one kernel  (layers/bert_embedding.cpp:24-65):
 * out = LN(word[ids] + type[type_ids] + pos[pos_ids]), adds in that order. */
TTMI_API int ttmi_bert_embedding(void* out, const int64_t* ids, const int64_t* pos_ids,
                                 const int64_t* type_ids, const void* word_table, const void* pos_table,
                                 const void* type_table, const void* gamma, const void* beta,
                                 int64_t num_ids, int64_t hidden, int64_t vocab, int64_t max_pos,
                                 int64_t num_types, float eps, int dtype, void* stream);
/* Same, also writing the unrounded LayerNorm output to out_f32 (start of an fp32 residual stream). */
TTMI_API int ttmi_bert_embedding_residual32(void* out, float* out_f32, const int64_t* ids, const int64_t* pos_ids,
                                            const int64_t* type_ids, const void* word_table,
                                            const void* pos_table, const void* type_table, const void* gamma,
                                            const void* beta, int64_t num_ids, int64_t hidden, int64_t vocab,
                                            int64_t max_pos, int64_t num_types, float eps, int dtype,
                                            void* stream);

/* kernels::common::Sequence / Fill / Transform  (layers/kernels/common.cpp:29-90), the three
 * helpers of layers::PrepareBertMasks (layers/prepare_bert_masks.cpp:24-66). */
TTMI_API int ttmi_fill_i64(int64_t* data, int64_t n, int64_t value, void* stream);
TTMI_API int ttmi_fill_f32(float* data, int64_t n, float value, void* stream);
/* data[r, c] = c for r < rows, c < cols */
TTMI_API int ttmi_sequence_rows_i64(int64_t* data, int64_t rows, int64_t cols, void* stream);
/* dst[i] = -10000 * (1 - src[i]) */
TTMI_API int ttmi_mask_transform(const int64_t* src, float* dst, int64_t n, void* stream);

/* kernels::SeqPool  (layers/kernels/seq_pool.cpp:124-155): in[B,S,H] -> out[B,H];
 * pool_type 0 = max, 1 = mean, 2 = first, 3 = last (layers/types.h PoolType order). */
TTMI_API int ttmi_seq_pool(const void* in, void* out, int64_t batch, int64_t seq, int64_t hidden, int pool_type,
                           int dtype, void* stream);

/* Smart-batch key-padding mask (python layers/modeling_smart_pad.py:465-475):
 * mask[b, 0, t] = 0 for t < len[b] else -1e9, shape [B,1,max_seq] fp32. */
TTMI_API int ttmi_smart_pad_mask(float* mask, const int32_t* cu_seqlens, int64_t batch, int64_t max_seq,
                                 void* stream);

/* Plain 2-D transpose out[c,r] = in[r,c], used once per weight at layer construction to
 * keep every weight K-contiguous ([out,in]) for the MFMA kernels. */
TTMI_API int ttmi_transpose_2d(const void* in, void* out, int64_t rows, int64_t cols, int dtype, void* stream);

/* kernels::Concat<T>  (layers/kernels/utils.cpp:33-93), the decoder's key/value cache append:
 * out[o, 0:a_inner] = a[o, :], out[o, a_inner:] = b[o, :] for o < outer, i.e. a concatenation along
 * one dimension with outer = product of the dimensions before it and *_inner = that dimension's
 * size times the product of the dimensions after it.  Pure data movement, any dtype. */
TTMI_API int ttmi_concat(const void* a, const void* b, void* out, int64_t outer, int64_t a_inner, int64_t b_inner,
                         int dtype, void* stream);

/* Element type conversion between TTMI_F32 / F16 / BF16 buffers. */
TTMI_API int ttmi_convert(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n, void* stream);

/* ------------------------------------------------------------------ MFMA GEMMs -------- */

/* kernels::MatMul  (layers/kernels/mat_mul.cpp:30-118).
 * C[M,N] = alpha * A[M,K] * op(B) + beta * C, all row-major with leading dimensions in
 * elements.  trans_b = 0: B is [K,N] (ldb >= N);  trans_b != 0: B is [N,K] (ldb >= K).
 * Problems with few output tiles and a long K run as K slices plus a reduction kernel; their fp32
 * partial tiles live in a per-stream workspace this library allocates on first use and keeps. */
TTMI_API int ttmi_gemm(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int64_t lda,
                       int64_t ldb, int64_t ldc, int trans_b, float alpha, float beta, int dtype,
                       void* stream);

/* kernels::BatchMatMul  (layers/kernels/mat_mul.cpp:119-213): strided-batched form of the
 * above; batch_count problems, strides in elements. */
TTMI_API int ttmi_gemm_strided_batched(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k,
                                       int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a,
                                       int64_t stride_b, int64_t stride_c, int64_t batch_count, int trans_b,
                                       float alpha, float beta, int dtype, void* stream);

/* BatchMatMul over a [batch, heads] grid of problems whose operands are strided views:
 * problem (b, h) uses A + b*a_batch + h*a_head, etc. (strides in elements).  With
 * c_batch = S*heads*d, c_head = d, ldc = heads*d the P*V product lands directly in
 * [B,S,h,d], i.e. BatchMatMul + TransposeForScore in one pass
 * (layers/multi_headed_attention.cpp:345-354). */
TTMI_API int ttmi_gemm_batched_heads(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k,
                                     int64_t lda, int64_t ldb, int64_t ldc, int64_t heads, int64_t a_batch,
                                     int64_t a_head, int64_t b_batch, int64_t b_head, int64_t c_batch,
                                     int64_t c_head, int64_t batch, int trans_b, float alpha, float beta,
                                     int dtype, void* stream);

/* Self-attention core in one kernel, for head_dim 64 and fp16/bf16/fp32:
 *   out[b, s, head*64 + :] = softmax(scale * q[b,head,s,:] k[b,head]^T + mask[b,:]) v[b,head]
 * q,k,v are [B,h,S,64]; `mask` is an additive fp32 [B,S] key mask or NULL; `out` is [B,S,h*64].
 * It replaces BatchMatMul + ApplyMaskAndSoftmax + BatchMatMul + TransposeForScore
 * (layers/multi_headed_attention.cpp:323-354) when the [B,h,S,S] probabilities are not an
 * output: the score tensor never reaches HBM.  With `cu_seqlens` (device int32 [B+1]) q,k,v are
 * the padded tensors of a packed batch (S = max length): keys and queries >= len[b] are never
 * read (pad rows need not be zero) and `out` is packed [sum(len), h*64]
 * (…smart_batch.cpp:368-392).  `v_seq_pitch` = 0: v is [B,h,S,64]; > 0: v is stored transposed,
 * [B,h,64,v_seq_pitch] with v_seq_pitch a multiple of 8 and >= S, the layout the QKV_SPLIT
 * epilogues write when asked to (the faster path: tiles of V^T are copied, not scattered). */
TTMI_API int ttmi_fused_attention(const void* q, const void* k, const void* v, const float* mask, void* out,
                                  const int32_t* cu_seqlens, int64_t batch, int64_t heads, int64_t seq,
                                  int64_t head_dim, int64_t v_seq_pitch, float scale, int dtype, void* stream);

/* Arguments of the fused epilogues; unused members are NULL / 0. */
typedef struct ttmi_epilogue_args {
  const void* bias;          /* [N], same dtype as C                                        */
  const void* residual;      /* [M,N] row-major, ld = ldc          (BIAS_RESIDUAL)          */
  int act;                   /* ttmi_act                            (BIAS_ACT)               */
  void* q; void* k; void* v; /* outputs [B,h,S,d]                   (QKV_SPLIT[_PAD])        */
  int64_t seq;               /* S (or max_seq for the padded form)                          */
  int64_t heads;             /* h                                                           */
  int64_t head_dim;          /* d; N must equal 3*h*d, or h*d: then only q is written -- MatMul +
                                AddBiasTransposeForScore of one projection
                                (layers/multi_headed_attention.cpp:73-88)                   */
  const int32_t* token_rows; /* device [M]: packed token -> b*max_seq+s (QKV_SPLIT_PAD)      */
  int64_t batch;             /* B                                   (QKV_SPLIT_PAD)          */
  int64_t v_seq_pitch;       /* 0: v is [B,h,S,d]; > 0: v is written transposed as
                                [B,h,d,v_seq_pitch] (multiple of 8, >= seq)  (QKV_SPLIT*)    */
} ttmi_epilogue_args;

/* MatMul with the following memory-bound op folded into the store of the accumulators:
 *   BIAS_ACT       = MatMul + AddBiasAct            (layers/bert_intermediate.cpp:43-46)
 *   BIAS_RESIDUAL  = MatMul + the `out+input+bias` part of AddBiasLayerNorm
 *                    (layers/bert_output.cpp:47-51, layers/multi_headed_attention.cpp:359-371)
 *   QKV_SPLIT[_PAD]= MatMul + SplitAddBiasTransposeForScore[Pad]
 *                    (layers/multi_headed_attention.cpp:199-203, ..._smart_batch.cpp:212-217)
 *   F32_OUT        = MatMul whose result leaves in fp32 (c is float*, ldc in floats; bias optional): what a 16-bit
 *                    model hands to AddBiasLayerNorm without rounding it first
 * B is always [N,K] here (weights are repacked K-contiguous at construction).
 * For the QKV forms `c` may be NULL. */
TTMI_API int ttmi_gemm_fused(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k,
                             int64_t lda, int64_t ldb, int64_t ldc, int epilogue,
                             const ttmi_epilogue_args* args, int dtype, void* stream);

/* Which kernel variant ttmi_gemm (epilogue TTMI_EPI_NONE, args NULL) or ttmi_gemm_fused would launch for an
 * aligned, densely packed product of this shape, as text: family (reg = register-staged, dma = global->LDS DMA,
 * dma_agpr = DMA with accumulators in AGPRs, dma3_agpr = the same with a third LDS stage for the A operand, wave = one wavefront per tile with its operand fragments straight from
 * global memory), wavefronts per workgroup, tile, K split; e.g. "dma8w_256x256", "wave1w_32x32_splitk3".
 * Nothing is launched.  No counterpart in the reference (cuBLAS picks its kernels out of sight); measurement
 * scripts use it to tie recorded per-kernel figures to the variant they were recorded on.  For the QKV epilogues
 * `args` supplies seq / heads / head_dim / v_seq_pitch (and batch); pointers in it are ignored. */
TTMI_API int ttmi_gemm_describe(int64_t m, int64_t n, int64_t k, int epilogue, const ttmi_epilogue_args* args, int dtype,
                                char* out, size_t capacity);


/* Measurement aid, never on a product path: a loop of nothing but matrix instructions on register operands, one
 * workgroup of eight wavefronts per entry of the grid, to find what the matrix pipes sustain on this chip for a
 * given kind of operand values.  It plays the part of the reference's GEMM micro-benchmark
 * (benchmark/turbo_transformers/layers/kernels/matmul_benchmark.cpp:60-70) one level further down.
 *   block      16 = v_mfma_f32_16x16x32, 32 = v_mfma_f32_32x32x16 (of `dtype` TTMI_F16 or TTMI_BF16);
 *   operands   device buffer of 65536 elements of `dtype` the operand registers are filled from;
 *   iters      loop iterations; each is 262144 FLOP per wavefront (eight wavefronts per workgroup);
 *   sink       one device float (keeps the result alive; not written in practice);
 *   clocks     device uint64[2 * workgroups]: per workgroup, shader-clock cycles and ticks of the constant
 *              100 MHz clock spent in the loop (their ratio is the shader clock the chip held). */
TTMI_API int ttmi_yardstick_mfma(int block, int dtype, const void* operands, int iters, int workgroups, float* sink,
                                 uint64_t* clocks, void* stream);

/* int8 path (quantized BERT: int8 x int8 -> int32 accumulators, exact).
 * ttmi_quantize_rows_i8: per-tensor symmetric dynamic scale from max|x| over the whole
 *   [m,k] activation: scale = max|x|/127 (1 if the tensor is all zero), q = clamp(rint(x/scale), -127, 127).
 *   `scale_dev` is a DEVICE float[TTMI_QUANT_SCALE_FLOATS]: [0] receives the scale, [1] max|x|, the rest is
 *   scratch (per-workgroup maxima; nothing has to be cleared between calls).
 * ttmi_gemm_i8: C_i32[M,N] = A_i8[M,K] * B_i8[N,K]^T.
 * ttmi_dequant_bias: out[m,n] = acc[m,n] * (*act_scale) * w_scale[n] + bias[n] (fp32 out; bias may be NULL).
 * ttmi_gemm_i8_dequant: ttmi_gemm_i8 followed by ttmi_dequant_bias in one kernel (the accumulators never
 *   reach memory); same operation order, same bits.  `act` other than TTMI_ACT_NONE also applies that
 *   activation, as ttmi_add_bias_act would after the bias (the FusedAddBiasGELU step of QBertIntermediate).  Together they stand in for the dynamically
 *   quantised Linear module the reference's QBert* layers call (qmodeling_bert.py:17,35). */
#define TTMI_QUANT_SCALE_FLOATS 514
/* Per-workgroup maxima handed from the kernel that PRODUCES an activation to the quantisation of the Linear that
 * consumes it, so that finding the dynamic scale costs no pass (and no launch) of its own:
 *   absmax_slots   DEVICE float[TTMI_ABSMAX_SLOTS]; a producer writes EVERY slot on every launch (max|output| of one
 *                  workgroup each, zero in the rest): nothing has to be cleared and nothing carries over between calls;
 *   slots_written  HOST int: TTMI_ABSMAX_SLOTS when the launch filled the slots, 0 when its workgroups outnumber
 *                  them (then the slots are untouched and the consumer calls ttmi_quantize_rows_i8 as before).
 * ttmi_add_bias_layer_norm_absmax   = ttmi_add_bias_layer_norm, the same bits in `out`;
 * ttmi_gemm_i8_dequant_absmax       = ttmi_gemm_i8_dequant, the same bits in `c` (maximum taken after the activation);
 * ttmi_fused_attention_absmax       = ttmi_fused_attention, the same bits in `out`; the maxima are left by dense
 *                                     fp32 launches only (any other call reports 0 slots written);
 * ttmi_quantize_rows_i8_from_absmax = the second half of ttmi_quantize_rows_i8: scale from the slots' maximum,
 *                                     scale_dev[0] / [1] as there, the same bits in `q`.
 * No counterpart in the reference, whose quantized Linear is its framework's dynamic quantisation
 * (qmodeling_bert.py:17,35). */
#define TTMI_ABSMAX_SLOTS 1024
TTMI_API int ttmi_add_bias_layer_norm_absmax(void* out, const void* input, const void* bias, const void* gamma,
                                             const void* beta, int64_t m, int64_t n, float eps, int dtype,
                                             float* absmax_slots, int* slots_written, void* stream);
TTMI_API int ttmi_fused_attention_absmax(const void* q, const void* k, const void* v, const float* mask, void* out,
                                         const int32_t* cu_seqlens, int64_t batch, int64_t heads, int64_t seq,
                                         int64_t head_dim, int64_t v_seq_pitch, float scale, int dtype,
                                         float* absmax_slots, int* slots_written, void* stream);
TTMI_API int ttmi_gemm_i8_dequant_absmax(const int8_t* a, const int8_t* b, float* c, const float* act_scale_dev,
                                         const float* w_scale, const float* bias, int act, int64_t m, int64_t n,
                                         int64_t k, int64_t lda, int64_t ldb, int64_t ldc, float* absmax_slots,
                                         int* slots_written, void* stream);
TTMI_API int ttmi_quantize_rows_i8_from_absmax(const float* x, int8_t* q, float* scale_dev, const float* absmax_slots,
                                               int64_t m, int64_t k, void* stream);
/* ttmi_quantize_weight_rows_i8: per-output-channel symmetric scales for a weight w[N,K] (fp32):
 *   scales[n] = max_k |w[n,k]| / 127 (1 if the row is zero), q[n,k] = clamp(rint(w[n,k]/scales[n]), -127, 127). */
TTMI_API int ttmi_quantize_weight_rows_i8(const float* w, int8_t* q, float* scales, int64_t n, int64_t k,
                                          void* stream);
TTMI_API int ttmi_quantize_rows_i8(const float* x, int8_t* q, float* scale_dev, int64_t m, int64_t k,
                                   void* stream);
TTMI_API int ttmi_gemm_i8(const int8_t* a, const int8_t* b, int32_t* c, int64_t m, int64_t n, int64_t k,
                          int64_t lda, int64_t ldb, int64_t ldc, void* stream);
TTMI_API int ttmi_gemm_i8_dequant(const int8_t* a, const int8_t* b, float* c, const float* act_scale_dev,
                                  const float* w_scale, const float* bias, int act, int64_t m, int64_t n, int64_t k,
                                  int64_t lda, int64_t ldb, int64_t ldc, void* stream);
/* ttmi_gemm_i8_dequant_qkv_split: the QKV projection of the quantized attention: the dequantised product plus
 *   bias[3*heads*head_dim] written straight to q,k,v[B,heads,seq,head_dim] (fp32), i.e. ttmi_gemm_i8_dequant
 *   without bias followed by ttmi_split_add_bias_transpose_for_score, with the same bits. */
TTMI_API int ttmi_gemm_i8_dequant_qkv_split(const int8_t* a, const int8_t* b, const float* act_scale_dev,
                                            const float* w_scale, const float* bias, float* q, float* k_out,
                                            float* v, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                                            int64_t seq, int64_t heads, int64_t head_dim, void* stream);
TTMI_API int ttmi_dequant_bias(const int32_t* acc, const float* act_scale_dev, const float* w_scale,
                               const float* bias, float* out, int64_t m, int64_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TTMI_H_ */
