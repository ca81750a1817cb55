/*
 * arcq.h -- C ABI of libarcq_hip.so: ARCQuant's quantized-linear hot path on MI355X (gfx950).
 *
 * Four operators, the ones the reference exports from its pybind11 module `agemm`
 * (kernels/src/bindings.cpp:547-575), take raw device pointers and sizes and return an
 * arcq_status.  All work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 * null stream) and nothing synchronises with the host, so a caller may enqueue further work
 * behind it; the reference launches on the legacy default stream and its callers
 * synchronise after every call (model/qLinearLayer.py:73).
 *
 * Numerics follow the reference's PyTorch fake-quant path (model/quantize.py), not its CUDA
 * kernels: block scale = amax/6 rounded as quantize_ue4m3 / quantize_ue8m0 do, x/scale as a
 * correctly rounded fp32 division, e2m1 by nearest value with ties toward the lower value,
 * the residual of the last `select_num` reordered channels kept in fp32 and quantized again.
 *
 * Data layout (internal to the quantizer <-> GEMM pair, like the reference's):
 *   K'      = K + select_num, channel order [K reordered | select_num residual]
 *   codes   u8 [rows, K'/2], row-major, element 2j in the low nibble of byte j;
 *           a code is sign<<3 | magnitude index over {0,.5,1,1.5,2,3,4,6}; zero is 0x0
 *   scales  u8 [rows, K'/G], row-major, G = 16 (NVFP4) or 32 (MXFP4)
 *           NVFP4 byte b: (1 + (b&7)/8) * 2^((b>>3) - 9)   (= standard E4M3 byte + 16 from 2^-6 up;
 *                 the extra low binades hold the values quantize_ue4m3 yields below 2^-6)
 *           MXFP4 byte b: 2^(b - 127)                      (standard E8M0)
 */
#ifndef ARCQ_H_
#define ARCQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  ARCQ_OK = 0,
  ARCQ_ERR_NULL = 1,     /* a required pointer is NULL */
  ARCQ_ERR_SHAPE = 2,    /* rows/K/select_num outside what the path defines */
  ARCQ_ERR_FORMAT = 3,   /* fmt is neither ARCQ_FMT_NVFP4 nor ARCQ_FMT_MXFP4 */
  ARCQ_ERR_ALIGN = 4,    /* a pointer is not 16-byte aligned */
  ARCQ_ERR_LAUNCH = 5,   /* the HIP runtime refused the launch (see arcq_last_hip_error) */
  ARCQ_ERR_INDEX = 6,    /* reorder_index is not a permutation of 0..K-1 (arcq_check_index) */
  ARCQ_ERR_WORKSPACE = 7 /* scratch memory unavailable: the stream is being captured and has none yet
                            (arcq_prepare_stream), or the problem exceeds a fixed scratch buffer */
} arcq_status;

enum { ARCQ_FMT_NVFP4 = 0, ARCQ_FMT_MXFP4 = 1 };

/* Library version (major*10000 + minor*100 + patch). */
int arcq_version(void);
const char *arcq_status_string(int status);
/* hipError_t of the last failed launch on this thread, as an int (0 = none). */
int arcq_last_hip_error(void);

/*
 * Scratch memory.  Three kernels need device memory beyond their inputs and outputs: the split-K GEMM
 * (fp32 partial tiles, arcq_matmul on narrow layers with few rows), the split decode attention
 * (partial softmax sums, arcq_kv_decode_i4 with few sequences) and arcq_tensor_scale /
 * arcq_reorder_quantize_x_absmax (a few words and one 8-byte slot per workgroup, through which the workgroups of a
 * launch exchange their maxima; zeroed once, every launch leaves them ready for the next).
 * The library keeps one buffer of each kind per (device, stream), allocated on the first call that
 * needs it and kept until arcq_release_stream or the end of the process (32 MiB + 8 MiB + 4 KiB when all
 * three exist); calls on one stream are serialised, so they never share a buffer with a call on another
 * stream.  An allocation cannot happen while the stream is being captured into a
 * graph: such a call returns ARCQ_ERR_WORKSPACE unless the stream has its buffers already.
 * arcq_prepare_stream allocates all three for (current device, stream), and resolves the address of
 * arcq_matmul_noalloc's fixed array on that device -- call it once before capturing on that stream.  A graph replayed on another stream still uses the buffers of the stream
 * it was captured on.  (The reference keeps no state between calls: its CUTLASS GEMM has no split-K
 * and it computes tensor scales with torch, kernels/src/nvfp4.cu:35-132, model/qLlamaLayer.py:73-77.)
 */
int arcq_prepare_stream(void *stream);
/* Frees the scratch buffers of (current device, stream) and forgets the pair: call it before destroying a
 * stream that ever ran one of the three kernels above (a later stream may get the same handle and would
 * inherit the buffers otherwise), and never while a graph captured on that stream may still be replayed.
 * Waits for the device.  ARCQ_OK also when the stream has no buffers.  No counterpart in the reference. */
int arcq_release_stream(void *stream);

/* Block size G of a format (16 / 32), or 0 for an unknown format. */
int arcq_group_size(int fmt);
/* Output buffer sizes in bytes for `rows` rows of K channels with select_num residual channels.
 * Replaces get_sfa_buffer_size_in_bytes / get_sfb_buffer_size_in_bytes
 * (kernels/src/bindings.cpp:83-95) and the QX/QW shape rule (bindings.cpp:133,181). */
size_t arcq_codes_bytes(int rows, int K, int select_num);
size_t arcq_scales_bytes(int rows, int K, int select_num, int fmt);

/*
 * Activation quantizer: gather x[:, reorder_index], divide by the tensor scale, block-quantize,
 * append the quantized residual of the last select_num channels.
 * Replaces agemm.reorder_quantize_x (kernels/src/bindings.cpp:122-163; kernels
 * reorder.cu:68-203, 380-555, down.cu:71-233) with the numerics of fake_reorder_quantize_x
 * (model/quantize.py:314-343).
 *   x              bf16 [M,K] row-major, device
 *   reorder_index  int16 [K], device; a permutation of 0..K-1 (not checked here)
 *   select_num     multiple of G, 0 <= select_num <= K
 *   K              multiple of 32, 32 <= K <= 32736 (int16 index range)
 *   global_scale / d_global_scale: the fp32 tensor scale values are divided by
 *                  (quantize.py:330).  If d_global_scale != NULL it is read on the device
 *                  (no host sync) and global_scale is ignored.
 *   codes, scales  outputs, sizes as arcq_codes_bytes / arcq_scales_bytes
 */
int arcq_reorder_quantize_x(const void *x, int M, int K, const int16_t *reorder_index, int select_num, int fmt,
                            float global_scale, const float *d_global_scale, void *codes, void *scales,
                            void *stream);

/*
 * Weight quantizer: same gather and block quantizer; the last select_num channels are
 * repeated verbatim (codes and scales) instead of a residual.
 * Replaces agemm.reorder_quantize_w (kernels/src/bindings.cpp:170-210; reorder.cu:210-330,
 * 562-696, down.cu:240-361) with the numerics of fake_reorder_quantize_w
 * (model/quantize.py:287-312).
 */
int arcq_reorder_quantize_w(const void *w, int N, int K, const int16_t *reorder_index, int select_num, int fmt,
                            float global_scale, const float *d_global_scale, void *codes, void *scales,
                            void *stream);

/*
 * Fused RMSNorm + activation quantizer.
 * Replaces agemm.rmsnorm_quantize_x (kernels/src/bindings.cpp:216-254; rmsnorm.cu:68-255).
 * Normalisation is the PyTorch one the reference's layers run before quantizing
 * (benchmarks/modeling_arc.py:237-242): h = bf16(x * rsqrt(mean(x^2) + eps)) in fp32,
 * y = bf16(gamma * h); mean(x^2) is the correctly rounded one (fp64 accumulation).
 *   gamma  bf16 [K], device
 * The reference's op has no tensor scale (it quantizes y as is); pass global_scale = 1 and
 * d_global_scale = NULL for that behaviour.
 */
int arcq_rmsnorm_quantize_x(const void *x, const void *gamma, float eps, int M, int K,
                            const int16_t *reorder_index, int select_num, int fmt, float global_scale,
                            const float *d_global_scale, void *codes, void *scales, void *stream);

/*
 * Fused SwiGLU + activation quantizer for the down projection's input: t = act_fn(gate) * up
 * formed as the reference's layers form it in bf16 -- SiLU in fp32 as g / (1 + exp(-g)), rounded to
 * bf16, times up, rounded to bf16 (model/qLlamaLayer.py:432, model/qMixtralLayer.py:531) -- and
 * quantized like arcq_reorder_quantize_x without t ever reaching memory.  The reference names this
 * fusion but does not ship it (benchmarks/modeling_arc.py:112, commented activate_quantize_x).
 *   gate, up  bf16 rows of K elements with a common row stride `ld` (elements, multiple of 8): for a
 *             fused gate_up projection output [M, 2K] pass up = gate + K and ld = 2K
 *   K         multiple of 32, 32 <= K <= 32736
 * arcq_swiglu_absmax computes max |t| over the tensor (numerator of the NVFP4 tensor scale,
 * model/qLlamaLayer.py:74) into *d_absmax, which the caller has set to 0; nothing synchronises.
 */
int arcq_swiglu_quantize_x(const void *gate, const void *up, int ld, int M, int K, const int16_t *reorder_index,
                           int select_num, int fmt, float global_scale, const float *d_global_scale, void *codes,
                           void *scales, void *stream);
int arcq_swiglu_absmax(const void *gate, const void *up, int ld, int M, int K, float *d_absmax, void *stream);

/*
 * NVFP4 tensor scale of an activation tensor, max |x| / divisor, as the reference's callers compute it
 * with torch before the quantizer (x.abs().max() / (448 * 6), model/qLlamaLayer.py:73-77), in one
 * launch and without a host round trip; an all-zero tensor gets 1.
 *   x        bf16 rows of K elements, row stride ld (elements, multiple of 8); K multiple of 8
 *   up       NULL, or the second operand of a fused SwiGLU: the scale is then that of
 *            act_fn(x) * up (x = gate), as arcq_swiglu_quantize_x forms it
 *   d_scale  fp32 scalar on the device, read by the quantizer (d_global_scale) and the GEMM (d_alpha_a)
 * Blocks combine their maxima through two words of the stream's scratch memory (arcq_prepare_stream).
 */
int arcq_tensor_scale(const void *x, const void *up, int ld, int M, int K, float divisor, float *d_scale, void *stream);

/*
 * The tensor scale and the activation quantizer under it as one call: what the reference's callers write as
 * scale = x.abs().max() / (448 * 6) followed by reorder_quantize_x(x / scale, ...) (model/qLlamaLayer.py:73-77,
 * kernels/src/bindings.cpp:122-163).  d_scale receives max |x| / divisor (1 for an all-zero tensor); codes and
 * scale bytes are those of arcq_reorder_quantize_x with d_global_scale = d_scale.
 * NVFP4 activations of up to 16 rows per CU (4096 on an MI355X) and K = 1024, 2048, 3072 or 4096 take ONE launch:
 * the rows stay in LDS while the workgroups exchange their maxima through the stream's scratch memory
 * (arcq_prepare_stream), so x is read once.  Everything else is arcq_tensor_scale followed by the quantizer.
 * A workgroup that does not hear from the others in time (they share the chip with other work) takes the maximum
 * over x by itself; the result does not depend on it.
 */
int arcq_reorder_quantize_x_absmax(const void *x, int M, int K, const int16_t *reorder_index, int select_num, int fmt,
                                   float divisor, float *d_scale, void *codes, void *scales, void *stream);

/*
 * Augmented-K block-scaled FP4 GEMM: C[M,N] = alpha * dq(A)[M,K'] @ dq(B)[N,K']^T, fp32
 * accumulation, bf16 output.
 * Replaces agemm.matmul (kernels/src/bindings.cpp:99-120 -> nvfp4.cu:35-132).
 *   a_codes/a_scales  activations as written by the quantizers above, M rows
 *   b_codes/b_scales  weights, N rows
 *   Kp                K' = K + select_num, a multiple of 64
 *   alpha             host factor; if d_alpha_a / d_alpha_b are non-NULL the fp32 values they
 *                     point to on the device are multiplied in as well (the reference's
 *                     scale_x * scale_w, model/qLinearLayer.py:69), without a host sync
 *   c                 bf16 [M,N] row-major
 */
int arcq_matmul(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales, int M, int N,
                int Kp, int fmt, float alpha, const float *d_alpha_a, const float *d_alpha_b, void *c,
                void *stream);

/*
 * The same GEMM with a residual added in the epilogue: C = bf16(bf16(alpha * acc) + residual), residual
 * bf16 [M,N] -- bit for bit what a bf16 add of arcq_matmul's output and the residual gives (the
 * reference's layers add the attention / MLP output to the hidden states as a separate torch op,
 * model/qLlamaLayer.py:147-168, benchmarks/modeling_arc.py:284-307), without the output's round trip through memory.
 */
int arcq_matmul_add(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales, int M, int N,
                    int Kp, int fmt, float alpha, const float *d_alpha_a, const float *d_alpha_b, const void *residual,
                    void *c, void *stream);

/*
 * arcq_matmul for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernel
 * choice and the same bits as arcq_matmul, but the split-K partial tiles live in a fixed 8 MiB array inside
 * the library's code object (one copy per GPU, held until the process ends) instead of a stream's scratch
 * buffer, and the call contains no allocation of any kind.
 *   - A problem whose plan needs more than arcq_matmul_noalloc_limit() bytes of partial tiles
 *     (arcq_matmul_scratch_bytes tells, 0 = none needed) is refused with ARCQ_ERR_WORKSPACE and nothing is
 *     launched: e.g. the NVFP4 4096 x 14336 down projection at 512 rows (two K slices, 16 MiB).  Every decode batch
 *     (M <= 64) of the Llama-3-8B shapes fits.
 *   - All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams,
 *     two threads) race.  The array keeps the last call's contents; every word a call reads back it has
 *     written first, so nothing needs clearing.
 *   - The array's address on a device is resolved (hipGetSymbolAddress, no allocation) by arcq_prepare_stream,
 *     or else by the first call of this entry point on that device whose plan cuts K: do one of the two
 *     before a capture.
 */
int arcq_matmul_noalloc(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales, int M, int N,
                        int Kp, int fmt, float alpha, const float *d_alpha_a, const float *d_alpha_b, void *c,
                        void *stream);
size_t arcq_matmul_noalloc_limit(void);
/* bytes of split-K partial tiles arcq_matmul's plan uses for this problem (0: the plan does not cut K) */
size_t arcq_matmul_scratch_bytes(int M, int N, int Kp, int fmt);

/*
 * Grouped launches for mixture-of-experts blocks.  The reference walks the experts in Python
 * (model/qMixtralLayer.py:458-471): per expert one torch.where (a host synchronisation), a gather of its
 * tokens, reorder_quantize_x with the expert's reorder_index (:530), two GEMMs against the expert's
 * weights, the activation quantizer again (:539) and the last GEMM.  Here the tokens are sorted by expert
 * once and each of those steps is ONE launch over all experts:
 *   seg_offsets  int32 [n_seg+1] on the device: rows seg_offsets[e] .. seg_offsets[e+1]-1 of the sorted
 *                activations belong to expert e (non-decreasing, seg_offsets[0] = 0, seg_offsets[n_seg] <= M;
 *                an expert may own no row; rows behind the last segment are left untouched)
 *   reorder_index      int16 [n_seg, K]: one channel order per expert
 *   d_global_scales    fp32 [n_seg] on the device: one NVFP4 tensor scale per expert (max |x_e| / 2688,
 *                      model/qLlamaLayer.py:73-77 applied to the expert's tokens as model/qMixtralLayer.py:530
 *                      does), or NULL for tensor scale 1 everywhere (MXFP4)
 * Nothing is read back to the host.  Codes and scale bytes of a row are those arcq_reorder_quantize_x /
 * arcq_swiglu_quantize_x write for that row with its expert's index and scale.
 * arcq_grouped_tensor_scale writes the n_seg scales (1 for an expert without rows or with only zeros);
 * `up` as for arcq_tensor_scale.  K <= 32736 for the quantizers.
 */
int arcq_grouped_reorder_quantize_x(const void *x, int M, int K, const int *seg_offsets, int n_seg,
                                    const int16_t *reorder_index, int select_num, int fmt, const float *d_global_scales,
                                    void *codes, void *scales, void *stream);
int arcq_grouped_swiglu_quantize_x(const void *gate, const void *up, int ld, int M, int K, const int *seg_offsets, int n_seg,
                                   const int16_t *reorder_index, int select_num, int fmt, const float *d_global_scales,
                                   void *codes, void *scales, void *stream);
int arcq_grouped_tensor_scale(const void *x, const void *up, int ld, int M, int K, const int *seg_offsets, int n_seg,
                              float divisor, float *d_scales, void *stream);
/*
 * Grouped GEMM: rows seg_offsets[e] .. seg_offsets[e+1]-1 of C = alpha * alpha_a[e] * alpha_b[e] *
 * dq(A rows of e) @ dq(B_e)^T with expert e's weights B_e = b_codes + e * N * Kp/2 (scales likewise:
 * the experts' quantized weights stacked [n_seg, N, ...]).  One launch; every workgroup finds its
 * expert and tile from seg_offsets on the device.  Replaces the per-expert agemm.matmul calls of
 * model/qMixtralLayer.py:466-543 -> model/qLinearLayer.py:65-81.
 *   d_alpha_a, d_alpha_b  fp32 [n_seg] on the device or NULL (activation / weight tensor scales per expert)
 *   residual              NULL or bf16 [M, N], added as by arcq_matmul_add
 *   Kp                    multiple of 128, >= 512; scale arrays 16-byte aligned (else ARCQ_ERR_SHAPE / _ALIGN)
 */
int arcq_grouped_matmul(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                        const int *seg_offsets, int n_seg, int M, int N, int Kp, int fmt, float alpha,
                        const float *d_alpha_a, const float *d_alpha_b, const void *residual, void *c, void *stream);

/*
 * GEMM with the SwiGLU of the next layer fused into its epilogue, for a fused gate/up projection whose weight
 * rows ALTERNATE gate_0, up_0, gate_1, up_1, ... (quantize the interleaved bf16 weight with
 * arcq_reorder_quantize_w): output columns 2j and 2j+1 of a token then sit in one lane, and instead of the
 * [M, N] projection output the kernel writes t [M, N/2] = act_fn(gate) * up, formed from the bf16-rounded
 * GEMM outputs exactly as the reference's layers form it from the projection output in bf16
 * (model/qLlamaLayer.py:432, model/qMixtralLayer.py:531): the same bits as the unfused sequence, without the
 * projection output passing through memory.  No counterpart in the reference (it names the fusion,
 * benchmarks/modeling_arc.py:112, and does not ship it).
 *   d_absmax  NULL, or fp32 [n_seg] ([1] for arcq_matmul_swiglu) zeroed by the caller: receives max |t| per
 *             expert (as the bits of a non-negative float, i.e. readable as fp32), the numerator of the
 *             NVFP4 tensor scale of the next quantizer; arcq_scales_from_absmax turns the maxima into
 *             scales max / divisor in place (1 for a maximum of 0) with an IEEE division
 *   N multiple of 16; Kp multiple of 128, >= 512; other arguments as for arcq_grouped_matmul / arcq_matmul
 */
int arcq_grouped_matmul_swiglu(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                               const int *seg_offsets, int n_seg, int M, int N, int Kp, int fmt, float alpha,
                               const float *d_alpha_a, const float *d_alpha_b, void *t, float *d_absmax, void *stream);
int arcq_matmul_swiglu(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales, int M, int N,
                       int Kp, int fmt, float alpha, const float *d_alpha_a, const float *d_alpha_b, void *t,
                       float *d_absmax, void *stream);
int arcq_scales_from_absmax(float *d_values, int n, float divisor, void *stream);

/*
 * Routing of a mixture-of-experts block (model/qMixtralLayer.py:441-452: softmax over the experts in fp32,
 * top-k, the k weights divided by their sum and cast to bf16; :456-471 then visits expert after expert and the
 * tokens routed to it).  Two launches, nothing read back: besides each token's choice the call writes what the
 * grouped launches take -- the expert segments, and for every row of the expert-sorted order its token and its
 * weight (pairs of one expert in ascending (token, slot) order, as a stable sort by expert number gives).
 * The arithmetic is torch's on this device (its warp softmax's summation order, exp(l - max) / sum, the top-k
 * weights divided by their sum left to right), so the weights are the same bits for top_k = 2; among equal
 * probabilities the lower expert number is taken (torch.topk leaves that choice unspecified).
 *   logits        [tokens, experts] bf16, or fp32 if logits_f32
 *   sel           int32 [tokens * top_k]   expert of (token, slot), slots in descending probability
 *   weight        bf16  [tokens * top_k]   normalised router weight of (token, slot)
 *   seg_offsets   int32 [experts + 1]      rows seg[e] .. seg[e+1]-1 of the sorted order belong to expert e
 *   position      int64 [tokens * top_k]   sorted row of (token, slot) (what arcq_moe_combine takes)
 *   token_of_row  int32 [tokens * top_k]   token whose activations sorted row r reads
 *   weight_of_row bf16  [tokens * top_k]   router weight of sorted row r
 *   workspace     arcq_moe_route_workspace_bytes(tokens, experts) bytes of device memory, contents irrelevant
 * experts <= 64, top_k <= 8 and <= experts.
 */
size_t arcq_moe_route_workspace_bytes(int tokens, int experts);
int arcq_moe_route(const void *logits, int logits_f32, int tokens, int experts, int top_k, int *sel, void *weight,
                   int *seg_offsets, int64_t *position, int *token_of_row, void *weight_of_row, void *workspace,
                   size_t workspace_bytes, void *stream);

/*
 * Last step of a mixture-of-experts block: out[t] = sum over token t's experts, in ascending expert number, of
 * bf16(y[row] * weight[row]), every partial sum rounded to bf16 -- what model/qMixtralLayer.py:466-471 gets
 * from `expert(x) * routing_weights[...]` followed by final_hidden_states.index_add_ per expert.  One launch,
 * one read of every expert-output row, no atomics (reproducible).
 *   y         bf16 [pairs, H]: the expert outputs in expert-sorted row order (arcq_grouped_matmul's output)
 *   position  int64 [tokens * top_k] on the device: row of y holding token t's j-th expert (the inverse of the
 *             sort order); entries outside [0, pairs) contribute nothing
 *   weight    bf16 [pairs]: router weights in the same sorted order
 *   H multiple of 8, top_k <= 8
 */
int arcq_moe_combine(const void *y, const int64_t *position, const void *weight, int tokens, int H, int top_k, int pairs,
                     void *out, void *stream);

/*
 * INT4 paged KV cache (the reference's decode-attention path: agemm.init_kv_i4 / append_kv_i4 /
 * batch_decode_i4, kernels/src/bindings.cpp:287-413 -> kernels/src/flashinfer.cu:9-112, with the
 * torch-side quantizer asym_quantize_and_pack_i4, model/kv_cache.py:23-37, fused into the append).
 * Container layout as the reference allocates it (model/kv_cache.py:148-160):
 *   kv_data   u8 [pages, n_layers, 2 (k, v), kv_heads, page_size, head_dim/2], element 2j in the low nibble
 *   kv_param  [pages, n_layers, 2, kv_heads, page_size, 2] = (scale, zero) per (token, head) in `dtype`;
 *             a stored n stands for n * scale - zero (model/kv_cache.py:39-43)
 *   kv_indptr int32 [batch+1], kv_indices int32, last_page_offset int32 [batch]: sequence b owns pages
 *             kv_indices[kv_indptr[b] .. kv_indptr[b+1]) and holds (pages_b - 1) * page_size +
 *             last_page_offset[b] tokens
 * dtype: ARCQ_DTYPE_F16 (the reference's) or ARCQ_DTYPE_BF16, for k, v, q, o and kv_param alike.
 * head_dim must be 128 (flashinfer.cu:212-223 instantiates nothing else).
 *
 * arcq_kv_append_i4 quantizes new keys / values [tokens, kv_heads, 128] and writes them into their
 * pages; the page table describes the state AFTER the append (as model/kv_cache.py:228-262 passes it).
 *   seqlen_indptr  int32 [batch+1] offsets of each sequence's new tokens in k / v (prefill,
 *                  replaces init_kv_i4), or NULL for one new token per sequence (append_kv_i4)
 *   max_new_tokens upper bound of new tokens per sequence (sizes the launch)
 * arcq_kv_decode_i4: o[b, h, :] = softmax(q[b, h] . K_b^T * sm_scale) V_b over the dequantized cache, one
 * query token per sequence; q, o [batch, num_qo_heads, 128]; num_qo_heads / num_kv_heads in {1, 2, 4}
 * (the reference's kernel takes equal head counts only).  fp32 softmax and accumulation.
 */
enum { ARCQ_DTYPE_F16 = 0, ARCQ_DTYPE_BF16 = 1 };
int arcq_kv_append_i4(const void *k, const void *v, int dtype, int batch, const int32_t *seqlen_indptr, int max_new_tokens,
                      void *kv_data, void *kv_param, const int32_t *kv_indptr, const int32_t *kv_indices,
                      const int32_t *last_page_offset, int n_layers, int layer_idx, int num_kv_heads, int page_size,
                      int head_dim, void *stream);
/*
 * One decode step's work between the qkv projection and the attention, in one launch: rotary
 * embedding of the new token's query and key heads (apply_rotary_pos_emb, model/qLlamaLayer.py:30-64,
 * called at :316-321, evaluated as torch does on tensors of the model dtype) and the quantized
 * append of its key and value heads (past_key_value.update, model/qLlamaLayer.py:324-327 ->
 * model/kv_cache.py:194-276).
 *   qkv        [batch, ld] per sequence: num_qo_heads query heads, num_kv_heads key heads,
 *              num_kv_heads value heads, 128 values each; ld >= that, multiple of 8
 *   cos_table, sin_table  [max_positions, 64] in `dtype`: cos / sin of position x inverse frequency,
 *              shared by both halves of a head
 *   positions  int32 [batch] on the device: position of each sequence's new token (clamped into the tables)
 *   q_out      [batch, num_qo_heads, 128] rotated queries, input of arcq_kv_decode_i4
 * The page table describes the state AFTER the append, as for arcq_kv_append_i4.
 */
int arcq_rope_kv_append_i4(const void *qkv, int ld, int dtype, int batch, int num_qo_heads, const void *cos_table,
                           const void *sin_table, int max_positions, const int32_t *positions, void *q_out,
                           void *kv_data, void *kv_param, const int32_t *kv_indptr, const int32_t *kv_indices,
                           const int32_t *last_page_offset, int n_layers, int layer_idx, int num_kv_heads, int page_size,
                           int head_dim, void *stream);
/*
 * The rotary embedding alone, for prompts (apply_rotary_pos_emb, model/qLlamaLayer.py:30-64, evaluated as
 * torch does on tensors of the model dtype): token t of the flattened [sequences x q_len] batch sits at
 * position pos0 + t % q_len.  qkv [tokens, ld] as above; the rotated query heads go to q_out
 * [tokens, num_qo_heads, 128] and the rotated key heads to k_out [tokens, num_kv_heads, 128]; the value
 * heads are not touched.  One pass over q and k instead of torch's six.
 */
int arcq_rope(const void *qkv, int ld, int dtype, long tokens, int q_len, int pos0, int num_qo_heads, int num_kv_heads,
              int head_dim, const void *cos_table, const void *sin_table, int max_positions, void *q_out, void *k_out,
              void *stream);
/* the same scatter for rows the caller has quantized already -- the exact argument set of the
 * reference's init_kv_i4 (seqlen_indptr given) and append_kv_i4 (seqlen_indptr NULL):
 * k_codes / v_codes u8 [tokens, kv_heads, 64], k_param / v_param [tokens, kv_heads, 2] */
int arcq_kv_store_i4(const void *k_codes, const void *v_codes, const void *k_param, const void *v_param, int batch,
                     const int32_t *seqlen_indptr, int max_new_tokens, void *kv_data, void *kv_param,
                     const int32_t *kv_indptr, const int32_t *kv_indices, const int32_t *last_page_offset, int n_layers,
                     int layer_idx, int num_kv_heads, int page_size, int head_dim, void *stream);
int arcq_kv_decode_i4(void *o, const void *q, int dtype, int batch, int num_qo_heads, const void *kv_data,
                      const void *kv_param, const int32_t *kv_indptr, const int32_t *kv_indices,
                      const int32_t *last_page_offset, int n_layers, int layer_idx, int num_kv_heads, int page_size,
                      int head_dim, float sm_scale, void *stream);

/*
 * Debug helper: checks on the device that reorder_index is a permutation of 0..K-1 and
 * returns ARCQ_ERR_INDEX otherwise.  Synchronises `stream`.  The reference performs no such
 * check (kernels/src/reorder.cu:117 indexes shared memory with whatever it is given).
 */
int arcq_check_index(const int16_t *reorder_index, int K, void *stream);

/*
 * Test helper: expands codes+scales to fp32 values q*s, rows x Kp, on the device.
 */
int arcq_dequantize(const void *codes, const void *scales, int rows, int Kp, int fmt, float *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ARCQ_H_ */
