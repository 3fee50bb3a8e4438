/*
 * C ABI of the MI355X (gfx950) W4A16 GEMM library, libw4a16.so.
 *
 * It replaces, for AMD CDNA4, TurboMind's `turbomind::GemmS4F16` operator and the
 * `convert_s4` family of weight-repack functions of lmdeploy.  Every entry point takes
 * plain pointers and sizes; device pointers are caller-owned HIP device memory and
 * `stream` is a `hipStream_t` passed as `void*` (NULL = the default stream).  No entry
 * point synchronises the device except `w4a16_measure`.  Functions return 0 on success
 * or a negative W4A16_E* code and never throw; `w4a16_last_error()` returns a
 * thread-local message for the last failure.
 *
 * Naming of sizes: `n_out` = output features (the reference's `m`), `tokens` = rows of
 * the activation matrix (the reference's `n`), `k` = input features.  The reference
 * passes them in that order: LlamaLinear.h:65-75 calls
 * Run(out, kernel, in, scales_and_zeros, output_dims, batch_size, input_dims, ...).
 */
#ifndef W4A16_H_
#define W4A16_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define W4A16_OK 0
#define W4A16_EGROUP (-1)    /* unsupported group size (128, 64 and 32 have kernels) */
#define W4A16_ESHAPE (-2)    /* no feasible kernel for this shape            */
#define W4A16_EHIP (-3)      /* the HIP runtime reported an error            */
#define W4A16_EARG (-4)      /* null pointer / negative size / bad enum      */
#define W4A16_EALGO (-5)     /* algo_id out of range                         */
#define W4A16_ESCRATCH (-6)  /* the split-K scratch this launch needs is not available */
#define W4A16_ETIMEOUT (-7)  /* a device-wide barrier of w4a16_gemm_sequence gave up       */
#define W4A16_ETUNING (-8)   /* a tuning file was written by another library version or GPU */

/* epilogues; 0 and 1 are GemmS4F16::Type (gemm_s4_f16.h:23-27), 2 is an extension */
#define W4A16_GEMM 0
#define W4A16_FUSED_SILU_FFN 1
#define W4A16_FUSED_ADD 2

typedef struct w4a16_handle w4a16_handle;

/* One row of `w4a16_measure`; the counterpart of turbomind::Metric (metric.h:13-54). */
typedef struct w4a16_metric {
    int   id;          /* algo_id accepted by w4a16_gemm                        */
    int   feasible;    /* 1 if the kernel can run this shape                    */
    int   best;        /* 1 for the algo the heuristic (algo_id < 0) would pick */
    int   kind;        /* 0 = decode kernel (column blocks), 1 = MFMA prefill kernel, 2 = decode kernel (strips) */
    int   tile_n;      /* output features per workgroup                         */
    int   tile_t;      /* tokens per workgroup                                  */
    int   slices;      /* decode: K slices (wave groups) per workgroup; prefill: workgroups that split K */
    int   grid;        /* workgroups launched                                   */
    float ms;          /* total time of `count` launches, +inf if not feasible  */
    int   count;       /* number of timed launches                              */
} w4a16_metric;

/* GemmS4F16::GemmS4F16 / ~GemmS4F16 (gemm_s4_f16.h:19-21, gemm_s4_f16.cu:236-252).
 * The handle owns two events and 256 KiB of arrival counters; it binds to the current device.
 * A fixed 64 MiB workspace for split-K partial sums is allocated by the first launch that splits K
 * (some shapes between 17 and 512 tokens, narrow matrices at up to 16) and kept until
 * w4a16_destroy.  That first launch must not be under graph capture: there, a handle that has no
 * workspace yet uses kernels that need none (algo_id < 0) or fails with W4A16_ESCRATCH (explicit
 * algo_id).  GEMMs issued through one handle must be ordered on one stream at a time, because they
 * share that scratch.  A handle has no lock: one host thread uses it at a time.  Every call that
 * launches through a handle checks that the handle's device is the current one (W4A16_EARG if not). */
int  w4a16_create(w4a16_handle** out);
void w4a16_destroy(w4a16_handle* h);

/* GemmS4F16::Run (gemm_s4_f16.h:41-51, gemm_s4_f16.cu:208-234,284-297).
 *   C  fp16 [tokens, n_out]  (W4A16_FUSED_SILU_FFN: [tokens, n_out/2])
 *   A  repacked int4 weights from w4a16_convert_s4_k_m8, k*n_out/2 bytes
 *   X  fp16 [tokens, k] row-major (the reference's B)
 *   Q  half2 [k/group_size, n_out] from w4a16_convert_s4_k_m8
 *   R  fp16 [tokens, n_out] residual, W4A16_FUSED_ADD only (may alias C), else NULL
 * Computes C = epilogue(X * dequant(A, Q)) with fp32 accumulation:
 *   W4A16_GEMM            C[t,n] = fp16(acc[t,n])                      (gemm_s4_f16.cu:22-29)
 *   W4A16_FUSED_SILU_FFN  g = fp16(acc[t,2j]), u = fp16(acc[t,2j+1]);
 *                         C[t,j] = fp16(g / (1 + exp(-g)) * u)         (gemm_s4_f16.cu:31-42)
 *   W4A16_FUSED_ADD       C[t,n] = fp16(float(R[t,n]) + float(fp16(acc[t,n])))
 *                         (no counterpart in GemmS4F16; the add of
 *                          llama_decoder_kernels.cu:52-57 applied as in LlamaDecoder.cc:228-235)
 * algo_id < 0 selects a kernel by heuristic (gemm_s4_f16.cu:184-206 `Estimate`).
 * group_size: 128 is the reference's only one (gemm_s4_f16.cu:243-245, "TODO: add more group sizes") and has
 * the whole kernel table.  64 and 32 are an extension served by one kernel family (strips of up to four column
 * tiles, 16 tokens per workgroup, the weights streamed once per 16 tokens): they take algo_id < 0 only
 * (W4A16_EALGO otherwise), w4a16_measure refuses them, and a persistent w4a16_gemm_sequence runs them as one
 * launch per GEMM.  Any other value: W4A16_EGROUP, "unsupported group size" (gemm_s4_f16.cu:119,233).
 * Requires k % 128 == 0 (weight tiles are 128 rows whatever the group size), n_out % 16 == 0, tokens >= 0; A and X aligned to 16
 * bytes, Q to 4, C and R to 4 (to 8 when an MFMA prefill kernel runs, i.e. above 32 tokens, except
 * for W4A16_FUSED_SILU_FFN).
 * Numerics: the kernels for up to 32 tokens (and narrow matrices up to ~128) scale each group's
 * fp32 partial sum by the fp16 scale; the MFMA prefill kernels multiply by the fp16 weight
 * fp16((q - z) * s).  Both treat a subnormal scale as zero, which is all that the reference's
 * flush-to-zero multiply (common.h:229-230 mul.ftz) ever does: a normal scale times a non-zero
 * integer is never subnormal.  The two families are within the 1e-2 tolerance of each other and of
 * the reference, but not bit-identical: the same input can give different bits on the
 * two sides of a hand-over point between kernel families. */
int w4a16_gemm(w4a16_handle* h, void* C, const void* A, const void* X, const void* Q, const void* R,
               int n_out, int tokens, int k, int group_size, int epilogue, int algo_id, void* stream);

/* w4a16_gemm for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  It takes
 * no handle (creating one allocates); where w4a16_gemm's split-K kernels use the handle's workspace,
 * this entry point uses a buffer that is part of the library's code object: 8 MiB of partial tiles
 * plus 4096 arrival counters, resident on every GPU the library runs on until the process ends.
 * Arguments, results and error codes are those of w4a16_gemm.  algo_id < 0 picks among the kernels
 * whose scratch fits that buffer; an explicit algo_id whose partial tiles for this shape do not
 * fit (n_out * tokens (padded to the tile) * splits * 4 bytes > 8 MiB, or more than 4096 output
 * tiles) fails with W4A16_ESCRATCH.  It calls no allocating routine; the buffer's device address
 * is looked up (hipGetSymbolAddress) by the first call on a device or by w4a16_create.  All calls
 * on one GPU share the one buffer: calls that can overlap on the GPU (different streams, or
 * different threads) race, so order them on one stream.  The counters a launch will use are cleared by
 * a small fill kernel before it. */
int w4a16_gemm_static(void* C, const void* A, const void* X, const void* Q, const void* R, int n_out, int tokens,
                      int k, int group_size, int epilogue, int algo_id, void* stream);

/* One GEMM of a sequence: the arguments of w4a16_gemm that differ from GEMM to GEMM. */
typedef struct w4a16_gemm_desc {
    void*       C;
    const void* A;
    const void* X;
    const void* Q;
    const void* R;        /* residual for W4A16_FUSED_ADD (may alias C), else NULL                    */
    int         n_out;
    int         k;
    int         epilogue;
    int         depends;  /* non-zero: this GEMM reads (X or R) what an earlier GEMM of the list writes,
                             or writes what an earlier one reads or writes; 0: it may overlap with them */
} w4a16_gemm_desc;

/* A list of GEMMs with a common token count, executed as if by `count` calls of w4a16_gemm (algo_id
 * -1) in list order, e.g. the four GEMMs of a decoder layer (LlamaDecoder.cc:205-235:
 * qkv, o - LlamaDecoderSelfAttentionLayer.cc:236-292 -, then LlamaFfnLayer.cc:87-103), or those of
 * several layers.
 * flags = 0: one launch per GEMM on `stream`.
 * flags = W4A16_SEQ_PERSISTENT, up to 16 tokens: the whole list (32 GEMMs at a time) runs as ONE
 * persistent launch of one workgroup per CU.  A GEMM with `depends` set starts behind a device-wide
 * barrier (outputs written through at agent scope, arrival on a two-level counter tree, activations
 * read at agent scope), across which the first weight tiles of the next GEMM are already in flight.
 * Results are bit-identical to w4a16_gemm with the strip kernel (one strip per CU).  Measured on
 * MI355X this is SLOWER than one launch per GEMM (a Llama-2-7B layer at 8 tokens: 44 us against 34
 * us inside a HIP graph): crossing the barrier costs 3 - 4.5 us per GEMM, a launch about 3 us.  It is
 * kept for callers for whom launches are dearer than that (no graphs, a busy host thread).
 * The persistent launch needs its workgroups resident all at once, which holds when nothing else
 * occupies the GPU's CUs for long; its barrier waits are bounded (w4a16_set_barrier_timeout, default
 * 50 ms): a workgroup that gives up sets an error word in the handle, and every workgroup still
 * finishes.  The error word is sticky: until w4a16_sequence_status has been called, every later
 * persistent launch on this handle passes its barriers without waiting, so its outputs are
 * undefined too.  A caller that replays a captured persistent launch must therefore poll
 * w4a16_sequence_status (between replays; it synchronises the stream).  Nothing is allocated and nothing synchronises, so the call can be captured in a HIP
 * graph (for T > 16, and for matrices that split K, after one call outside capture: see w4a16_create). */
#define W4A16_SEQ_PERSISTENT 1
int w4a16_gemm_sequence(w4a16_handle* h, const w4a16_gemm_desc* gemms, int count, int tokens, int group_size,
                        int flags, void* stream);

/* Synchronises `stream` and reports whether a barrier of an earlier w4a16_gemm_sequence on this handle
 * gave up: W4A16_OK, or W4A16_ETIMEOUT (once; the barrier state is then cleared on `stream` and the handle
 * is usable again).  Outputs of every persistent launch between the timeout and this call are undefined. */
int w4a16_sequence_status(w4a16_handle* h, void* stream);

/* Time limit of one barrier wait of w4a16_gemm_sequence, 0 .. 3600 seconds. */
int w4a16_set_barrier_timeout(w4a16_handle* h, double seconds);

/* The int4 branch of LlamaFfnLayer<T>::forward (src/turbomind/models/llama/LlamaFfnLayer.cc:67-116)
 * as one call: gating = SiLU-gated fused gate/up GEMM (kFusedSiluFfn) into `gating_buf`
 * [tokens, inter_size], then ffn_output = gating * W2 (+ residual if `residual` is not null: the add
 * half of the fused add-norm that follows in LlamaDecoder.cc:228-235; `residual` may alias
 * `ffn_output`).  A13/Q13 are the converted fused w1|w3 weights (n_out = 2 * inter_size, k =
 * hidden_units), A2/Q2 the converted w2 (n_out = hidden_units, k = inter_size).  It is the two-GEMM
 * w4a16_gemm_sequence with flags 0: two launches back to back on `stream` (a single persistent
 * launch was built and measured slower, see there).  Nothing is allocated, so the call can be
 * captured in a HIP graph. */
int w4a16_ffn(w4a16_handle* h, void* ffn_output, void* gating_buf, const void* ffn_input, const void* A13,
              const void* Q13, const void* A2, const void* Q2, const void* residual, int hidden_units,
              int inter_size, int tokens, int group_size, void* stream);

/* GemmS4F16::Measure (gemm_s4_f16.h:29-39, gemm_s4_f16.cu:98-169): times every feasible
 * kernel (10 warm-up + 100 timed launches each) and writes up to `capacity` rows sorted
 * by time; returns the number of rows, or a negative error.  Synchronises `stream` (so it cannot
 * run under capture).  The handle remembers the fastest kernel for (n_out, tokens, k); later
 * `w4a16_gemm` calls with algo_id < 0 and exactly that shape use it (see `w4a16_pick`).  Because
 * kernel families round differently (see w4a16_gemm), a Measure call can change the low bits that
 * later w4a16_gemm calls of that shape return; `w4a16_clear_tuning` restores the heuristic. */
int w4a16_measure(w4a16_handle* h, void* C, const void* A, const void* X, const void* Q, const void* R,
                  int n_out, int tokens, int k, int group_size, int epilogue,
                  w4a16_metric* metrics, int capacity, void* stream);

/* The algo_id that `w4a16_gemm(..., algo_id = -1, ...)` would use for this shape: the fastest one a
 * previous `w4a16_measure` on this handle found for exactly (n_out, tokens, k), else the heuristic's
 * choice.  The reference's Measure only reports (gemm_s4_f16.cu:98-169) and its Run always
 * estimates (gemm_s4_f16.cu:171-182); remembering the measurement is an extension.  Host-only. */
int w4a16_pick(const w4a16_handle* h, int n_out, int tokens, int k);

/* Forgets every measurement remembered by `w4a16_measure` on this handle. */
int w4a16_clear_tuning(w4a16_handle* h);

/* Writes what w4a16_measure has remembered on this handle to a text file, and reads such a file back into a
 * handle, so that a machine measures its shapes once (boxes of one GPU model have differed by up to 19 % on the
 * same kernel, and with them the best choice).  The file names the library version, the CU count of the device
 * and the size of the kernel table; w4a16_load_tuning refuses a file whose three do not match the running
 * library and the handle's device (W4A16_ETUNING, nothing loaded).  Both return the number of shapes written /
 * taken over (entries whose kernel cannot run the shape are skipped), or a negative error.  An extension like
 * w4a16_pick: the reference's Measure only reports (gemm_s4_f16.cu:98-169).  Host-only. */
int w4a16_save_tuning(const w4a16_handle* h, const char* path);
int w4a16_load_tuning(w4a16_handle* h, const char* path);

/* Number of kernels `w4a16_gemm` can dispatch to (valid algo_id are 0 .. count-1). */
int w4a16_algo_count(void);

/* convert_s4_k_m8 (format.h:15-24, format.cu:97-113).  Inputs are the AWQ tensors
 *   A_src  uint32 [k, m/8], qzeros uint32 [k/group_size, m/8], scales fp16 [k/group_size, m]
 * (pack order of lmdeploy/pytorch/modules/linear.py:85,105-108).  Outputs
 *   A_dst  uint32 [k*m/8]  weights in the gfx950 tiled layout (same byte count as A_src)
 *   Q_dst  half2  [k/group_size, m] = (64 + zero, scale), bit-identical to the reference's
 * `workspace` (k/group_size*m halves) is accepted for signature compatibility and unused.
 * m = output features, must be a multiple of 16; k a multiple of 128; group_size 128, 64 or 32 (the weight
 * layout does not depend on it, Q has k / group_size rows). */
int w4a16_convert_s4_k_m8(uint32_t* A_dst, void* Q_dst, void* workspace, const uint32_t* A_src,
                          const void* scales, const uint32_t* qzeros, int m, int k, int group_size,
                          void* stream);

/* The fused q|k|v matrix of a decoder layer, straight from the three AWQ tensors of the checkpoint:
 * what deploy_awq does with transpose_qk_s4 on q and k (lmdeploy/serve/turbomind/deploy.py:633-639;
 * scales by `permute`, :371-383), merge_qkv (:251-260) and convert_s4 (:660-670), in one gather.
 * qweight[i] uint32 [k, n_i/8], qzeros[i] uint32 [k/group_size, n_i/8], scales[i] fp16 [k/group_size, n_i] for
 * i = q, k, v with n = n_q, n_kv, n_kv.  Within every head of size_per_head columns of q and k,
 * output column 2i + r is source column r * size_per_head/2 + i.  A_dst: k * (n_q + 2 n_kv) / 2
 * bytes, Q_dst: half2 [k/group_size, n_q + 2 n_kv]. */
int w4a16_deploy_qkv(uint32_t* A_dst, void* Q_dst, const uint32_t* const qweight[3], const uint32_t* const qzeros[3],
                     const void* const scales[3], int n_q, int n_kv, int k, int size_per_head, int group_size,
                     void* stream);

/* The fused gate|up matrix (w13) from the AWQ tensors of gate_proj (w1) and up_proj (w3): what
 * deploy_awq does with fuse_w1_w3_s4 (deploy.py:641-658: output column 2j = w1 column j, 2j + 1 =
 * w3 column j, for weights, zeros and scales) and convert_s4 (:660-670), in one gather.
 * A_dst: k * 2 * inter_size / 2 bytes, Q_dst: half2 [k/group_size, 2 * inter_size]. */
int w4a16_deploy_w13(uint32_t* A_dst, void* Q_dst, const uint32_t* w1_qweight, const uint32_t* w3_qweight,
                     const uint32_t* w1_qzeros, const uint32_t* w3_qzeros, const void* w1_scales, const void* w3_scales,
                     int inter_size, int k, int group_size, void* stream);

/* reformat_s4_k_m8 (format.h:13, format.cu:69-75): the weight half of the conversion alone,
 * AWQ words [k, m/8] -> the tiled layout the GEMM kernels read (here the gfx950 one).
 * format.h:11 `reformat_s4_k8_m` is an unused alternative layout and has no counterpart. */
int w4a16_reformat_s4_k_m8(uint32_t* dst, const uint32_t* src, int m, int k, void* stream);

/* fuse_w1_w3_s4_k_m8 (format.h:28, format.cu:123-130): AWQ-packed cat(w1, w3) [2, k, m/8]
 * -> AWQ-packed [k, 2m/8] with logical column 2j = w1[:, j], 2j+1 = w3[:, j]. */
int w4a16_fuse_w1_w3_s4_k_m8(uint32_t* dst, const uint32_t* src, int m, int k, void* stream);

/* transpose_qk_s4_k_m8_hf (format.h:26, format.cu:115-121): AWQ-packed [k, m/8]; within
 * every head of size_per_head columns, dst column 2i+r = src column r*size_per_head/2 + i. */
int w4a16_transpose_qk_s4_k_m8_hf(uint32_t* dst, const uint32_t* src, int m, int k, int size_per_head,
                                  void* stream);

/* dequantize_s4 (format.h:30, format.cu:132-142): `count` AWQ words -> 8*count fp16 holding
 * the raw nibble values in logical column order.  Runs on `stream` (the reference ignores it). */
int w4a16_dequantize_s4(void* dst, const uint32_t* src, size_t count, void* stream);

/* Inverse of w4a16_convert_s4_k_m8 (no counterpart in the reference; exists so that the
 * repack can be checked bit for bit): recovers the AWQ tensors from (A, Q).  Any of the
 * three outputs may be NULL. */
int w4a16_unpack_repacked(uint32_t* qweight, uint32_t* qzeros, void* scales, const uint32_t* A,
                          const void* Q, int m, int k, int group_size, void* stream);

/* Dequantised weights W fp16 [k, m] row-major from (A, Q), computed exactly as the
 * reference kernel does (common.h:218-235): W = mul.ftz(sub.ftz(64+q, 64+z), s). */
int w4a16_dequantize_repacked(void* W, const uint32_t* A, const void* Q, int m, int k, int group_size,
                              void* stream);

/* Converts weights already in the REFERENCE's tiled layout (output of its
 * convert_s4_k_m8, i.e. a `.qweight` file written by deploy.py:142-146) to the gfx950
 * layout.  Q needs no conversion.  m % 32 == 0, k % 128 == 0. */
int w4a16_from_reference_layout(uint32_t* A_dst, const uint32_t* A_ref, int m, int k, void* stream);

const char* w4a16_last_error(void);
const char* w4a16_version(void);

#ifdef __cplusplus
}
#endif
#endif /* W4A16_H_ */
