/*
 * C ABI of libnt_hip.so: hand-written gfx950 (MI355X) kernels for the programs
 * that ninetoothed.make produces (tiled matmul / addmm, row softmax, fused
 * scaled-dot-product attention forward, conv2d as implicit GEMM).
 *
 * The type layer is the one the reference emits into its generated
 * `ninetoothed.h` (reference: src/ninetoothed/aot.py:558-586): tensors travel
 * BY VALUE as {data, shape, strides} with strides counted in ELEMENTS, the
 * stream is an opaque pointer (a hipStream_t here), and every launch function
 * returns an int: 0 on success, a hipError_t value when the runtime refuses
 * the launch, NINETOOTHED_NO_KERNEL (1) when no kernel exists for the given
 * configuration (reference: src/ninetoothed/build.py:167-170 `return 1;`).
 * Zero-dimensional tensors carry scalars: `data` points to a HOST double
 * (floating point) or a HOST int64_t (integer / boolean), `shape` and
 * `strides` are not read (reference: src/ninetoothed/aot.py:725-733, 624-628).
 *
 * Launches are asynchronous on the given stream and never synchronise; the
 * caller owns every tensor.  Only launch_nt_conv2d, launch_nt_attention on
 * FLOAT32 tensors, on tensors it cannot read in place (see there) or on few query blocks against many keys (split key range:
 * parts x batch x heads x seq_q x (head_dim + 1) floats; not when the caller
 * passes block sizes), and launch_nt_matmul / launch_nt_addmm on problems with few
 * output tiles and a long K (split-K: parts x M x N floats, at most 64 MiB; not
 * when the caller passes block sizes), on FLOAT8_E5M2 operands (fp16 copies of the operands, and of addmm's
 * input: 2 bytes per element) or, from 2^21 multiply-adds on, on fp16 / bf16 operands that the direct-to-LDS kernels
 * cannot read in place (dense copies, (M + N) x K elements) use scratch device memory: one buffer per (device, stream,
 * purpose) that the library allocates (hipMalloc) the first time a call needs
 * it, grows (hipFree + hipMalloc, which wait for the device) when a later call
 * needs more, and otherwise reuses, so that steady-state calls allocate
 * nothing; nt_release_workspaces frees them.  Every other launch allocates
 * nothing.  All functions may be called from several host threads.
 */
#ifndef NINETOOTHED_HIP_H
#define NINETOOTHED_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NINETOOTHED_TRUE 1
#define NINETOOTHED_FALSE 0
#define NINETOOTHED_NONE 0

/* returned when no kernel matches the request (dtype / rank / block sizes) */
#define NINETOOTHED_NO_KERNEL 1

/* returned by launch_nt_matmul_static_scratch when the call would need more scratch memory than the
 * library's fixed array holds (NINETOOTHED_STATIC_SCRATCH_BYTES); nothing has been launched then */
#define NINETOOTHED_SCRATCH_LIMIT 2
#define NINETOOTHED_STATIC_SCRATCH_BYTES (16u << 20)

/* same member order as the reference's enum (src/ninetoothed/aot.py:524-537) */
enum NineToothedDataType {
    NINETOOTHED_INT8,
    NINETOOTHED_INT16,
    NINETOOTHED_INT32,
    NINETOOTHED_INT64,
    NINETOOTHED_UINT8,
    NINETOOTHED_UINT16,
    NINETOOTHED_UINT32,
    NINETOOTHED_UINT64,
    NINETOOTHED_FLOAT16,
    NINETOOTHED_BFLOAT16,
    NINETOOTHED_FLOAT32,
    NINETOOTHED_FLOAT64,
    /* extension beyond the reference's enum: 8-bit floating point with 5 exponent
     * and 2 mantissa bits, the operand type of the second case of
     * tests/test_matmul.py:61-88 and tests/test_addmm.py:57-90; accepted by
     * launch_nt_matmul and launch_nt_addmm (input, mat1, mat2 fp8, output fp16).
     * An e5m2 value is the upper byte of the fp16 value it equals: the operands are
     * widened exactly into fp16 copies in the stream's scratch buffers and the product runs
     * on the fp16 kernels (products exact, sums in fp32); without scratch memory (graph
     * capture before an eager call of the same size) a kernel that widens while it loads
     * serves the call, much slower. */
    NINETOOTHED_FLOAT8_E5M2
};

typedef struct {
    void *data;
    uint64_t *shape;
    int64_t *strides;
} NineToothedTensor;

typedef void *NineToothedStream;

typedef int NineToothedResult;

/*
 * Block-size arguments (`block_size_*`) are the values of the arrangement's
 * meta symbols.  0 means "library's choice" (the tuned / heuristic tile); a
 * positive value is honoured when a kernel instance with that tile exists and
 * otherwise mapped to the nearest instance -- results do not depend on it.
 */

/* output[M,N] = lhs[M,K] @ rhs[K,N], fp32 accumulation, one rounding on store.
 * Replaces the kernel generated for tests/test_matmul.py:14-45 (== README.md:40-62):
 * generated launch function src/ninetoothed/generation.py:545-600.
 * `dtype` is the element type of lhs/rhs; `output_dtype` that of output
 * (FLOAT16, BFLOAT16 or FLOAT32).  Any strides are accepted.
 * FLOAT32 operands (output FLOAT32) are multiplied as they are on the fp32
 * MFMA (32x32x2), products and sums in fp32, by the any-stride kernel.
 * FLOAT8_E5M2 operands (output FLOAT16 or FLOAT32) are widened to fp16 on the
 * way into LDS -- exact, the format is the upper byte of fp16 -- and multiplied
 * on the fp16 MFMA path with fp32 accumulation. */
NineToothedResult launch_nt_matmul(NineToothedStream stream,
                                   NineToothedTensor lhs,
                                   NineToothedTensor rhs,
                                   NineToothedTensor output,
                                   int dtype, int output_dtype,
                                   int block_size_m, int block_size_n,
                                   int block_size_k);

/* output[b] = lhs[b] @ rhs[b] for tensors [B, M, K], [B, K, N], [B, M, N]: the kernel the reference generates
 * (src/ninetoothed/generation.py:46-133) for the matmul application of tests/test_matmul.py:41-45 under an
 * arrangement that tiles a leading batch dimension by 1 (`tile((1, BLOCK_SIZE_M, BLOCK_SIZE_N))`, the level
 * squeezed) -- the reference has no test of its own for it.  One launch: the grid holds tiles x B workgroups.
 * An operand whose first extent is 1 is shared by all products; everything else as launch_nt_matmul (the
 * fast instances need batch strides that are multiples of 8 elements; FLOAT8_E5M2 operands are not taken). */
NineToothedResult launch_nt_batched_matmul(NineToothedStream stream,
                                           NineToothedTensor lhs,
                                           NineToothedTensor rhs,
                                           NineToothedTensor output,
                                           int dtype, int output_dtype,
                                           int block_size_m, int block_size_n,
                                           int block_size_k);

/* output = beta * input + alpha * round_to_dtype(mat1 @ mat2), epilogue in fp32.
 * Replaces the kernel generated for tests/test_addmm.py:13-38 (argument order
 * input, mat1, mat2, beta, alpha, output as in its application).  beta and
 * alpha are 0-d tensors holding a host double.  dtype FLOAT32: all four tensors
 * hold fp32 and the product is not rounded. */
NineToothedResult launch_nt_addmm(NineToothedStream stream,
                                  NineToothedTensor input,
                                  NineToothedTensor mat1,
                                  NineToothedTensor mat2,
                                  NineToothedTensor beta,
                                  NineToothedTensor alpha,
                                  NineToothedTensor output,
                                  int dtype,
                                  int block_size_m, int block_size_n,
                                  int block_size_k);

/* output[r, :] = softmax(input[r, :]) over the last of two dims, in fp32
 * arithmetic.  Replaces the kernel generated for tests/test_softmax.py:10-27
 * (one program per row, BLOCK_SIZE >= row length).  Up to 128 row segments of
 * 64 KiB or more each (256 KiB where a segment fits the registers of one
 * workgroup, and then up to 16) are cut into parts that run on as many
 * workgroups, in two launches; the parts' maxima and sums (8 bytes each, at
 * most 256 per segment) go through a scratch buffer of `stream`, without which
 * one workgroup per segment runs. */
NineToothedResult launch_nt_softmax(NineToothedStream stream,
                                    NineToothedTensor input,
                                    NineToothedTensor output,
                                    int dtype, int block_size);

/* Same as launch_nt_softmax with the kernel variant fixed: 0 = library's
 * choice, 1 = one wavefront per row segment, 2 = one workgroup per row segment
 * (measurement aid of the tile selection; no counterpart in the reference). */
NineToothedResult launch_nt_softmax_config(NineToothedStream stream, int config,
                                           NineToothedTensor input,
                                           NineToothedTensor output,
                                           int dtype, int block_size);

/* o = softmax(scale * q k^T [+ causal mask]) v for q,k,v,o of shape
 * [batch, heads, seq, head_dim] (k/v may have their own seq length).
 * Replaces the kernel generated for tests/test_attention.py:14-70; that
 * program has scale == 1, the scale tensor (0-d, host double) is this
 * library's extension for the 1/sqrt(head_dim) configuration.
 * is_causal is a 0-d tensor holding a host int64_t.
 * dtype FLOAT16 / BFLOAT16, or FLOAT32 (the fp32 case of
 * tests/test_attention.py:99-117, rtol = atol = 0.025 there).  FLOAT32 tensors
 * with head_dim 32, 64 or 128 and no block-size hints run in fp32 throughout on
 * the fp32 MFMA (a sixteenth of the fp16 rate, nothing narrowed, no scratch
 * memory).  Other head dimensions, and calls that give a hint -- the fast way
 * -- run on fp16 copies: K and V are first narrowed into the library's scratch
 * buffer of `stream`, Q is narrowed while it is scaled, the products run on
 * the fp16 MFMA path with fp32 accumulation and O is written unrounded.
 * block_size_m / block_size_n are hints (0 = library's choice): block_size_m
 * >= 256 selects 256 query rows per workgroup, block_size_n <= 32 the 32-key
 * blocks with three workgroups per CU, block_size_n >= 64 the plain 64-key
 * loop; without hints a call runs the variant recorded for its problem by
 * nt_tune_attention, else the software-pipelined 64-key loop (non-causal: with
 * 256 query rows and eight waves per workgroup when that still fills the chip
 * twice).  Without a scale tensor the scores are scaled by log2(e) rounded to
 * the element type, as the reference program's literal is.  On the fp16
 * copies of FLOAT32 tensors values beyond the fp16 range overflow, which the
 * reference's fp32 kernel does not.  K and V of one (batch, head) must span
 * less than 4 GiB (16-bit tensors).
 * head_dim: 32, 64, 128 and 256 have kernels of their size; any other multiple of
 * 8 up to 256 runs on the next of these sizes with the missing columns read as
 * zeros (K and V of one (batch, head) then span less than 2 GiB).  Head dimensions up to 256 that are no multiples
 * of 8, a last dimension with another stride than 1, and tensors whose rows do not start on 16-byte boundaries run on
 * padded dense copies of Q, K and V in the stream's scratch buffers (4 x batch x heads x seq x head_dim rounded up
 * to 8 elements), with O copied back; a head dimension above 256 returns NINETOOTHED_NO_KERNEL. */
NineToothedResult launch_nt_attention(NineToothedStream stream,
                                      NineToothedTensor q,
                                      NineToothedTensor k,
                                      NineToothedTensor v,
                                      NineToothedTensor is_causal,
                                      NineToothedTensor scale,
                                      NineToothedTensor o,
                                      int dtype,
                                      int block_size_m, int block_size_n);

/* output[N,K,P,Q] = conv2d(input[N,C,H,W], filter[K,C,R,S]) with stride 1,
 * dilation 1 (launch_nt_conv2d_strided takes others) and zero padding (padding_h, padding_w), computed as the implicit
 * GEMM [N*P*Q, C*R*S] x [C*R*S, K] the arrangement of
 * tests/test_conv2d.py:13-48 describes.
 * Ways to run it, tried in this order unless block_size_m names one (4, 3, 2, 1)
 * or nt_tune_conv2d has recorded one for the problem:
 * 4 -- 1 x 1 filters without padding (P*Q and C multiples of 8): one batched
 *   launch of the GEMM kernels on the tensors as they lie, without scratch;
 * 3 -- one launch on the tensors as they lie, no scratch memory: the filter is
 *   the row-major left operand, rows of the right operand are (channel, filter
 *   tap)-shifted pixel runs of the NCHW input; needs an output width that is a
 *   multiple of 8, padding_w <= 1, C*R*S a multiple of 32, R*S / gcd(32, R*S) <= 25, pixels of an input row
 *   contiguous, contiguous filter and output, K filling 256-wide tiles to 4/5;
 * 2 -- fp16 / bf16 tensors of any strides (a contiguous NCHW output is stored in
 *   16-byte pieces of 8 positions, a channels-last one in pieces of 8 channels,
 *   any other element by element): the
 *   input is first repacked to channels-last (a contiguous channels-last input
 *   with C' == C is read where it is) and the filter to [R*S*C', K']
 *   (C' = C rounded up to a multiple of 32 -- to 8 or 16 for up to 16 channels --, K' = K
 *   rounded up to 8, zero filled) in the library's scratch
 *   buffers of `stream` (N*C'*H*W + K'*C'*R*S elements), then the direct-to-LDS
 *   GEMM loop runs;
 * 1 -- the scratch-free gather kernel, which serves every shape, and calls whose
 *   scratch cannot be allocated (out of memory; a stream under graph capture that
 *   has no buffer yet).
 * FLOAT32 tensors run on way 1 with the fp32 MFMA. */
NineToothedResult launch_nt_conv2d(NineToothedStream stream,
                                   NineToothedTensor input,
                                   NineToothedTensor filter,
                                   NineToothedTensor output,
                                   int dtype,
                                   int padding_h, int padding_w,
                                   int block_size_m, int block_size_n,
                                   int block_size_k);

/* launch_nt_conv2d for windows that move by (stride_h, stride_w) over the padded input and whose taps lie
 * (dilation_h, dilation_w) apart: output position (p, q) and tap (r, s) read input (p * stride_h + r * dilation_h -
 * padding_h, q * stride_w + s * dilation_w - padding_w), zeros outside the input.  This is the arrangement of
 * tests/test_conv2d.py:28-36 with `tile(..., strides=(-1, -1, stride_h, stride_w), dilation=(1, 1, dilation_h,
 * dilation_w))` (src/ninetoothed/tensor.py:199-286).  The output holds, per dimension, either the windows that fit
 * (`floor_mode=True`: (H + 2 padding - dilation (R - 1) - 1) / stride + 1, rounded down) or one more that hangs over
 * the edge (`Tensor.tile`'s default rounds up; what hangs over reads as padding); other sizes are rejected.
 * Steps of 1 with the fitting output are launch_nt_conv2d.  Otherwise way 2 (repacking pass plus GEMM loop, same
 * conditions and scratch buffers) or way 1 (gather kernel) runs; block_size_m = 2 or 1 names one. */
NineToothedResult launch_nt_conv2d_strided(NineToothedStream stream,
                                           NineToothedTensor input,
                                           NineToothedTensor filter,
                                           NineToothedTensor output,
                                           int dtype,
                                           int padding_h, int padding_w,
                                           int stride_h, int stride_w,
                                           int dilation_h, int dilation_w,
                                           int block_size_m, int block_size_n,
                                           int block_size_k);

/*
 * launch_nt_matmul for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 *
 * Same arguments, kernels, tile choice and results as launch_nt_matmul.  The difference is where the
 * partial products of a split-K launch go (problems with few output tiles and a long K: parts x M x N
 * floats): not into a workspace that the library allocates, but into a fixed array of
 * NINETOOTHED_STATIC_SCRATCH_BYTES (16 MiB) that is part of the library's code object -- every GPU the
 * library runs on holds its copy until the process ends.  This function never calls hipMalloc / hipFree
 * or any allocating routine.  When the partial products of the split that launch_nt_matmul would use
 * exceed the array, the K range is cut into as many parts as fit (same kernels, another summation order);
 * a call for which not even two parts fit (M x N x 8 bytes > the array) returns
 * NINETOOTHED_SCRATCH_LIMIT and launches nothing (it does not fall back to another kernel); problems
 * that run in one pass need no scratch memory and are accepted at any size (the untuned choice splits
 * only products of fewer than 256 tiles of 64 x 64, which always fit; a tuned choice may name a split-K
 * instance for a larger one).  fp32 products and products a few tiles over whole rounds of the chip, whose
 * partial products launch_nt_matmul puts into allocated buffers, run in one pass here.  Operands that
 * launch_nt_matmul would copy into allocated buffers (FLOAT8_E5M2; fp16 / bf16 operands that the
 * direct-to-LDS kernels cannot read in place) run here on the kernels that read them in place, slower.
 *
 * All calls on one GPU share that GPU's array, on whatever stream: calls whose kernels may overlap on a
 * GPU (different streams, or replays of graphs captured from them) race on it and must be ordered by the
 * caller.  Every launch overwrites all of the array it later reads, so nothing has to be cleared between
 * calls.
 */
NineToothedResult launch_nt_matmul_static_scratch(NineToothedStream stream,
                                                  NineToothedTensor lhs,
                                                  NineToothedTensor rhs,
                                                  NineToothedTensor output,
                                                  int dtype, int output_dtype,
                                                  int block_size_m, int block_size_n,
                                                  int block_size_k);

/* ---- tile selection (stands in for the reference's Triton autotuner,
 * src/ninetoothed/generation.py:372-516 and src/ninetoothed/auto_tuner.py:11-152) ---- */

/* Number of GEMM kernel instances compiled into the library. */
int nt_gemm_num_configs(void);

/* Writes a short description ("256x256x64 w8 s2 ...") of instance `config`
 * into `buffer` (at most `size` bytes, NUL terminated).  Returns 0, or
 * NINETOOTHED_NO_KERNEL for an unknown index. */
NineToothedResult nt_gemm_config_name(int config, char *buffer, int size);

/* Runs instance `config` (as launch_nt_addmm when input.data != NULL, as
 * launch_nt_matmul otherwise).  Returns NINETOOTHED_NO_KERNEL when the
 * instance cannot handle the shapes / strides given. */
NineToothedResult launch_nt_gemm_config(NineToothedStream stream, int config,
                                        NineToothedTensor input,
                                        NineToothedTensor mat1,
                                        NineToothedTensor mat2,
                                        NineToothedTensor beta,
                                        NineToothedTensor alpha,
                                        NineToothedTensor output,
                                        int dtype, int output_dtype);

/* Times every instance that accepts the problem with hipEvents on `stream` and stores
 * the winner in the per-device cache that launch_nt_matmul / launch_nt_addmm
 * consult when block sizes are 0.  How: the instance of the untuned rule first
 * runs untimed for about 20 ms (so that nothing is measured on a part that is
 * still raising its clocks); each instance's launch time is estimated over
 * `iters` launches; then the instances take turns over five rounds (three or one
 * when a round takes longer than 0.1 / 0.4 s), each timed over a region of about
 * 3 ms per round, and an instance's figure is the minimum of its rounds -- a
 * clock dip has to hit the same instance in every round to change the choice.
 * The instance of the untuned rule stays the choice unless another one is more
 * than 2 % faster.  This call synchronises.  Returns 0 and the winner in
 * *best_config, its time per launch in *best_ms.  On a stream that is being
 * captured into a graph nothing is timed or recorded: returns 0 with
 * *best_config = -1.  A problem that a single instance takes (fp32 or fp8 operands; fp16 / bf16 operands that the
 * direct-to-LDS instances cannot read in place -- a K that is no multiple of 8, rows off 16-byte boundaries, an lhs
 * stored by columns: launch_nt_matmul / launch_nt_addmm run those on dense copies from 2^21 multiply-adds on: the
 * instances are then timed on the copies and the winner recorded for the copies' problem) and no copies has
 * nothing to time: returns 0 with *best_config = -2 and records nothing. */
NineToothedResult nt_tune_gemm(NineToothedStream stream,
                               NineToothedTensor input,
                               NineToothedTensor mat1,
                               NineToothedTensor mat2,
                               NineToothedTensor beta,
                               NineToothedTensor alpha,
                               NineToothedTensor output,
                               int dtype, int output_dtype, int iters,
                               int *best_config, float *best_ms);

/* As nt_tune_gemm for launch_nt_attention: times its loop variants (0 plain 64-key blocks; 1 256 query rows per
 * workgroup; 2 32-key blocks; 3 software-pipelined; 4 software-pipelined with eight waves) on the given tensors the
 * same way and records the fastest for later launches of the same problem (element type, batch, heads, both
 * sequence lengths, head dimension, causal flag) without block-size hints; the variant of the untuned rule stays
 * unless another one is more than 2 % faster.  *best_variant = -1 when nothing was timed (a stream that is being
 * captured into a graph), -2 when the problem has no alternatives (FLOAT32 tensors, head dimensions other than 64
 * and 128, shapes whose key range is split). */
NineToothedResult nt_tune_attention(NineToothedStream stream,
                                    NineToothedTensor q, NineToothedTensor k, NineToothedTensor v,
                                    NineToothedTensor is_causal, NineToothedTensor scale,
                                    NineToothedTensor o,
                                    int dtype, int iters, int *best_variant, float *best_ms);

/* As nt_tune_gemm for launch_nt_conv2d: times the ways to run the convolution -- 4 = a 1 x 1 filter as a batch of
 * plain products, 3 = one launch on the tensors as they lie, 2 = repacking pass plus GEMM loop, 1 = gather kernel; a
 * way that does not take the problem is skipped -- and records the fastest (the block_size_m value that selects
 * it) for later launches of the same problem with block_size_m = 0; a way that needs scratch memory or more
 * launches replaces one before it in that order only when it is more than 3 % faster.  *best_path = -1 when
 * nothing was timed (graph capture). */
NineToothedResult nt_tune_conv2d(NineToothedStream stream,
                                 NineToothedTensor input, NineToothedTensor filter, NineToothedTensor output,
                                 int dtype, int padding_h, int padding_w, int iters,
                                 int *best_path, float *best_ms);

/* Persistence of the tuned choices in the line-pair CSV format of the
 * reference's AutoTuningCache (src/ninetoothed/templates/auto_tuning_cache.h:27-75,
 * writer src/ninetoothed/build.py:683-703): a line of integers for the problem,
 * then a line for the choice; the first pair has an empty problem line and holds
 * a default.  A problem line starts with the program (0 = matmul / addmm: dtype,
 * output dtype, M, N, K, addmm, rhs layout [0 row-major, 1 transposed, 2 other strides; + 4 for operands that
 * the direct-to-LDS instances cannot read in place]; 1 = attention: dtype, batch, heads, seq_q, seq_k, head_dim, causal;
 * 2 = conv2d: dtype, N, C, H, W, K, R, S, padding_h, padding_w, dense input);
 * a choice line starts with the variant (GEMM instance index, attention variant,
 * conv2d path) and may go on with descriptive integers (the GEMM instance's
 * block M, N, K).  Both act on the table of the current device.
 * The default pair's choice line holds nt_tune_file_format(), a number that changes with the numbering of the
 * variants: loading ignores a file that holds another one (0 entries, no error), and it drops every choice that
 * the program does not recognise -- a GEMM instance index without this build's block M, N, K of that instance
 * next to it, an attention variant or conv2d path outside the range.  (The reference's reader takes any line
 * pair, src/ninetoothed/templates/auto_tuning_cache.h:52-75; its files are bound to one build by a fingerprint
 * in build.py:619-662 instead.) */
NineToothedResult nt_tune_cache_save(const char *path);
NineToothedResult nt_tune_cache_load(const char *path, int *entries);
int nt_tune_file_format(void);

/* The cached GEMM instance for a problem with a row-major rhs, or -1. */
int nt_tune_cache_lookup(int dtype, int output_dtype, int m, int n, int k, int addmm);

/* The recorded choice for a problem of program `kind` (as in the cache file: 0, 1, 2) given by the `count`
 * integers of its problem line (without the program), or -1. */
int nt_tune_lookup(int kind, const int *values, int count);

/* Writes which kernel served the calling host thread's latest launch_nt_* call into `buffer` (at most `size`
 * bytes, NUL terminated): the program's kind, the index of the GEMM instance / attention variant / conv2d path /
 * softmax kernel, and a description, e.g. "attention variant 3: software-pipelined loop, 64-key blocks, four waves
 * (128 query rows), two workgroups per CU"; "none" before the first launch.  The counterpart of reading the
 * winning configuration off a Triton autotuner (`best_config`), which the reference's generated kernels allow. */
NineToothedResult nt_last_launch(char *buffer, int size);

/*
 * Element-wise / reducing tile programs that are none of the programs above.
 *
 * Replaces the Triton kernel the reference generates for an arbitrary
 * arrange-and-apply pair (src/ninetoothed/generation.py:28-837) for the class
 * of programs whose application is a map over tiles with an optional reduction
 * (the programs of tests/test_add.py, test_clone.py, test_pad.py, test_pow.py,
 * test_dropout.py, test_max_pool2d.py, test_generation.py:139-151 of the
 * reference).  The host lowers the arrangement's index maps and the
 * application's dataflow graph into two small stack programs; one kernel
 * interprets them per output element:
 *
 *   - the iteration space is `num_vars` index variables with `extents`; the
 *     first `num_vars - num_reduced` enumerate the output elements (the last of
 *     them varies fastest across lanes), the rest the reduced positions;
 *     `num_dynamic` further variables take their value from the data
 *     (`output[row] = input` with `row` loaded from a tensor,
 *     tests/test_generation.py:72-115; `x.source[rows, columns]` and
 *     `ntl.load(x.source.data_ptr() + offsets)`, tests/test_clone.py:23-37);
 *   - index code (one segment per operand, and per `.offsets()` use) computes a
 *     flat element offset from the variables with + * // % by constants
 *     (src/ninetoothed/tensor.py:258-274, 462-471, 555-556) and checks
 *     0 <= index < size where the arrangement needs a mask
 *     (src/ninetoothed/tensor.py:571-584); a masked load yields `other`, a
 *     masked store is skipped (src/ninetoothed/generation.py:638-744);
 *   - value code evaluates the expression in double precision with an explicit
 *     rounding step after every operation whose result the reference holds in
 *     a narrower type, so + - * / and sqrt are the correctly rounded fp16 /
 *     bf16 / fp32 operations; `value_code[0 .. reduce_split)` runs per reduced
 *     position, the rest once per output element on the reduced value.
 *
 * Code words are (opcode | argument << 8); the opcodes are the NT_MAP_I_* /
 * NT_MAP_V_* values below.
 *
 * launch_nt_map specialises: the first launch of a program (same code, index
 * constants, extents and element types) translates it to HIP source, compiles
 * it with hipRTC (loaded on demand) and caches the kernel per device; later
 * launches only pass pointers, `other` values and value constants.  Without
 * hipRTC, or with NT_MAP_INTERPRET=1 in the environment, an interpreter kernel
 * executes the same programs (the struct travels by value as its argument).
 * No device memory is allocated either way.
 */
#define NT_MAP_MAX_OPERANDS 8
#define NT_MAP_MAX_VARS 16
#define NT_MAP_MAX_INDEX_CODE 320
#define NT_MAP_MAX_INDEX_CONSTANTS 96
#define NT_MAP_MAX_SEGMENTS 16
#define NT_MAP_MAX_VALUE_CODE 128
#define NT_MAP_MAX_VALUE_CONSTANTS 32
#define NT_MAP_MAX_PHASES 4

enum NineToothedMapIndexOp {
    NT_MAP_I_END,    /* the offset is on top of the stack */
    NT_MAP_I_CONST,  /* push index_constants[arg] */
    NT_MAP_I_VAR,    /* push variable arg */
    NT_MAP_I_MULC,   /* top *= index_constants[arg] */
    NT_MAP_I_ADD,    /* pop b; top += b */
    NT_MAP_I_DIVC,   /* top = floor(top / index_constants[arg]) */
    NT_MAP_I_MODC,   /* top = top - floor(top / c) * c */
    NT_MAP_I_CHECK   /* pop v; valid &= 0 <= v < index_constants[arg] */
};

enum NineToothedMapValueOp {
    NT_MAP_V_LOAD,      /* push operand arg at its offset (`other` when masked) */
    NT_MAP_V_CONST,     /* push value_constants[arg] */
    NT_MAP_V_OFFSET,    /* push the result of index segment arg */
    NT_MAP_V_ADD, NT_MAP_V_SUB, NT_MAP_V_MUL, NT_MAP_V_DIV, NT_MAP_V_FLOORDIV, NT_MAP_V_MOD, NT_MAP_V_POW,
    NT_MAP_V_MAX, NT_MAP_V_MIN,
    NT_MAP_V_LT, NT_MAP_V_LE, NT_MAP_V_GT, NT_MAP_V_GE, NT_MAP_V_EQ, NT_MAP_V_NE, NT_MAP_V_AND, NT_MAP_V_OR,
    NT_MAP_V_NEG, NT_MAP_V_NOT, NT_MAP_V_ABS, NT_MAP_V_EXP, NT_MAP_V_EXP2, NT_MAP_V_LOG, NT_MAP_V_LOG2,
    NT_MAP_V_SQRT, NT_MAP_V_RSQRT, NT_MAP_V_SIGMOID, NT_MAP_V_TANH, NT_MAP_V_SIN, NT_MAP_V_COS, NT_MAP_V_FLOOR, NT_MAP_V_CEIL,
    NT_MAP_V_WHERE,     /* pop b, a, c; push c ? a : b */
    NT_MAP_V_ROUND,     /* round top to NineToothedDataType arg (integers truncate) */
    NT_MAP_V_RAND,      /* pop offset, seed; push the Philox-4x32-10 uniform float of (seed, offset) */
    NT_MAP_V_SETVAR,    /* pop v; dynamic variable arg = (integer) v: a data-dependent level index */
    NT_MAP_V_REDUCED    /* tile mode: push the result of reduction phase arg (arg < the phase being computed) */
};

enum NineToothedMapReduceOp { NT_MAP_REDUCE_NONE, NT_MAP_REDUCE_MAX, NT_MAP_REDUCE_MIN, NT_MAP_REDUCE_SUM };

/* How the value reaches the output element: a plain store, or an atomic add
 * (`ntl.atomic_add(pointer, value)`, tests/test_data_ptr.py:17-18; 32 / 64 bit
 * integers, float and double only). */
enum NineToothedMapStoreOp { NT_MAP_STORE_ASSIGN, NT_MAP_STORE_ATOMIC_ADD };

typedef struct {
    void *data;
    int32_t dtype;    /* NineToothedDataType */
    int32_t segment;  /* index segment that yields its element offset */
    double other;     /* value of masked loads */
} NineToothedMapOperand;

typedef struct {
    int32_t num_vars;     /* enumerated variables: output elements, then reduced positions */
    int32_t num_reduced;
    int32_t num_dynamic;  /* variables num_vars .. num_vars + num_dynamic - 1 are set by NT_MAP_V_SETVAR */
    int32_t store_op;     /* NineToothedMapStoreOp */
    int64_t extents[NT_MAP_MAX_VARS];
    int32_t num_operands;
    int32_t output;              /* operand that is stored */
    NineToothedMapOperand operands[NT_MAP_MAX_OPERANDS];
    int32_t num_segments;
    int32_t segment_begin[NT_MAP_MAX_SEGMENTS];
    int32_t index_code[NT_MAP_MAX_INDEX_CODE];
    int64_t index_constants[NT_MAP_MAX_INDEX_CONSTANTS];
    int32_t value_code_length;
    int32_t reduce_split;
    int32_t reduce_op;           /* NineToothedMapReduceOp */
    int32_t reduce_dtype;        /* type the reduction accumulates in (sums of fp16 / bf16: FLOAT32) */
    int32_t value_code[NT_MAP_MAX_VALUE_CODE];
    double value_constants[NT_MAP_MAX_VALUE_CONSTANTS];
    /* Tile mode (num_phases > 0; needs reduce_op == NONE, num_reduced == num_dynamic == 0, a plain
     * store): whole-tile reductions whose results the stored expression uses on every element of
     * the tile (normalisations: `x / ntl.sum(x)`, `(x - mean) * ntl.rsqrt(var + eps)`, ...).  The
     * first num_grid variables enumerate the tiles, the others the elements of a tile.  One
     * workgroup takes a tile: for k = 0 .. num_phases - 1 it reduces, over the tile's elements,
     * the term value_code[phase_end[k-1] .. phase_end[k]) (phase_end[-1] = 0) with phase_op[k],
     * accumulating in phase_dtype[k]; then value_code[phase_end[num_phases-1] .. value_code_length)
     * is evaluated and stored per element.  NT_MAP_V_REDUCED reads an earlier phase's result. */
    int32_t num_phases;
    int32_t num_grid;
    int32_t phase_end[NT_MAP_MAX_PHASES];
    int32_t phase_op[NT_MAP_MAX_PHASES];     /* NineToothedMapReduceOp, not NONE */
    int32_t phase_dtype[NT_MAP_MAX_PHASES];
} NineToothedMapProgram;

/* Runs one store of such a program.  Returns NINETOOTHED_NO_KERNEL when the
 * program does not fit the limits above or names an unknown opcode / type. */
NineToothedResult launch_nt_map(NineToothedStream stream, const NineToothedMapProgram *program);

/* Writes the HIP source launch_nt_map specialises `program` to (NUL terminated)
 * into `buffer`; the counterpart of the generated source file the reference's
 * handle exposes as `_source` (src/ninetoothed/jit.py:121-128).  Returns
 * hipErrorInvalidValue when `size` is too small. */
NineToothedResult nt_map_source(const NineToothedMapProgram *program, char *buffer, int size);

/* Library version string, e.g. "nt_hip 0.1 gfx950". */
const char *nt_version(void);

/* Frees every scratch buffer the library holds (see the introduction).  Waits
 * for the device.  A HIP graph captured from a call that used such a buffer
 * refers to it by address: do not release the buffers, or let a larger call on
 * the same stream replace them, while that graph is still replayed.
 * No counterpart in the reference, whose kernels need none. */
void nt_release_workspaces(void);

#ifdef __cplusplus
}
#endif

#endif /* NINETOOTHED_HIP_H */
