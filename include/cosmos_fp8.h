/* libcosmosfp8 - C ABI of the MI355X (gfx950) FP8 hot path.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream
 * (hipStream_t passed as void*; NULL = the null stream).  The library never
 * allocates or frees device memory through these calls, never synchronises the
 * device and never reads a result back to the host; the caller owns every
 * buffer, including workspaces.  Return value: 0 on success, a negative
 * CFP8_E* code otherwise; cfp8_last_error() returns a thread-local message for
 * the last failure on the calling thread.
 *
 * Common contract: bf16 inputs are row-major with the stated leading
 * dimension (in elements), base pointers 16-byte aligned, leading dimensions
 * and column counts multiples of 8 for bf16 / 16 for fp8 unless stated.
 * fp8 = OCP e4m3fn (max 448, NaN 0x7F), never fnuz.
 *
 * Scale formula (all granularities, mode 0):
 *     amax = max|x|;  scale = max(amax, 1e-12) / 448  (fp32, IEEE division)
 *     byte = e4m3fn_rne(clamp(fp32(x) / scale, -448, 448))
 * A NaN in a reduction set gives scale 0x7FC00000 and bytes 0x7F.
 *
 * "Replaces" cites the call in nvidia-cosmos/cosmos-rl that a binding of the
 * entry point stands in for.
 */
#ifndef COSMOS_FP8_H
#define COSMOS_FP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CFP8_OK 0
#define CFP8_EINVAL (-1)    /* null pointer, bad shape, bad alignment          */
#define CFP8_EARCH (-2)     /* device is not gfx950                            */
#define CFP8_ELAUNCH (-3)   /* HIP reported a launch failure                   */
#define CFP8_EWORKSPACE (-4)/* workspace missing or too small                  */

/* output element types of the GEMM epilogues */
#define CFP8_OUT_BF16 0
#define CFP8_OUT_F32 1

/* 1x128 group formulas */
#define CFP8_GROUP_MODE_DIV 0    /* the scale formula above                                 */
#define CFP8_GROUP_MODE_DEEPEP 1 /* x*(448/clamp(amax,1e-4)), scale=amax/448, no pre-clamp  */

int cfp8_version(void);
const char* cfp8_last_error(void);

/* Rowwise dynamic quantisation: per row amax -> scale -> e4m3.
 * x bf16 [rows, cols] (ld_x), q fp8 [rows, cols] (ld_q), scales fp32 [rows].
 * Replaces vllm._custom_ops.scaled_fp8_quant(w, scale=None,
 * use_per_token_if_dynamic=True) at
 * cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:995-997 and
 * cosmos_rl/rollout/vllm_rollout/monkey_patch_for_fp8.py:47-49 (weights), and the
 * per-token activation quantisation inside Fp8LinearOp.apply installed at
 * monkey_patch_for_fp8.py:74-79.  cols % 8 == 0. */
int cfp8_quant_rowwise(const void* x, int64_t rows, int64_t cols, int64_t ld_x,
                       void* q, int64_t ld_q, float* scales, void* stream);

/* Source element types of cfp8_quant_rowwise_from. */
#define CFP8_IN_BF16 0
#define CFP8_IN_F16 1
#define CFP8_IN_F32 2

/* Rowwise quantisation straight from a received weight in its transfer dtype:
 * q, scales = quant_rowwise(x.to(bfloat16)) with x bf16, fp16 or fp32, written
 * wherever the caller points q (e.g. the engine's own fp8 parameter, ld_q its row
 * pitch) and scales.  One kernel in place of the three passes
 *   recv.to(view.dtype); view.copy_(...)        cosmos_rl/policy/model/base.py:1053-1069
 *   ops.scaled_fp8_quant(weight, ...)           cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:995-997
 *   param.copy_(quantized); scale.copy_(scale)  cosmos_rl/rollout/worker/rollout_control.py:889-898
 * for receives that cover whole rows of a weight.  ld_x in elements of x_dtype. */
int cfp8_quant_rowwise_from(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld_x,
                            void* q, int64_t ld_q, float* scales, void* stream);

/* Rowwise quantisation of many weights in as few launches as their shapes allow: what
 * cfp8_quant_rowwise_from does for each descriptor, with the tensors of equal row-length class
 * and source dtype sharing a launch (the table travels in the kernel arguments).  For the batch of
 * completions that a weight sync runs together once their shards have landed,
 * cosmos_rl/rollout/worker/rollout_control.py:1308-1319 (each completion quantises one full weight,
 * :856-898); one launch per weight leaves every weight under ~50 MB bound by the ramp-up of its
 * launch.  The descriptor array lives in HOST memory and is read before the call returns.
 * Results are bit-identical to per-tensor calls.  Per descriptor: the contract of
 * cfp8_quant_rowwise_from. */
typedef struct cfp8_rowwise_desc {
    const void* x;     /* [rows, cols] of x_dtype, row pitch ld_x elements, 16-byte aligned */
    void* q;           /* fp8 out, row pitch ld_q bytes, 8-byte aligned                     */
    float* scales;     /* device, rows floats out                                            */
    int64_t rows, cols, ld_x, ld_q;
    int32_t x_dtype;   /* CFP8_IN_*                                                          */
    int32_t reserved;  /* 0                                                                  */
} cfp8_rowwise_desc;
int cfp8_quant_rowwise_multi(const cfp8_rowwise_desc* descs, int64_t n, void* stream);

/* Tensorwise dynamic quantisation of many tensors in two passes (grid amax,
 * then cast), without a host round trip in between.
 * Replaces the torchao tensorwise recipe selected at
 * cosmos_rl/utils/fp8/fp8_util.py:121-137 (hp_tensor_to_float8_dynamic).
 * The descriptor array lives in HOST memory; amax_ws is a device array of
 * n * CFP8_TENSORWISE_AMAX_SLOTS floats (scratch, overwritten).
 * numel % 8 == 0 for every tensor.
 * With the read-once form switched on (cfp8_tensorwise_resident, off by default), tensors that fill three quarters
 * or more of the GPU's registers and LDS and still fit (106-141 MB of bf16 on a 256-CU MI355X, numel % 512 == 0:
 * the MLP weights of a 7-8 B model) are read once: one launch of one workgroup per CU keeps them on the chip
 * between the two passes.  Smaller tensors that fill three quarters of a half, a third ... an eighth of the chip
 * (down to 13 MB) are held several at a time, each by its share of the CUs, in the same kernel; in between the workgroups meet through a small array in device memory that the library
 * owns (one per GPU, so two read-once launches must not run on one GPU at the same time - which their need for
 * every CU rules out anyway).
 * The order in which the tensors of a call are quantised is unspecified; the results do not depend on it. */
#define CFP8_TENSORWISE_AMAX_SLOTS 64
typedef struct cfp8_tensor_desc {
    const void* x;   /* bf16, contiguous, 16-byte aligned */
    void* q;         /* fp8 out, numel bytes              */
    float* scale;    /* device, 1 float out               */
    int64_t numel;
} cfp8_tensor_desc;

int cfp8_quant_tensorwise_multi(const cfp8_tensor_desc* descs, int64_t n,
                                float* amax_ws, void* stream);

/* Switch for the read-once form of cfp8_quant_tensorwise_multi (and _multi_static): enable != 0 allows it, 0 (the
 * default) makes every tensor take the two separate passes, a negative value only queries.  Returns the previous
 * setting.  The read-once launch needs all its workgroups on the GPU at the same time, one per CU, so it is for a
 * process that has the GPU to itself while it quantises (the trainer's cast of its weights; not a rollout worker
 * that quantises on a copy stream beside generation, cosmos_rl/rollout/worker/rollout_control.py:1312-1317).
 * Where the workgroups cannot all be resident (another stream's or process's kernel holds CUs, two such launches
 * at once, a CU mask) the meeting of a tensor cannot complete: every workgroup waits at most the bound below,
 * marks that tensor and the ones behind it in the launch and leaves, and two small kernels that follow every such
 * launch on the same stream quantise exactly the marked tensors as two ordinary passes.  The call's
 * results are therefore the same bits either way; what a failed meeting costs is the wait.  It is recorded: the
 * last of a tensor's CFP8_TENSORWISE_AMAX_SLOTS slots in amax_ws is its status word, nonzero when the read-once
 * launch gave the tensor up, until the workspace is next used.  No counterpart in the reference. */
int cfp8_tensorwise_resident(int enable);

/* *given_up (device int32) = how many of the n tensors of the last call on amax_ws carry a set status word.
 * amax_ws NULL: the library's own slots, those of cfp8_quant_tensorwise_multi_static.
 * One small launch on `stream`; nothing is read back by the library.  A caller that finds a nonzero count
 * after synchronising knows that the read-once form does not have the GPU to itself and switches it off. */
int cfp8_tensorwise_status(const float* amax_ws, int64_t n, int32_t* given_up, void* stream);

/* Tuning and test hook of the read-once form (process-wide; negative or zero arguments leave a value as it is):
 * wait_us > 0 sets the bound of a workgroup's wait at a tensor's meeting (default 20000 us); extra_arrivals >= 0
 * makes every meeting expect that many arrivals more than the grid has workgroups - with 1, no meeting can
 * complete and every tensor of a read-once launch is given up and repaired, which is how the test suite drives
 * that path with every wave leaving its kernel normally.  0 restores the real count. */
int cfp8_tensorwise_resident_tuning(int64_t wait_us, int extra_arrivals);

/* Split-phase forms of the above.  Pass 1 alone leaves partial maxima of |x| of
 * tensor i in amax_ws[i*SLOTS .. i*SLOTS+SLOTS-2] (non-negative fp32 bit
 * patterns, a NaN pattern if the tensor holds one; their maximum as unsigned
 * integers is the tensor's amax) and zero in the last slot, the status word; pass 2
 * alone folds those slots, writes scale and bytes.  Between the two a caller may
 * combine amax_ws across devices with an elementwise all-reduce max over the uint32
 * view - the tensor-parallel Float8 case of
 * cosmos_rl/policy/model/gpt/parallelize.py:268-280.  The slots pass 2 finds need not
 * hold the maximum of the very tensor it casts (another rank's data went into them):
 * a quotient beyond +-448 saturates to +-448, as the reference's clamp in front of
 * its cast does.  q and scale may be null in pass 1. */
int cfp8_tensorwise_amax_multi(const cfp8_tensor_desc* descs, int64_t n,
                               float* amax_ws, void* stream);
int cfp8_tensorwise_cast_multi(const cfp8_tensor_desc* descs, int64_t n,
                               float* amax_ws, void* stream);

/* cfp8_quant_tensorwise_multi without a workspace argument and without any allocation: the amax
 * slots are a fixed array inside the library's device image (CFP8_TENSORWISE_STATIC_MAX_TENSORS *
 * CFP8_TENSORWISE_AMAX_SLOTS * 4 bytes = 128 KiB, held on every GPU the library is used on until
 * the process ends).  No counterpart in the reference: it is for callers that cannot allocate
 * device memory - code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  The call makes no hipMalloc / hipFree and calls no allocating routine; inputs and
 * outputs are still the caller's.  n > CFP8_TENSORWISE_STATIC_MAX_TENSORS returns
 * CFP8_EWORKSPACE.  All calls on one GPU share the one array (each call clears the slots it
 * uses first), so two calls that overlap on one GPU - different streams, or different threads -
 * race; calls on one stream are ordered and safe.  Results are bit-identical to
 * cfp8_quant_tensorwise_multi. */
#define CFP8_TENSORWISE_STATIC_MAX_TENSORS 512
int cfp8_quant_tensorwise_multi_static(const cfp8_tensor_desc* descs, int64_t n, void* stream);

/* Single-tensor form of cfp8_quant_tensorwise_multi. */
int cfp8_quant_tensorwise(const void* x, int64_t numel, void* q, float* scale,
                          float* amax_ws, void* stream);

/* 128x128 block quantisation of a batch of matrices.
 * x bf16 [batch, rows, cols] contiguous; scales fp32
 * [batch, ceil(rows/128), ceil(cols/128)] row-major (the layout
 * cosmos_rl/policy/model/deepseek_v3/weight_mapper.py:236-243 reads).
 * transpose_out == 0: q is [batch, rows, cols]; != 0: q is [batch, cols, rows]
 * (the K-major "nt" operand of the block GEMM when the weight arrives [K, N]).
 * Replaces dsgemm_utils.prepare_fp8_weight at
 * cosmos_rl/policy/kernel/group_gemms.py:132.  cols % 8 == 0 (and rows % 16 == 0
 * when transposing). */
int cfp8_quant_block128(const void* x, int64_t batch, int64_t rows, int64_t cols,
                        void* q, float* scales, int transpose_out, void* stream);

/* 1x128 group quantisation of activations.  x bf16 [rows, cols] (ld_x),
 * q fp8 [rows, cols] (ld_q), scales fp32 [rows, ceil(cols/128)] row-major.
 * Replaces dsgemm_kernels.groupwise_activation_quant / dsgemm_utils.prepare_fp8_input
 * at cosmos_rl/policy/kernel/group_gemms.py:188-191, 213-218; mode
 * CFP8_GROUP_MODE_DEEPEP is per_token_cast_to_fp8 of tests/test_deepep.py:75-85. */
int cfp8_quant_group128(const void* x, int64_t rows, int64_t cols, int64_t ld_x,
                        void* q, int64_t ld_q, float* scales, int mode, void* stream);

/* SwiGLU between the expert GEMMs fused with the 1x128 quantisation of its result:
 *   h = bf16(bf16(silu(gate)) * up),  q, scales = quant_group128(h, CFP8_GROUP_MODE_DIV)
 * gate, up bf16 [rows, cols] (two GEMM outputs, or the two halves of one fused
 * gate_up output: up = gate + cols, ld_gate = ld_up = 2 * cols); h is never
 * written.  Replaces `self.activation_function(gate_proj_out) * up_proj_out`
 * followed by `groupwise_activation_quant` / `prepare_fp8_input` at
 * cosmos_rl/policy/kernel/group_gemms.py:209-218 for the SiLU activation.
 * silu(x) = x / (1 + exp(-x)) in fp32; exp is a fixed sequence of correctly
 * rounded fp32 operations (two-part ln2 reduction, degree-7 Horner polynomial with
 * fused multiply-adds, ldexp), so the result is the same bits on any IEEE machine. */
int cfp8_swiglu_quant_group128(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                               int64_t rows, int64_t cols, void* q, int64_t ld_q, float* scales,
                               void* stream);

/* Grouped gate_up GEMM with the SwiGLU + 1x128 requantisation as its epilogue: what
 * cfp8_gemm_grouped_block128 (on the concatenated gate and up weights) followed by
 * cfp8_swiglu_quant_group128 compute, bit for bit, without writing the bf16 [M, 2 I] product to memory
 * and reading it back.  Replaces cosmos_rl/policy/kernel/group_gemms.py:194-218 as one launch.
 * b fp8 [E, 2 I, K] holds gate and up rows interleaved in units of 16 (one MFMA tile): for every block j of 128
 * intermediate features and p = 0 .. 7, rows [256 j + 32 p, + 16) = gate rows [128 j + 16 p, + 16) and rows
 * [256 j + 32 p + 16, + 16) = the up rows of the same features - a lane of the GEMM then holds a gate value and the up
 * value it is multiplied with, and the SwiGLU needs no exchange.  sb fp32 [E, 2 I / 128, K / 128]: scale row 2 j = the
 * block scales of gate block j, row 2 j + 1 those of up block j (ops.interleave_gate_up builds both).  One 128 x 256
 * tile holds both halves of a 1x128 group of h = silu(gate) * up.  q fp8 [M, I] (pitch ld_q bytes), scales fp32
 * [M, I / 128]; rows with m_indices < 0 are left untouched.  M % 128 == 0, I % 128 == 0, K % 128 == 0. */
int cfp8_gemm_grouped_swiglu_quant(const void* a, int64_t ld_a, const float* sa, const void* b, const float* sb,
                                   const int32_t* m_indices, void* q, int64_t ld_q, float* scales,
                                   int64_t M, int64_t I, int64_t K, int64_t E, void* stream);

/* Permutation indices that regroup tokens from (source rank, local expert) order into expert
 * order with every group padded to a multiple of `alignment` rows (an expert without tokens
 * still gets `alignment` rows).  tokens_per_expert_group int64 [num_ranks * experts_per_rank],
 * rank-major.  Outputs: m_sizes, m_offsets int32 [experts_per_rank] (padded group sizes and
 * their inclusive cumulative sum), start_index_values int64 [num_ranks * experts_per_rank]
 * (exclusive prefix sum of the counts), permuted_indices int32 [capacity]: source row of every
 * output row, -1 for padding rows and for rows past sum(m_sizes).  Passing a capacity bound
 * (e.g. tokens + experts * alignment) keeps the call free of a host read-back.
 * Replaces generate_permute_indices / fill_indices_wrapper at
 * cosmos_rl/policy/kernel/moe/indices.py:24-118, 147-220. */
int cfp8_generate_permute_indices(const int64_t* tokens_per_expert_group, int experts_per_rank,
                                  int num_ranks, int64_t alignment, int32_t* permuted_indices,
                                  int64_t capacity, int32_t* m_sizes, int32_t* m_offsets,
                                  int64_t* start_index_values, void* stream);

/* out[i, :] = x[indices[i], :] for indices[i] >= 0, zeros for -1: the row gather that applies
 * permuted_indices to the token matrix (the reference indexes with torch:
 * cosmos_rl/policy/kernel/moe/moe.py token regrouping before group_gemms.py:152-156).
 * Rows are row_bytes wide (multiple of 16); pitches in bytes. */
int cfp8_gather_rows(const void* x, int64_t ld_x_bytes, const int32_t* indices, int64_t rows_out,
                     int64_t row_bytes, void* out, int64_t ld_out_bytes, void* stream);

/* Weighted combine of expert outputs back into token order (bf16 in, bf16 out):
 *   out[t, :] = sum over slots s = 0 .. topk-1, in that order, of weights[t, s] * rows[row_map[t, s], :]
 * row_map int32 [tokens, topk]; a slot with row_map < 0 or >= num_rows contributes nothing.
 * topk <= 64, hidden % 8 == 0, pitches in elements.
 *   CFP8_COMBINE_BF16_STEPS (weights bf16): every product and every partial sum is rounded to
 *     bf16, starting from +0 -- bit for bit what GroupedExperts.forward accumulates with
 *     `expert_out * weights[idx, top, None]` and `y.scatter_add_` on bf16 tensors when the slots
 *     of a token are ordered by ascending expert id (the order of its loop over experts):
 *     cosmos_rl/policy/kernel/moe/moe.py:240-262.
 *   CFP8_COMBINE_F32 (weights bf16 or fp32): fp32 accumulator acc = fma(row, weight, acc), one
 *     rounding at the end -- the arithmetic of the vendored Triton kernel
 *     cosmos_rl/policy/kernel/megatron_moe/permutation.py:336-428 (whether its multiply and add
 *     contract into an fma is the Triton compiler's choice; fma is assumed here). */
#define CFP8_COMBINE_BF16_STEPS 0
#define CFP8_COMBINE_F32 1
int cfp8_combine_rows(const void* rows, int64_t ld_rows, int64_t num_rows, const int32_t* row_map,
                      const void* weights, int weights_dtype, int64_t tokens, int topk, int64_t hidden,
                      int mode, void* out, int64_t ld_out, void* stream);

/* MXFP4 quantisation of bf16 rows: every block of 32 consecutive elements of a row gets one
 * e8m0 scale byte 2^ceil(log2(amax / 6)) and 32 e2m1 codes (round to nearest, ties away from zero),
 * two per byte, even element in the low nibble.  q uint8 [rows, cols / 2] (pitch ld_q bytes,
 * multiple of 4), scales uint8 [rows, cols / 32] (pitch ld_scales bytes), cols % 32 == 0, ld_x in
 * elements (multiple of 8).  NaN / infinity inputs give unspecified codes.
 * Replaces quantize_mx4 = triton_kernels' downcast_to_mxfp(w, torch.uint8, axis=1) at
 * cosmos_rl/rollout/vllm_rollout/monkey_patch_for_mxfp4.py:18-24 together with the two transposes
 * around it at cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:1018-1029 (blocks along the last
 * axis of the [experts * out, in] weight); the engine-specific swizzle that follows there
 * (:1037-1045) is not part of this call. */
int cfp8_quant_mxfp4(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q,
                     void* scales, int64_t ld_scales, void* stream);

/* The consumer of cfp8_quant_mxfp4's output: out[m, n] = sa[m] * sum_k a[m, k] * value(w[g, n, k]), where
 * value = e2m1 code * 2^(ws[g, n, k / 32] - 127).  a e4m3 [M, K] (pitch ld_a bytes) with one fp32 scale per
 * row (cfp8_quant_rowwise of the activations), w packed e2m1 [num_groups, N, K / 2] (row pitch ld_w bytes),
 * ws e8m0 [num_groups, N, K / 32] (row pitch ld_ws bytes); groups lie N rows apart.  The matrix instruction
 * takes the weight codes and their block scales as they are (v_mfma_scale_f32_16x16x128_f8f6f4, A in e2m1
 * with hardware-applied e8m0 scales, B in e4m3); accumulation in fp32.  m_indices null: one weight matrix
 * (num_groups 0 or 1).  m_indices int32 [M] (device): row m uses group m_indices[m], groups start on
 * multiples of 128 rows, M % 128 == 0, rows with a negative index are padding and their outputs are left
 * untouched (the layout of cfp8_gemm_grouped_block128).  K % 32 == 0 (not necessarily % 128: GPT-OSS has
 * K = 2880), N % 16 == 0, ld_a and ld_w multiples of 16, a and w 16-byte aligned, ld_out in elements
 * (multiple of 4).  out_dtype CFP8_OUT_BF16 or CFP8_OUT_F32.
 * In the reference the quantised expert weights of mxfp4_quantization
 * (cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:1000-1045) are handed to the rollout engine's FusedMoE
 * layers (monkey_patch_for_mxfp4.py:27-47, w13_weight / w2_weight), whose matrix product lives in the
 * third-party triton_kernels package; this entry is that product for the unswizzled [E, N, K / 2] layout
 * of vllm_rollout.py:1025-1033, on activations quantised per token as in the FP8 linear. */
int cfp8_gemm_mxfp4(const void* a, int64_t ld_a, const float* sa, const void* w, int64_t ld_w, const void* ws,
                    int64_t ld_ws, const int32_t* m_indices, int64_t num_groups, void* out, int64_t ld_out,
                    int out_dtype, int64_t M, int64_t N, int64_t K, void* stream);

/* The linear layer on MXFP4 weights from bf16 activations: per-token dynamic FP8 quantisation of x (bf16 [M, K], ld_x in
 * elements, multiple of 8, x 16-byte aligned; the arithmetic of cfp8_quant_rowwise) followed by cfp8_gemm_mxfp4 on one
 * weight matrix.  Up to 4 tokens with K <= 4096 run as one launch (the quantisation inside the weight-streaming
 * kernel, bit-identical to the two steps) and need no workspace; otherwise the quantised activations and their scales
 * go to `workspace` (device memory, 256-byte aligned, at least cfp8_linear_workspace_bytes(M, K) bytes).  The other
 * arguments are those of cfp8_gemm_mxfp4.  The counterpart of cfp8_linear_rowwise for the weights of
 * cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:1000-1045. */
int cfp8_linear_mxfp4(const void* x, int64_t ld_x, const void* w, int64_t ld_w, const void* ws, int64_t ld_ws,
                      void* out, int64_t ld_out, int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                      size_t workspace_bytes, void* stream);

/* cfp8_gather_rows followed by cfp8_quant_group128 (CFP8_GROUP_MODE_DIV) as one pass: row r of the
 * output quantises row src_rows[r] of x (bf16 [*, cols], ld_x in elements), a zero row where src_rows[r] < 0.
 * The gathered bf16 matrix [rows_out, cols] that the reference builds with torch indexing before
 * group_gemms.py:188-191 is never written.  q fp8 [rows_out, cols] (ld_q), scales fp32 [rows_out, ceil(cols/128)]. */
int cfp8_gather_quant_group128(const void* x, int64_t ld_x, const int32_t* src_rows, int64_t rows_out, int64_t cols,
                               void* q, int64_t ld_q, float* scales, void* stream);

/* The same result as cfp8_gather_quant_group128, computed from the token side: every row of x (bf16 [tokens, cols])
 * is quantised once and its bytes and scales are stored to the rows row_map[t, 0 .. topk) of the output (int32, device;
 * negative or >= rows_out = no row), and the rows r with src_rows[r] < 0 are written as zero rows.  For top-k routing
 * this reads and quantises a token once instead of once per expert it goes to.  row_map and src_rows must describe
 * the same layout (src_rows[r] == t exactly for the rows r listed in row_map[t, :]); rows that neither names are
 * left untouched.  topk <= 64.  Same reference lines as cfp8_gather_quant_group128 (the torch indexing in front of
 * cosmos_rl/policy/kernel/group_gemms.py:188-191, with the layout cosmos_rl/policy/kernel/moe/moe.py:244-263 implies). */
int cfp8_scatter_quant_group128(const void* x, int64_t ld_x, int64_t tokens, int64_t cols, const int32_t* row_map,
                                int64_t topk, const int32_t* src_rows, int64_t rows_out, void* q, int64_t ld_q,
                                float* scales, void* stream);

/* Block dequantisation y = fp8 * s[i/128, j/128]; out_dtype CFP8_OUT_BF16 or
 * CFP8_OUT_F32.  Replaces weight_dequant at
 * cosmos_rl/policy/model/deepseek_v3/weight_mapper.py:246-259. */
int cfp8_dequant_block128(const void* q, const float* scales, int64_t rows, int64_t cols,
                          void* y, int out_dtype, void* stream);

/* 1x128 group dequantisation, the inverse of cfp8_quant_group128: y[i, j] = fp8[i, j] * scale[i, j / 128].
 * q fp8 [rows, cols] (pitch ld_q bytes); y bf16 or fp32 [rows, cols] (pitch ld_y elements, rows 16-byte aligned);
 * cols % 8 == 0, not necessarily a multiple of 128 (the last group is then short).
 * scale_kind CFP8_SCALE_F32: scales fp32 [rows, ceil(cols/128)], pitch ld_scales floats.
 * scale_kind CFP8_SCALE_E8M0: one exponent byte per group, [rows, ceil(cols/128)] with pitch ld_scales bytes, value
 *   2^(byte - 127) formed as the bit pattern byte << 23 - what viewing the reference's packed int32 scales as uint8
 *   and shifting gives (four groups per int32, lowest byte first).
 * Replaces per_token_cast_back of tests/test_deepep.py:86-108 (float scales, and its `x_scales.dtype == torch.int`
 * branch :97-99); the product is formed in fp32 and rounded once, to nearest even, for bf16. */
#define CFP8_SCALE_F32 0
#define CFP8_SCALE_E8M0 1
int cfp8_dequant_group128(const void* q, int64_t ld_q, const void* scales, int64_t ld_scales, int scale_kind,
                          int64_t rows, int64_t cols, void* y, int64_t ld_y, int out_dtype, void* stream);

/* Rowwise scaled mm on quantised operands:
 *   out[m, n] = (sum_k a[m,k] b[n,k]) * sa[m] * sb[n]
 * a fp8 [M, K] (ld_a), b fp8 [N, K] (ld_b) - the contiguous buffer whose .t()
 * the reference passes -, sa [M], sb [N], out [M, N] (ld_out).
 * Replaces torch._scaled_mm(qx, w.t(), scale_a, scale_b, out_dtype=bf16) reached
 * through cosmos_rl/rollout/vllm_rollout/monkey_patch_for_fp8.py:26-34.
 * K % 16 == 0, N % 16 == 0 (the dimensions module_filter_fn of cosmos_rl/utils/fp8/fp8_util.py:62-87 lets
 * through).  The tuned kernels take K % 128 == 0; any other K runs the generic tile kernel with its last K step
 * masked. */
int cfp8_scaled_mm_rowwise(const void* a, int64_t ld_a, const float* sa,
                           const void* b, int64_t ld_b, const float* sb,
                           void* out, int64_t ld_out, int out_dtype,
                           int64_t M, int64_t N, int64_t K, void* stream);

/* FP8 linear: per-token dynamic quantisation of x (bf16 [M, K]) into the
 * workspace followed by the rowwise scaled mm, as one call.
 * Replaces Fp8LinearOp.apply (monkey_patch_for_fp8.py:74-79).
 * workspace: at least cfp8_linear_workspace_bytes(M, K) bytes, 256-byte aligned.
 * cfp8_linear_workspace_bytes_split(M, N, K) >= that is the size with which the call may also
 * cut K into slices for weights with few rows and a long K at 17..64 tokens (a decode-time
 * down projection: 3584 x 18944 runs 2-3x faster); the extra bytes hold fp32 partial sums.
 * Any size in between is valid and simply selects the unsplit kernel.  K % 16 == 0, N % 16 == 0. */
size_t cfp8_linear_workspace_bytes(int64_t M, int64_t K);
size_t cfp8_linear_workspace_bytes_split(int64_t M, int64_t N, int64_t K);
int cfp8_linear_rowwise(const void* x, int64_t ld_x, const void* w, int64_t ld_w,
                        const float* w_scale, void* out, int64_t ld_out, int out_dtype,
                        int64_t M, int64_t N, int64_t K,
                        void* workspace, size_t workspace_bytes, void* stream);

/* Block-scaled "nt" GEMM on quantised operands:
 *   out[m, n] = sum_kb (a[m, kb] . b[n, kb]) * sa[m, kb] * sb[n/128, kb]
 * a fp8 [M, K], sa fp32 [M, K/128]; b fp8 [N, K]; sb addressed as
 * sb[(n/128) * sb_stride_n + kb * sb_stride_k] so both [N/128, K/128] and
 * [K/128, N/128] layouts work.  K % 128 == 0, N % 16 == 0.
 * The dense (one expert) case of deep_gemm's fp8 GEMM used at
 * cosmos_rl/policy/kernel/group_gemms.py:194-225. */
int cfp8_gemm_block128(const void* a, int64_t ld_a, const float* sa,
                       const void* b, int64_t ld_b, const float* sb,
                       int64_t sb_stride_n, int64_t sb_stride_k,
                       void* out, int64_t ld_out, int out_dtype,
                       int64_t M, int64_t N, int64_t K, void* stream);

/* Grouped contiguous block-scaled GEMM.  Row r of a belongs to expert
 * m_indices[r] (int32, device); groups are contiguous and start on multiples of
 * 128 rows; rows with a negative index are padding and are not written.
 * b fp8 [E, N, K] contiguous, sb fp32 [E, ceil(N/128), K/128].
 * Replaces deep_gemm.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous at
 * cosmos_rl/policy/kernel/group_gemms.py:194-225. */
int cfp8_gemm_grouped_block128(const void* a, int64_t ld_a, const float* sa,
                               const void* b, const float* sb, const int32_t* m_indices,
                               void* out, int64_t ld_out, int out_dtype,
                               int64_t M, int64_t N, int64_t K, int64_t E, void* stream);

/* Which kernels a GEMM call would launch, without launching anything and without a device: the
 * dispatch code of the entry point named by `kind` runs with launches switched off and writes, for
 * each kernel in order, "<kernel> grid=<workgroups> block=<threads> lds=<bytes>" separated by "; "
 * into buf.  `cus` stands in for the device's compute-unit count (256 on MI355X), which several
 * choices depend on; with_split_workspace says whether CFP8_DISPATCH_LINEAR is given the larger
 * workspace of cfp8_linear_workspace_bytes_split.  No counterpart in the reference: it exists so
 * that a test can pin, on any machine, that a shape still takes the kernel form its parity tests
 * cover.  CFP8_DISPATCH_GROUPED_SWIGLU takes N = 2 I. */
#define CFP8_DISPATCH_ROWWISE 0        /* cfp8_scaled_mm_rowwise          */
#define CFP8_DISPATCH_LINEAR 1         /* cfp8_linear_rowwise             */
#define CFP8_DISPATCH_BLOCK 2          /* cfp8_gemm_block128              */
#define CFP8_DISPATCH_GROUPED 3        /* cfp8_gemm_grouped_block128      */
#define CFP8_DISPATCH_GROUPED_SWIGLU 4 /* cfp8_gemm_grouped_swiglu_quant  */
int cfp8_gemm_dispatch_info(int kind, int64_t M, int64_t N, int64_t K, int out_dtype, int cus,
                            int with_split_workspace, char* buf, size_t buf_bytes);

#ifdef __cplusplus
}
#endif
#endif /* COSMOS_FP8_H */
