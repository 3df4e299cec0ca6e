/*
 * libwoq — MI355X (gfx950) weight-only quantized matmul, C ABI.
 *
 * This is the drop-in boundary for the computation behind TensorRT-LLM's
 * WeightOnlyQuantMatmulPlugin and WeightOnlyGroupwiseQuantMatmulPlugin.  TensorRT does not
 * exist on ROCm, so the boundary sits one level under the plugins' `enqueue`: at the pair
 *   weight_only::kernel_launcher(arch, Params&, stream)          (small-M kernel) and
 *   CutlassFpAIntBGemmRunner::gemm(A, B, scales, zeros, bias, alpha, C, m, n, k, group, ...)
 * and at the torch custom ops that prepare weights.  Every entry point below names the
 * reference interface it replaces (paths relative to the reference checkout).
 *
 * Conventions
 *   - plain C types only; all device pointers are HIP device pointers; `stream` is a hipStream_t
 *     passed as void* (NULL = the default stream);
 *   - every function returns 0 on success or a negative woq_status; the message of the last
 *     failure on the calling thread is available from woq_last_error();
 *   - nothing is thrown across the boundary, nothing is allocated on the device by woq_matmul
 *     (the caller supplies the workspace), the library keeps no per-call state, and calls on
 *     different streams may run concurrently.
 */
#ifndef WOQ_H_
#define WOQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WOQ_ABI_VERSION 1
/* tag of the preprocessed-weight byte layout (gfx950 tile layout, see woq_preprocess_weights) */
#define WOQ_LAYOUT_VERSION 1

typedef enum woq_status
{
    WOQ_OK = 0,
    WOQ_ERR_INVALID_ARGUMENT = -1, /* null pointer, bad enum, inconsistent optional inputs */
    WOQ_ERR_BAD_SHAPE = -2,        /* m/n/k/group_size violate an alignment rule */
    WOQ_ERR_UNSUPPORTED = -3,      /* a combination the reference also rejects (e.g. W4A8 with g64) */
    WOQ_ERR_WORKSPACE = -4,        /* workspace missing or smaller than woq_workspace_bytes() */
    WOQ_ERR_RUNTIME = -5,          /* a HIP call failed (no device, launch failure) */
    WOQ_ERR_VALUE = -6             /* data out of range (e.g. an int4 value outside [-8, 7]) */
} woq_status;

/* element types of activations / scales / outputs
 * (the plugins' `type_id`: nvinfer1::DataType kHALF / kBF16; fp8 only as a W4A8 activation) */
typedef enum woq_dtype
{
    WOQ_FP16 = 0,
    WOQ_BF16 = 1,
    WOQ_FP8_E4M3 = 2, /* OCP e4m3fn */
    WOQ_FP32 = 3      /* only as a host-side weight/scale type of woq_symmetric_quantize */
} woq_dtype;

/* cutlass_kernels::QuantType — cpp/tensorrt_llm/kernels/cutlass_kernels/cutlass_preprocessors.h:32-48 */
typedef enum woq_quant_type
{
    WOQ_W8_A16 = 0,
    WOQ_W4_A16 = 1,
    WOQ_W4_AFP8 = 2
} woq_quant_type;

/* quant_algo bit flags of the groupwise plugin —
 * cpp/tensorrt_llm/plugins/weightOnlyGroupwiseQuantMatmulPlugin/weightOnlyGroupwiseQuantMatmulPlugin.cpp:29-37 */
#define WOQ_ALGO_BIAS 1
#define WOQ_ALGO_ZERO 2
#define WOQ_ALGO_PRE_QUANT_SCALE 4
#define WOQ_ALGO_FP8_ALPHA 8 /* W4A8: fp8 MFMA path, `alpha` applied in the epilogue */
#define WOQ_ALGO_INT8_WEIGHT 16

/* which kernel family runs; AUTO follows the M-regime rule of woq_select_regime() */
typedef enum woq_regime
{
    WOQ_REGIME_AUTO = 0,
    WOQ_REGIME_STREAM = 1, /* weight-streaming kernels (decode GEMV; accept m <= 128, W4A8 m <= 32); with 4 to
                              16 rows on long-K / narrow-N shapes they split K through the workspace when
                              it is large enough, and run unsplit when it is not */
    WOQ_REGIME_GEMM = 2    /* tiled MFMA GEMMs: deferred-scale 32/64-row tiles or exact-dequantize 64/128/256-row
                              tiles (whichever is estimated cheaper for the shape), the fp8 kernel for W4A8;
                              may split K through the workspace */
} woq_regime;

/*
 * One matmul call.  Replaces weight_only::Params
 * (cpp/tensorrt_llm/kernels/weightOnlyBatchedGemv/common.h:63-101) and the argument lists of
 * CutlassFpAIntBGemmRunnerInterface::gemm
 * (cpp/tensorrt_llm/kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm.h:55-96); field meaning
 * follows the plugins' enqueue (weightOnlyQuantMatmulPlugin.cpp:283-339,
 * weightOnlyGroupwiseQuantMatmulPlugin.cpp:407-495):
 *
 *   out[m, n] = T( alpha * sum_k  S(act[m, k]) * W[k, n]  + bias[n] )
 *   W[k, n]   = q[k, n] * scales[g(k), n] + zeros[g(k), n]      (zeros are additive, pre-scaled)
 *   S(a)      = a * pre_quant_scale[k] when given, else a
 *
 *   act              [m, k]            act_dtype (fp16 / bf16; fp8 e4m3 only with FP8_ALPHA)
 *   pre_quant_scale  [k]               out_dtype, required iff quant_algo & PRE_QUANT_SCALE
 *   weight           woq_preprocessed_bytes(k, n, quant_type) bytes from woq_preprocess_weights
 *   scales           [ceil(k/group_size), n] or [n] when group_size == 0 (one scale per column);
 *                    out_dtype, except W4A8 where they hold fp16 whatever out_dtype is
 *   zeros            same shape/type as scales, required iff quant_algo & ZERO
 *   bias             [n]               out_dtype, required iff quant_algo & BIAS
 *   out              [m, n]            out_dtype
 *   n                LOGICAL number of output columns (the reference plugins receive the packed
 *                    column count and multiply it back: `real_n`)
 *   group_size       0 (per-channel, the WeightOnlyQuantMatmul plugin), 64, 128, or any larger multiple
 *                    of 64 (W4A8: 128 and any larger multiple of 128) - what the reference's Hopper
 *                    kernels accept, a multiple of their K tile
 *                    (launchers/fpA_intB_launcher_sm90.inl:191-198); above 128 the last group may be
 *                    shorter: scales / zeros then hold ceil(k / group_size) rows
 *   alpha            used only with FP8_ALPHA; otherwise must be 1 or is ignored as in the reference
 *   workspace        device scratch of at least woq_workspace_bytes(...) bytes (may be NULL when
 *                    that is 0)
 */
typedef struct woq_matmul_args
{
    const void* act;
    const void* pre_quant_scale;
    const void* weight;
    const void* scales;
    const void* zeros;
    const void* bias;
    void* out;
    float alpha;
    int32_t m;
    int32_t n;
    int32_t k;
    int32_t group_size;
    int32_t quant_algo; /* WOQ_ALGO_* bits */
    int32_t act_dtype;  /* woq_dtype of `act` */
    int32_t out_dtype;  /* woq_dtype of out / scales / zeros / bias / pre_quant_scale: fp16 or bf16 */
    int32_t regime;     /* woq_regime; 0 = automatic */
    void* workspace;
    size_t workspace_bytes;
} woq_matmul_args;

/* Runs the matmul on `stream`.  m == 0 returns WOQ_OK at once (weightOnlyQuantMatmulPlugin.cpp:303).
 * Replaces the bodies of both plugins' enqueue(): kernel_launcher(...) for small m and
 * apply_per_channel_scale + Runner::gemm(...) otherwise. */
int woq_matmul(const woq_matmul_args* args, void* stream);

/* Validates exactly like woq_matmul but launches nothing (usable without a GPU). */
int woq_matmul_check(const woq_matmul_args* args);

/* woq_matmul for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose plugins
 * always receive a workspace from TensorRT.  Same arguments and results, bit for bit, as
 * woq_matmul; `workspace` / `workspace_bytes` are ignored: the split-K partial sums and the
 * smoothed activations go to a device array of WOQ_STATIC_SCRATCH_BYTES that the library itself
 * holds on every GPU it runs on until the process ends.  The call allocates and frees nothing.  A
 * call that would need more scratch than that returns WOQ_ERR_WORKSPACE and launches nothing.
 * All calls on one GPU share that GPU's array: calls that may overlap there (different streams)
 * race; order them, or use woq_matmul with separate workspaces.  Every element of the scratch a
 * call reads was written by that call, so nothing is cleared between calls.
 * Set-up that is not stream work - looking up the array's device address (hipGetSymbolAddress), reading
 * the WOQ_* environment, raising a kernel's dynamic-LDS limit (hipFuncSetAttribute, once per kernel
 * variant and device) - happens on first use: call woq_static_init() on each device before the first
 * woq_matmul_static there, and, before capturing a call into a HIP graph, run that same call (same
 * shape and flags, hence the same kernel variant) once outside capture. */
#define WOQ_STATIC_SCRATCH_BYTES (32u << 20)
int woq_matmul_static(const woq_matmul_args* args, void* stream);
size_t woq_static_scratch_bytes(void);
/* Resolves the scratch array's address on the CURRENT device and reads the environment overrides, so that
 * woq_matmul_static itself makes no non-stream runtime call for them.  Idempotent; WOQ_OK or
 * WOQ_ERR_RUNTIME.  (woq_matmul_static still resolves the address by itself if this was not called.) */
int woq_static_init(void);

/* Device scratch that is enough for every woq_matmul call of this n, k, quant_algo with AT MOST m
 * rows (pass the largest m, as the reference passes its profile's maxM): a region for smoothed
 * activations (PRE_QUANT_SCALE, GEMM regime) followed by the float32 partial sums of the
 * split-K GEMM that skinny problems use, or of the streaming kernels' K split at 4 to 16 rows (one
 * [m, n] slab per slice of K, summed in slice order, so
 * results are bit-reproducible from run to run; the reference's split-K workspace).  Replaces
 * CutlassFpAIntBGemmRunner::getWorkspaceSize (fpA_intB_gemm_template.h:549-582) plus the
 * plugin's own m*k*sizeof(half) smoothing buffer (weightOnlyGroupwiseQuantMatmulPlugin.cpp:377-379). */
size_t woq_workspace_bytes(int32_t m, int32_t n, int32_t k, int32_t quant_algo, int32_t act_dtype);

/*
 * Grouped (mixture-of-experts) matmul: expert e multiplies its own rows of `act` with its own
 * weight matrix, out[rows_e] = act[rows_e] x dequant(W_e) (+ bias_e).  Replaces
 * MoeGemmRunner<T, uint8_t | cutlass::uint4b_t>::moeGemm / moeGemmBiasAct without an activation
 * (kernels/internal_cutlass_kernels/include/moe_gemm_kernels.h:235-244) with the weight-only
 * scales of QuantParams::Int (moe_kernels.h:144-198); groupwise scales / zeros are accepted too.
 *   base.act     [total_rows, k], rows sorted by expert;  base.out  [total_rows, n]
 *   base.m       total_rows
 *   base.weight  num_experts preprocessed matrices back to back (what woq_preprocess_weights
 *                writes for experts = num_experts), woq_preprocessed_bytes(k, n, type) apart
 *   base.scales / base.zeros   [num_experts, n] (group_size 0) or [num_experts, k/group_size, n]
 *   base.bias    [num_experts, n] or NULL
 *   total_rows_before_expert   device memory, int64 [num_experts]: rows of experts 0..e
 *                (inclusive prefix sums, non-decreasing, last = total_rows; the reference's
 *                total_tokens_including_expert); experts may own no rows
 *                With num_experts == 1 it may be NULL: the one expert owns all base.m rows
 *                (the plain matmul with a fused activation).
 *   activation   WOQ_ACT_* applied to (acc + bias) in float32, as moeGemmBiasAct's activation_type.
 *                Gated ones (SWIGLU, GEGLU) read value column j and gate column j + n/2 and write
 *                out [total_rows, n/2] = value * f(gate), the reference's chunk order
 *                (functional.py:804-821, tests/functional/test_moe.py:186-190); n % 32 == 0 then.
 *   residual     optional [total_rows, n_out], same type as out: out = T(f(acc + bias) + residual),
 *                the skip connection behind o_proj / down projections (no counterpart in the
 *                reference's GEMM runners, which leave it to a following elementwise layer).
 * pre_quant_scale, FP8_ALPHA and the workspace are not used (must be NULL / unset).
 * AUTO regime: the streaming kernel while the average expert has at most 16 rows (an expert with
 * more streams its weights once per 16 rows), tiled MFMA kernels above.
 */
typedef enum woq_activation /* values of the reference's ActivationType (moe_gemm_kernels.h:197-206) */
{
    WOQ_ACT_GELU = 0,
    WOQ_ACT_RELU = 1,
    WOQ_ACT_SILU = 2,
    WOQ_ACT_SWIGLU = 3,
    WOQ_ACT_GEGLU = 4,
    WOQ_ACT_IDENTITY = 5
} woq_activation;

typedef struct woq_grouped_matmul_args
{
    woq_matmul_args base;
    const int64_t* total_rows_before_expert;
    int32_t num_experts;
    int32_t activation;   /* woq_activation; note that 0 is GELU, as in the reference */
    const void* residual; /* NULL, or [total_rows, n_out] in the output type: added after the activation */
} woq_grouped_matmul_args;

int woq_grouped_matmul(const woq_grouped_matmul_args* args, void* stream);

/* Validation only (no launch): what woq_grouped_matmul would return for these arguments. */
int woq_grouped_matmul_check(const woq_grouped_matmul_args* args);

/* The regime the built-in rule picks for AUTO: STREAM for m <= 16; for 17 <= m <= 64 (16-bit
 * activations) STREAM where the streaming kernel's estimated time is below the GEMM plan's (small n
 * with short k, e.g. 4096 x 4096 up to 64 rows, 8192 x 8192 up to ~20), GEMM otherwise; for W4A8
 * STREAM up to 32 rows (24 where k >= 2 n) - crossovers measured on MI355X.  Counterpart of the tactic choice
 * (`m < SMALL_M_FAST_PATH`, weightOnlyQuantMatmulPlugin.h:138 and gemmPluginProfiler.cpp:161-178). */
int woq_select_regime(int32_t m, int32_t n, int32_t k, int32_t quant_algo);

/* ---- tactic profiler ------------------------------------------------------------------------ */

/* Times, on `stream`, the built-in choice and every candidate way this library has of running the
 * 16-bit problem `args` describes (streaming launch shapes; deferred-scale / exact-dequantize GEMM
 * kernels, tile heights and K splits) for every m in [min_m, 15], the powers of two from 16 below
 * max_m, and max_m, and records per row count the fastest candidate if it beats the built-in choice
 * by more than 4 % (else "heuristic") in a process-wide table.  Later woq_matmul calls with regime
 * AUTO on the same (n, k, quant_algo, group_size, out_dtype) use the entry of their m, else of the
 * next profiled row count above it, else the built-in heuristics (also when the workspace they are
 * given is too small for the tuned choice, or the entry names a kernel this build lacks).  Replaces
 * GemmPluginProfiler::profileTactics (plugins/common/gemmPluginProfiler.cpp:118-216, timing loop
 * :329-367, lookup :221-250) as called from the plugins' configGemm / initialize
 * (weightOnlyQuantMatmulPlugin.cpp:255-275).  A set-up call: the buffers of `args` must hold
 * max_m rows (workspace: woq_workspace_bytes for max_m; candidates that need more are skipped),
 * `out` is overwritten, the stream is synchronised, 512 MiB of device memory are allocated and
 * freed (the last-level cache is evicted between timed runs), and it must not run under stream
 * capture.  W4A8 problems have one kernel per regime: accepted, nothing recorded. */
int woq_profile_tactics(const woq_matmul_args* args, int32_t min_m, int32_t max_m, void* stream);

/* Entries in the table; emptying it (back to the heuristics). */
int woq_tactic_count(void);
void woq_clear_tactics(void);

/* Writes what a woq_matmul call with these arguments would go by: "heuristic", or the tuned entry
 * ("stream mt=.. ns=.. waves=.. pf=.. lds=..", "gemm exact|skinny rt=.. splits=.."; "heuristic"
 * also for an entry that recorded the built-in choice as the fastest). */
int woq_describe_tactic(const woq_matmul_args* args, char* buf, size_t len);

/* The table as text (one line per entry), so that it can be stored next to a model and loaded
 * instead of profiling again: the reference serialises its tactic map into the engine
 * (weightOnlyQuantMatmulPlugin.cpp:374-391, gemmPluginProfiler.cpp:69-116).  Export returns the
 * bytes needed including the terminator and writes only if len suffices; import adds the entries
 * of `text` to the table (all or none) and rejects text this library did not write. */
size_t woq_export_tactics(char* buf, size_t len);
int woq_import_tactics(const char* text);

/* ---- host-side weight preparation (CPU buffers) ------------------------------------------- */

/* Bytes of the preprocessed weight of one [k, n] matrix.  Equals k*n*bits/8 whenever k is a
 * multiple of 128 (int4) / 64 (int8); otherwise K is padded up to that multiple. */
size_t woq_preprocessed_bytes(int64_t k, int64_t n, int32_t quant_type);

/* Row-major signed [experts, k, n] (int4: two per byte along n, low nibble first) ->
 * the opaque layout the kernels of THIS library read.  Same contract as
 * preprocess_weights_for_mixed_gemm (cutlass_preprocessors.cpp:564-615; torch op
 * trtllm::preprocess_weights_for_mixed_gemm, thop/weightOnlyQuantOp.cpp:123-151): lossless,
 * arch-specific bytes.  Requires n % 16 == 0 and k % 32 == 0. */
int woq_preprocess_weights(void* dst, const void* src, int64_t experts, int64_t k, int64_t n, int32_t quant_type);

/* Inverse of woq_preprocess_weights (no reference counterpart: the reference layout is
 * write-only; provided so the layout is testable and checkpoints can be converted back). */
int woq_unpreprocess_weights(void* dst_row_major, const void* src, int64_t experts, int64_t k, int64_t n,
    int32_t quant_type);

/* Decodes a buffer produced by the REFERENCE's preprocess_weights_for_mixed_gemm on SM `arch`
 * (80..89 / >=100: permute+transpose+interleave+bias; 90: no column interleave) back to
 * row-major signed, so existing TensorRT-LLM checkpoints can be re-laid-out for gfx950.
 * Inverts cutlass_preprocessors.cpp:163-615. */
int woq_import_reference_weights(void* dst_row_major, const void* src_reference_layout, int64_t experts, int64_t k,
    int64_t n, int32_t quant_type, int32_t arch);

/* The single steps of the reference's preprocess on packed row-major weights, as its torch debug
 * operators expose them (thop/weightOnlyQuantOp.cpp:65-120, 252-281, 371-385; the steps themselves
 * cutlass_preprocessors.cpp:186-240 permute_B_rows_for_mixed_gemm, :245-385 subbyte_transpose,
 * :404-507 add_bias_and_interleave_quantized_tensor_inplace).  [experts][k][n] elements of the
 * quant type's width in `src`; `dst` (same size, must not alias) receives the step's result:
 * PERMUTE_ROWS keeps the shape, SUBBYTE_TRANSPOSE writes [experts][n][k], ADD_BIAS_AND_INTERLEAVE
 * works on the flat buffer.  Nothing on the matmul path uses them. */
enum woq_ref_step
{
    WOQ_REF_STEP_PERMUTE_ROWS = 0,
    WOQ_REF_STEP_SUBBYTE_TRANSPOSE = 1,
    WOQ_REF_STEP_ADD_BIAS_AND_INTERLEAVE = 2
};
int woq_reference_layout_step(void* dst, const void* src, int64_t experts, int64_t k, int64_t n, int32_t quant_type,
    int32_t step);

/* Per-column symmetric quantizer + preprocess.  Replaces symmetric_quantize<ComputeType, WeightType>
 * (cutlass_preprocessors.cpp:652-762) behind trtllm::symmetric_quantize_last_axis_of_batched_matrix
 * and trtllm::_symmetric_quantize_last_axis_of_batched_matrix (thop/weightOnlyQuantOp.cpp:153-251).
 * weight [experts, k, n] of weight_dtype (fp32/fp16/bf16); scales [experts, n] of scale_dtype;
 * `processed` (preprocessed bytes) and `unprocessed` (row-major packed) may each be NULL. */
int woq_symmetric_quantize(void* processed, void* unprocessed, void* scales, const void* weight, int64_t experts,
    int64_t k, int64_t n, int32_t quant_type, int32_t weight_dtype, int32_t scale_dtype);

/* trtllm::pack_int8_tensor_to_packed_int4 / trtllm::unpack_int4_packed_tensor_to_int8
 * (thop/weightOnlyQuantOp.cpp:284-353).  n_unpacked must be even. */
int woq_pack_int4(void* packed, const void* unpacked_int8, size_t n_unpacked);
int woq_unpack_int4(void* unpacked_int8, const void* packed, size_t n_packed);

/* ---- device helpers ------------------------------------------------------------------------ */

/* out[m, k] = T_out(T_in(act[m, k] * scale[k])), T_out = T_in or fp8 e4m3.  Replaces
 * apply_per_channel_scale_kernel_launcher<T_in, T_out> (kernels/preQuantScaleKernel.cu:42-149). */
int woq_apply_per_channel_scale(void* out, const void* act, const void* per_channel_scale, int32_t m, int32_t k,
    int32_t in_dtype, int32_t out_dtype, void* stream);

/* RMSNorm fused with the smoothing pass in front of the matmul (one pass over the activations):
 *   normed = T(x * rsqrt(mean(x^2) + eps) * gamma [+ beta]),  out = T_out(T(normed * pre_quant_scale))
 * with T = dtype (fp16 / bf16) and T_out = dtype or fp8 e4m3 (the W4A8 activation).  Replaces
 * invokeGeneralRmsNorm (kernels/rmsnormKernels.cu:230-262, arithmetic at :29-38 and :83-124)
 * followed by apply_per_channel_scale_kernel_launcher (kernels/preQuantScaleKernel.cu:137-149).
 * x, out [m, k]; gamma, beta, pre_quant_scale [k] of dtype; beta and pre_quant_scale may be NULL.
 * k % 8 == 0.  The sum of squares is accumulated in float32 in this kernel's own order. */
int woq_rmsnorm_prequant(void* out, const void* x, const void* gamma, const void* beta, const void* pre_quant_scale,
    float eps, int32_t m, int32_t k, int32_t dtype, int32_t out_dtype, void* stream);

/* Materialises W[k, n] = T(q*scale + zero) from preprocessed weights with the same device code
 * the GEMM main loop uses (counterpart of the identity-activation round trip in
 * tests/quantization/test_weight_only_quant_matmul.py:147-164).  dtype fp16/bf16, or fp8 e4m3
 * with fp16 scales (the W4A8 B operand). */
int woq_dequantize(void* out, const void* weight, const void* scales, const void* zeros, int32_t k, int32_t n,
    int32_t group_size, int32_t quant_type, int32_t dtype, void* stream);

/* ---- misc ------------------------------------------------------------------------------------ */

/* The WOQ_* environment variables (experiment overrides of the built-in kernel choices) are read
 * once, at the first call that consults them; this reads them again.  For tests and tuning scripts;
 * no counterpart in the reference. */
void woq_reload_env(void);

const char* woq_last_error(void);

/* Which kernel the last matmul call of this thread launched, as text: "gemm exact rt=16 splits=1
 * persistent=1", "gemm skinny rt=4 splits=2", "stream mt=.. ns=.. waves=.. pf=.. slots=.. k_slices=..",
 * "stream wide ns=.. waves=.. pf=.. slots=..", "gemm w4a8 ...", "stream w4a8 ..."; empty before the
 * first call.  For tests of the dispatch rules and for tuning scripts; no counterpart in the
 * reference.  The pointer stays valid until the thread's next call of this function. */
const char* woq_last_launch(void);
int woq_abi_version(void);
int woq_layout_version(void);

#ifdef __cplusplus
}
#endif
#endif /* WOQ_H_ */
