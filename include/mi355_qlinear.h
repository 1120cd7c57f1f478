/*
 * mi355_qlinear -- C ABI of the MI355X (gfx950) quantized-linear kernels.
 *
 * One shared library, plain pointers and sizes, no framework types.  Every pointer
 * is a device pointer unless stated otherwise; every call only enqueues work on
 * `stream` (a hipStream_t passed as void*, NULL = the default stream) and returns
 * without synchronizing, so all entry points are usable inside HIP graph capture.
 * The library never allocates or frees device memory: outputs and workspaces are
 * the caller's.
 *
 * Return value: 0 on success, otherwise one of the MI355_ERR_* codes; the message
 * for the calling thread is available from mi355_last_error().
 *
 * Each entry point names the reference interface it stands in for (paths relative
 * to the SGLang source tree).
 */
#ifndef MI355_QLINEAR_H
#define MI355_QLINEAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_QLINEAR_ABI_VERSION 1

/* Element types (values are part of the ABI). */
enum {
  MI355_F32 = 0,
  MI355_F16 = 1,
  MI355_BF16 = 2,
  MI355_FP8_E4M3FN = 3, /* OCP E4M3: max 448, no infinity, 0x7f/0xff NaN */
  MI355_I8 = 4,
  MI355_I32 = 5
};

/* How the group quantizer scales an element once the group's amax is known. */
enum {
  MI355_QUANT_DIV = 0, /* s = amax / qmax;          q = x / s           (per_token_group_quant_8bit.cu:86,:110) */
  MI355_QUANT_RCP = 1, /* s = amax / qmax;          q = x * (1.0f / s)  (fp8_kernel.py:156-158)                */
  MI355_QUANT_MUL = 2  /* s = amax * (1.0f / qmax); q = x * (qmax/amax) (per_token_group_quant_8bit_v2.cu:77-78) */
};

/* What is stored per group. */
enum {
  MI355_SCALE_F32 = 0,         /* float at s[row * s_stride_row + kgroup * s_stride_col]                       */
  MI355_SCALE_UE8M0_PACKED = 1 /* biased exponent byte of a power-of-two scale, four consecutive k-groups per
                                  32-bit word, words column-major: byte address
                                  (kgroup/4) * s_stride_col * 4 + row * 4 + kgroup % 4; the unused bytes of a
                                  row's last word are written as zero
                                  (per_token_group_quant_8bit.cu:54-61, per_token_group_quant_8bit_v2.cu:305-329) */
};

enum {
  MI355_OK = 0,
  MI355_ERR_INVALID_ARGUMENT = 1, /* a shape, stride, alignment or enum the contract excludes */
  MI355_ERR_UNSUPPORTED = 2,      /* valid in the reference, not implemented here             */
  MI355_ERR_LAUNCH = 3,           /* the HIP runtime refused the launch                       */
  MI355_ERR_WORKSPACE = 4         /* workspace missing or smaller than *_workspace_bytes()     */
};

int mi355_qlinear_abi_version(void);

/*
 * Optional set-up of the current device: resolves the device addresses of the library's two built-in device arrays (the
 * scratch of mi355_fp8_blockwise_mm_noalloc and a constant of mi355_fp8_scaled_mm).  Those entry points do the same on
 * their first call on a device; a caller that captures them into a HIP graph calls this first, once per device with that
 * device current, because the first look-up may load the code object and is refused during a capture.  No counterpart in
 * the reference (torch extensions are initialised by their import).  Idempotent and thread-safe.
 */
int mi355_qlinear_init(void);

/* Message of the last failing call on this thread ("" if none).  Host pointer, valid until the next call. */
const char* mi355_last_error(void);

/*
 * Per-token-group 8-bit quantization.
 * Replaces sgl_per_token_group_quant_8bit    (sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:116-217),
 *          sgl_per_token_group_quant_8bit_v2 (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:394-514,
 *                                             without its MoE-only silu/masked variants),
 *          and the Triton kernels behind per_token_group_quant_fp8
 *                                            (python/sglang/srt/layers/quantization/fp8_kernel.py:121-323).
 *
 *   x        [M, K] contiguous, x_dtype in {F32, F16, BF16}
 *   q        [M, K] contiguous, q_dtype FP8_E4M3FN (round to nearest even) or I8 (truncation toward zero)
 *   s        scales, see scale_kind; caller-allocated, written in place
 *   group    elements per scale along K; a power of two with group * sizeof(x element) in [16, 2048] bytes,
 *            dividing K
 *   amax = max(eps, max |x|) in fp32; q is clamped to [qmin, qmax] before conversion
 *   pow2_floor  only for UE8M0 with DIV/RCP: lower bound on amax/qmax before rounding up to a power of two
 *            (1e-10f reproduces per_token_group_quant_8bit.cu:88; 0 reproduces fp8_kernel.py:207-208)
 */
int mi355_group_quant_8bit(const void* x, int x_dtype, void* q, int q_dtype, void* s, int64_t M, int64_t K,
                           int group, float eps, float qmin, float qmax, int mode, int scale_kind,
                           float pow2_floor, int64_t s_stride_row, int64_t s_stride_col, void* stream);

/*
 * Blockwise-scaled FP8 GEMM:  out[m,n] = cast( sum_kb (sum_{k in kb} a[m,k] * b[n,k]) * sa[m,kb] * sb[n/128,kb] ).
 * Replaces fp8_blockwise_scaled_mm (sgl-kernel/csrc/gemm/fp8_blockwise_gemm_kernel.cu:368-465) and
 *          w8a8_block_fp8_matmul   (python/sglang/srt/layers/quantization/fp8_kernel.py:691-773, :1068-1164).
 *
 *   a   [M, K] e4m3fn, K contiguous, row stride lda (bytes == elements)
 *   b   [N, K] e4m3fn, K contiguous, row stride ldb: the weight as stored.  The reference's column-major
 *       `mat_b [K, N]` (stride(0) == 1) is this same memory with ldb = mat_b.stride(1).
 *   sa  fp32, element (m, kb) at sa[m * sa_sm + kb * sa_sk], kb < ceil(K/128)
 *   sb  fp32, element (nb, kb) at sb[nb * sb_sn + kb * sb_sk], nb < ceil(N/128)
 *   out [M, N] BF16, F16 or F32, row stride ldo
 *   K and N need not be multiples of 128 (ragged last blocks are masked like fp8_kernel.py:738-751).
 *   workspace: at least mi355_fp8_blockwise_mm_workspace_bytes(M, N, K) bytes of device memory (may be NULL
 *   when that is 0); used for split-K partial sums, contents undefined afterwards.
 */
size_t mi355_fp8_blockwise_mm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_fp8_blockwise_mm(const void* a, const void* b, const float* sa, const float* sb, void* out, int out_dtype,
                           int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t sa_sm, int64_t sa_sk,
                           int64_t sb_sn, int64_t sb_sk, int64_t ldo, void* workspace, size_t workspace_bytes,
                           void* stream);

/*
 * Grouped blockwise FP8 GEMM: the expert GEMMs of a mixture-of-experts layer in one call.  Token rows of all experts are
 * stacked; expert e owns rows expert_offsets[e] .. expert_offsets[e] + problem_sizes[3 * e] - 1 and
 *   out[r, n] = cast( sum_kb scales_a[r, kb] * scales_b[e, n / 128, kb] * sum_{k in block kb} a[r, k] * b[e, n, k] )
 *   a             e4m3fn [total_m, K], row stride lda;  scales_a fp32, element (r, kb) at scales_a[r * sa_sm + kb * sa_sk]
 *   b             e4m3fn, expert e's [N, K] matrix at b + e * b_expert_stride, row stride ldb (bytes = elements)
 *   scales_b      fp32, block (e, nb, kb) at scales_b[e * sb_expert_stride + nb * sb_sn + kb * sb_sk]
 *   problem_sizes int32 [num_experts, 3] ON THE DEVICE: (rows, N, K) per expert; only the row counts are read, N and K
 *                 are the arguments (the reference's callers build every row with the same N and K)
 *   expert_offsets int32 [num_experts] ON THE DEVICE: first stacked row of each expert
 *   out           bfloat16 or float16 [total_m, N], row stride ldo; rows owned by no expert are left untouched
 * Row counts and offsets are clamped into [0, total_m] on the device, so inconsistent routing data gives wrong rows, not
 * out-of-bounds accesses.  K % 128 == 0 and 16-byte aligned operand rows are required (MI355_ERR_UNSUPPORTED otherwise).
 * The tile schedule and the re-laid-out token scales live in `workspace` (256-byte aligned,
 * >= ..._workspace_bytes(num_experts, total_m, N, K)); nothing is allocated, three or four launches on `stream`.
 * Replaces fp8_blockwise_scaled_grouped_mm (sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:650-810, set-up kernel
 * sgl-kernel/csrc/moe/cutlass_moe_helper.cu:17-80, Python sgl-kernel/python/sgl_kernel/moe.py:96-135; caller
 * cutlass_fused_experts_fp8, python/sglang/srt/layers/moe/cutlass_moe.py:146-201).  The reference's pointer, stride and
 * scale-layout arrays are scratch its own set-up kernel fills; here that scratch is the workspace.
 * ..._plan writes "kernel=grouped_pingpong+grouped_dma3 small_tile=<64|128>x256 max_big_tiles=<n> max_small_tiles=<n>
 * tiles_n=<n>" (host only): experts are cut into 256-row tiles plus, for a rest of at most 128 rows, small tiles.
 */
size_t mi355_fp8_blockwise_scaled_grouped_mm_workspace_bytes(int64_t num_experts, int64_t total_m, int64_t N, int64_t K);
int mi355_fp8_blockwise_scaled_grouped_mm_plan(int64_t num_experts, int64_t total_m, int64_t N, int64_t K, char* buf,
                                               size_t buf_len);
int mi355_fp8_blockwise_scaled_grouped_mm(const void* a, const void* b, const float* scales_a, const float* scales_b, void* out,
                                          int out_dtype, const int32_t* problem_sizes, const int32_t* expert_offsets,
                                          int64_t num_experts, int64_t total_m, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                          int64_t b_expert_stride, int64_t sa_sm, int64_t sa_sk, int64_t sb_expert_stride,
                                          int64_t sb_sn, int64_t sb_sk, int64_t ldo, void* workspace, size_t workspace_bytes,
                                          void* stream);

/*
 * Blockwise FP8 GEMM with power-of-two (UE8M0) scales on BOTH operands, the form DeepSeek-V3 checkpoints take after
 * requant_weight_ue8m0 and activations take from per_token_group_quant_fp8(scale_ue8m0=True):
 *   out[m,n] = cast( sum_kb 2^(ea[m,kb] - 127) * 2^(eb[n,kb] - 127) * sum_{k in block kb} a[m,k] * b[n,k]  (+ bias[n]) )
 *   sa_words  int32, four exponent bytes per word (byte kb & 3 of word kb >> 2): word (m, kw) at sa_words[kw * sa_sk + m]
 *             (token index fastest: the packed column-major layout of create_per_token_group_quant_fp8_output_scale)
 *   sb_words  int32, same packing per weight ROW: word (n, kw) at sb_words[n * sb_sn + kw * sb_sk]; the rows of one
 *             128-channel block carry the same bytes (what the 128 x 128 block requantization produces); one row of the
 *             block is read, which one depends on the kernel
 *   bias      NULL or [N] in the output dtype, added in the epilogue
 * On gfx950 the matrix instruction applies such scales itself (v_mfma_scale_f32_16x16x128_f8f6f4), so for large M, for
 * the mid-M shapes on the three-stage kernel and for the decode sizes (M <= 16, both decode kernels) the K loop carries
 * no scale arithmetic at all and nothing runs in front of the GEMM (K % 128 == 0 and, above decode sizes, token words
 * with a 16-byte aligned base and a pitch that is a multiple of four words); other shapes (ragged K, the generic and
 * the two-stage kernels' shapes) expand the exponents to fp32 scales in the workspace and take the kernels of
 * mi355_fp8_blockwise_mm.  Replaces w8a8_block_fp8_matmul_deepgemm / deep_gemm gemm_nt_f8f8bf16
 * (python/sglang/srt/layers/quantization/fp8_kernel.py:1047-1065; caller deepgemm_w8a8_block_fp8_linear_with_fallback,
 * fp8_utils.py:217-255), whose kernel lives in the DeepGEMM package, not in the reference tree.
 */
size_t mi355_fp8_blockwise_mm_ue8m0_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_fp8_blockwise_mm_ue8m0(const void* a, const void* b, const void* sa_words, const void* sb_words, const void* bias,
                                 void* out, int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                 int64_t sa_sk, int64_t sb_sn, int64_t sb_sk, int64_t ldo, void* workspace,
                                 size_t workspace_bytes, void* stream);

/*
 * mi355_fp8_blockwise_mm for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose operators allocate
 * their workspaces through the framework.  Same arguments and results as mi355_fp8_blockwise_mm without the workspace:
 * split-K partial sums go to a MI355_NOALLOC_SCRATCH_BYTES array that lives in the library's device image (each GPU
 * that loads the library holds one until the process ends).  The call allocates and frees nothing.
 *   - A problem whose partial sums do not fit (splits * M * N * 4 bytes, see mi355_fp8_blockwise_mm_plan) is rejected
 *     with MI355_ERR_WORKSPACE; problems that need no split always pass.
 *   - All calls on one GPU share that GPU's array: calls that may overlap in time on one GPU (different streams,
 *     different threads) race on it and must be serialized by the caller.  Calls on one stream are ordered and safe.
 *   - The device must be the current device of the calling thread.  The first call on a device looks up the array's
 *     address (hipGetSymbolAddress); make that call outside graph capture.
 */
#define MI355_NOALLOC_SCRATCH_BYTES (32u << 20)
int mi355_fp8_blockwise_mm_noalloc(const void* a, const void* b, const float* sa, const float* sb, void* out,
                                   int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                   int64_t sa_sm, int64_t sa_sk, int64_t sb_sn, int64_t sb_sk, int64_t ldo, void* stream);

/*
 * Measurement aid, not an operator (no counterpart in the reference): the large-M kernel of mi355_fp8_blockwise_mm with
 * the global loads of its K loop taken out.  K blocks 0 and 1 and the token scales of blocks 0..3 are fetched once;
 * every later K block multiplies those again, so the matrix instructions, promotion FMAs, LDS reads, barriers and the
 * epilogue are the operator's, on the operator's operand values, and `out` is NOT the product.  Timed beside the
 * operator on the same buffers it gives the ceiling the schedule and the chip's sustained clock set once memory is out
 * of the picture (bench.py --workload fp8_ceiling).  Accepts only shapes the operator runs on that kernel, with K a
 * multiple of 128 (at least 512) and M-major token scales (sa_sm == 1, sa_sk % 4 == 0, 16-byte aligned base).
 */
int mi355_fp8_blockwise_mm_kloop_ceiling(const void* a, const void* b, const float* sa, const float* sb, void* out,
                                         int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                         int64_t sa_sm, int64_t sa_sk, int64_t sb_sn, int64_t sb_sk, int64_t ldo, void* stream);

/*
 * Measurement aid, not an operator (no counterpart in the reference): the fp8 matrix-instruction stream of the large-M
 * kernels with every operand in registers (no LDS, no global loads, no barriers), `workgroups` workgroups of 8 waves,
 * `iters` rounds of 16 instructions of 2 * 16 * 16 * 128 FLOP per wave.  mode 0: C = 0 and four promotion FMAs per result
 * (the fp32-scale kernel's compute phase); 1: accumulating in place (the UE8M0 kernel's); 2: C = 0, no vector arithmetic;
 * 3: as 2 with v_mfma_f32_32x32x64_f8f6f4 (8 instructions of twice the FLOP), the instruction shape the kernels do not use.
 * a, b: 8 * 4 * 64 * 32 = 65536 bytes of e4m3fn operand values each (the timing depends on them through the chip's power
 * management); out: workgroups * 512 floats.  bench.py --workload mfma_stream reports the rates.
 */
int mi355_probe_fp8_mfma_stream(int mode, int workgroups, int iters, const void* a, const void* b, void* out, void* stream);

/*
 * The same for the INT8 kernels (measurement aid, no counterpart in the reference): the same number of operations per
 * round and wave, accumulating in place.  mode 0: 32 v_mfma_i32_16x16x64_i8 (the instruction the INT8 kernels use);
 * 1: 16 v_mfma_i32_32x32x32_i8.  a, b: 65536 bytes of int8 operand values each; out: workgroups * 512 int32.
 */
int mi355_probe_int8_mfma_stream(int mode, int workgroups, int iters, const void* a, const void* b, void* out, void* stream);

/*
 * Per-token x per-channel INT8 GEMM:  acc = sum_k a[m,k] * b[n,k] exactly in int32;
 *   out[m,n] = cast( f32(acc) * (sb[n] * sa[m]) + f32(bias[n]) ).
 * Replaces int8_scaled_mm (sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:663-747; epilogue order of
 *          sgl-kernel/csrc/cutlass_extensions/epilogue/epilogue_per_row_per_col_scale.h:273-303).
 *
 *   a [M, K] int8 row stride lda;  b [N, K] int8 row stride ldb (the reference's column-major mat_b [K, N]);
 *   sa [M], sb [N] fp32 contiguous; bias NULL or [N] in the output dtype; out [M, N] BF16/F16 row stride ldo.
 *   out_dtype MI355_I32 writes the raw accumulators instead (sa, sb, bias ignored): the hook that lets a
 *   test prove the accumulation exact before any rounding.
 */
size_t mi355_int8_scaled_mm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_int8_scaled_mm(const void* a, const void* b, const float* sa, const float* sb, const void* bias, void* out,
                         int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldo,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Host-only query: which kernel and tiling mi355_fp8_blockwise_mm / mi355_int8_scaled_mm would run for a shape.
 * Stands in for the reference's shape dispatchers, which are compile-time ladders nobody can ask
 * (sgl-kernel/csrc/gemm/fp8_blockwise_gemm_kernel.cu:181-195, sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:603-661);
 * here the choice is observable so that tests can prove every kernel variant is reached.
 *   aligned  nonzero if both operand base pointers and row strides are multiples of 16 bytes (rows are assumed dense)
 *   buf      receives a NUL-terminated "key=value ..." line:
 *            kernel=decode|decode_wavesplit|dma3|pingpong|pingpong128|pipelined|generic bm= bn= splits= kb_per_split=
 *            groups_per_wg= aligned= stages=   (stages: LDS stages of the mid-M kernel's pipeline, 0 for the other kernels)
 * Launches nothing and touches no device state.
 */
int mi355_fp8_blockwise_mm_plan(int64_t M, int64_t N, int64_t K, int aligned, char* buf, size_t buf_len);
int mi355_int8_scaled_mm_plan(int64_t M, int64_t N, int64_t K, int aligned, char* buf, size_t buf_len);

/*
 * Host-only: the measured constants of the dispatcher's time models (sglang_amd/csrc/route_constants.h holds the table and
 * where each number comes from) and the plan a shape would get with ONE constant multiplied by `factor`.  No counterpart
 * in the reference, whose dispatch ladders hold their thresholds inline (fp8_blockwise_gemm_kernel.cu:181-195,
 * int8_gemm_kernel.cu:603-661); here a test perturbs every constant by +-10 % and checks that the benchmark shapes stay on
 * their kernels.  The perturbed copy is local to the calling thread and gone when the call returns.
 *   constant_index  0 .. mi355_route_constant_count() - 1;  is_fp8 nonzero for the FP8 GEMM, zero for the INT8 GEMM
 */
int mi355_route_constant_count(void);
const char* mi355_route_constant_name(int index);
double mi355_route_constant_value(int index);
int mi355_gemm_plan_perturbed(int is_fp8, int64_t M, int64_t N, int64_t K, int aligned, int constant_index, double factor,
                              char* buf, size_t buf_len);

/*
 * Per-token INT8 activation quantization: absmax = max(1e-10, max |x[m,:]|), s[m] = absmax / 127,
 * q = round-half-away-from-zero(x * (127 / absmax)).
 * Replaces per_token_quant_int8 (python/sglang/srt/layers/quantization/int8_kernel.py:28-89, without cal_sum).
 *   x [M, K] contiguous F32/F16/BF16; q [M, K] int8 contiguous; s [M] fp32.  K * sizeof(x element) % 16 == 0.
 */
int mi355_per_token_quant_int8(const void* x, int x_dtype, void* q, float* s, int64_t M, int64_t K, void* stream);

/*
 * The same with the row sums: x_sum[m] = T(sum_k f32(x[m,k])), accumulated in fp32 and rounded to the input's type T, which
 * is also the type of x_sum [M].  Replaces per_token_quant_int8(cal_sum=True) (int8_kernel.py:52-54, :66-69; the INT8
 * mixture-of-experts path uses the sums).  The reference's reduction order is whatever Triton's tl.sum emits, so the sum is
 * defined up to fp32 reassociation; codes and scales are those of mi355_per_token_quant_int8, bit for bit.
 */
int mi355_per_token_quant_int8_sum(const void* x, int x_dtype, void* q, float* s, void* x_sum, int64_t M, int64_t K, void* stream);

/*
 * Per-token FP8 activation quantization: s[m] = max |x[m,:]| / 448 (no floor), q = e4m3fn(clamp(x * (1 / s[m]))) rounded to
 * nearest even; a row of zeros gives s = 0 and zeros.
 * Replaces sgl_per_token_quant_fp8 (sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:162-227, arithmetic of its
 *          warp-per-token kernel :15-85; its small-batch kernel :91-160 omits the zero test and yields NaN for such a row).
 *   x [M, K] contiguous F32/F16/BF16; q [M, K] e4m3fn contiguous; s [M] fp32.  K * sizeof(x element) % 16 == 0.
 */
int mi355_per_token_quant_fp8(const void* x, int x_dtype, void* q, float* s, int64_t M, int64_t K, void* stream);

/* Per-token-group FP8 quantization with the whole row as ONE group: s[m] = max(absmax of row m, eps) / 448 and
 * q = e4m3fn(clamp(x * (1 / s[m]), -448, 448)) (mode MI355_QUANT_RCP) or q = e4m3fn(clamp(x / s[m], -448, 448)) with a
 * true division (mode MI355_QUANT_DIV).
 *
 * Replaces per_token_group_quant_fp8 called with group_size == K, which is how the reference quantizes the weights of a
 * 16-bit checkpoint per output channel at load time (python/sglang/srt/layers/quantization/fp8.py:368-375:
 * per_token_group_quant_fp8(layer.weight, layer.weight.shape[-1]), the Triton kernel fp8_kernel.py:122-161 = RCP), and
 * sgl_per_token_group_quant_8bit with such a group (sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:25-114 = DIV).
 * mi355_group_quant_8bit covers power-of-two groups of up to 2048 input bytes; this entry covers rows of any length
 * that is a multiple of 16 bytes.
 * x [M, K] contiguous f32/f16/bf16 (16-byte aligned), q [M, K] e4m3fn (8-byte aligned), s [M] fp32. */
int mi355_row_group_quant_fp8(const void* x, int x_dtype, void* q, float* s, int64_t M, int64_t K, float eps, int mode,
                              void* stream);

/*
 * Weight-side 128 x 128 block quantization (load time: re-quantizing a block-FP8 checkpoint to power-of-two scales).
 *   mi355_block_cast_to_fp8:  x [m, n] contiguous F32/F16/BF16 -> q [m, n] e4m3fn, s [ceil(m/128), ceil(n/128)] fp32
 *       contiguous;  amax = max(1e-4, max |x| over the block), s = 2^ceil(log2(amax / 448)) exactly, q = e4m3fn(x * (1 / s)).
 *       Replaces per_block_cast_to_fp8 + ceil_to_ue8m0 (python/sglang/srt/layers/quantization/fp8_utils.py:487-505), which
 *       the reference writes in torch ops (zero padding to whole blocks included, which changes no maximum).
 *   mi355_block_dequant_fp8:  q [n, k] e4m3fn, s [ceil(n/128), ceil(k/128)] fp32 contiguous -> out [n, k] = T(float(q) * s).
 *       Replaces block_quant_dequant (fp8_utils.py:392-413) for 128 x 128 blocks.
 */
int mi355_block_cast_to_fp8(const void* x, int x_dtype, void* q, float* s, int64_t m, int64_t n, void* stream);
int mi355_block_dequant_fp8(const void* q, const float* s, void* out, int out_dtype, int64_t n, int64_t k, void* stream);

/*
 * silu(gate) * up fused in front of the 1 x 128 FP8 group quantizer (the MoE expert MLP's activation + quantization).
 *   x [E, T, 2 * H] contiguous F16/BF16, each row gate | up;  q [E, T, H] e4m3fn contiguous;
 *   v = T( float(T(silu(float(gate)))) * float(up) ) in the input's type T, then per 128 values amax = max(1e-10, max |v|),
 *   e = ceil(log2(amax / 448)), q = e4m3fn(clamp(v * 2^-e)), scale byte e + 127.
 *   s_words: int32 words of four exponent bytes (byte kg & 3 of word kg >> 2 for group kg of a row); word (e, t, kw) lies
 *   at s_words[e * s_expert_stride + kw * s_k_stride + t] - token index fastest, the packed column-major layout of
 *   create_per_token_group_quant_fp8_output_scale(scale_ue8m0=True).  Unused bytes of a row's last word are set to 0.
 *   masked_m: NULL, or [E] int32 on the device: tokens t >= masked_m[e] of expert e are neither read nor written.
 * Replaces sgl_per_token_group_quant_8bit_v2 with fuse_silu_and_mul (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:
 * 394-514, kernel :250-392, masked scheduler :194-238), which exists for exactly this scale format.  exp is evaluated by a
 * fixed sequence of fp32 operations, within 1 ulp (the reference uses the GPU's approximate intrinsic).  H % 128 == 0.
 */
int mi355_silu_mul_group_quant_fp8(const void* x, int x_dtype, void* q, void* s_words, int64_t E, int64_t T, int64_t H,
                                   const int32_t* masked_m, int64_t s_expert_stride, int64_t s_k_stride, void* stream);

/*
 * Per-tensor FP8 activation quantization: ONE fp32 scale for the whole tensor, q = e4m3fn(clamp(x * (1 / scale))).
 *   is_static == 0: scale = max |x| / 448 is computed first.  *scale must hold 0.0f on entry (block maxima are merged into
 *                   it with an atomic max; the reference's wrapper passes torch.zeros(1) the same way).
 *   is_static != 0: *scale is given.  scale_rows, if not NULL, receives `rows` copies of it (the per-token shape that
 *                   fp8_scaled_mm wants for a per-tensor scale).
 * Replaces sgl_per_tensor_quant_fp8 (sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:102-130, kernels :10-100) and the
 * Triton static_quant_fp8 (python/sglang/srt/layers/quantization/fp8_kernel.py:593-665), whose arithmetic is the same.
 * A tensor of zeros quantized dynamically gets scale 0 and, like in the reference, codes of +448 (0 * inf = NaN meets
 * fmin/fmax).  x: numel contiguous F32/F16/BF16 elements, 16-byte aligned; q: numel e4m3fn bytes, 8-byte aligned.
 */
int mi355_per_tensor_quant_fp8(const void* x, int x_dtype, void* q, float* scale, int64_t numel, int is_static,
                               float* scale_rows, int64_t rows, void* stream);

/*
 * Per-token x per-channel FP8 GEMM:  out[m,n] = cast( sa[m] * sb[n] * sum_k a[m,k] * b[n,k] + f32(bias[n]) ), fp32 accumulate.
 * Replaces fp8_scaled_mm (sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:1450-1532, epilogue :529-547; caller apply_fp8_linear,
 *          python/sglang/srt/layers/quantization/fp8_utils.py:565-853).
 *   a [M, K] e4m3fn row stride lda;  b [N, K] e4m3fn row stride ldb (the reference's column-major mat_b [K, N]);
 *   sa [M], sb [N] fp32 contiguous; bias NULL or [N] in the output dtype; out [M, N] BF16/F16 row stride ldo.
 *   It runs on the blockwise kernels (token scale applied when a 128-wide K block is promoted, channel scale and bias
 *   in the epilogue); workspace as for mi355_fp8_blockwise_mm.
 */
size_t mi355_fp8_scaled_mm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_fp8_scaled_mm(const void* a, const void* b, const float* sa, const float* sb, const void* bias, void* out,
                        int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldo,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * One block-FP8 linear layer in one call:  out = cast( blockwise_mm(quantize_1x128(x), w) + f32(bias) ).
 * Replaces the call sequence of cutlass_w8a8_block_fp8_linear_with_fallback / triton_w8a8_block_fp8_linear
 *          (python/sglang/srt/layers/quantization/fp8_utils.py:184-214, :281-301): per_token_group_quant_fp8, the blockwise
 *          GEMM and `output += bias`.  The activation is quantized with q = x / s (s = max(amax, 1e-10) / 448) into the
 *          workspace, with M-major scales, and the bias is added in fp32 in the GEMM epilogue (the reference adds it
 *          after rounding the GEMM result to the output type).  At decode sizes (M <= 16, 16-bit x, N % 128 == 0) there
 *          is no quantizer launch where that is the faster way: the GEMM kernel quantizes the tokens itself (the streaming
 *          kernel in its prologue, the mid-M kernel by producer waves), with the same arithmetic, and the result is
 *          bit-identical to the two-step sequence.
 *          mi355_fp8_block_linear_plan (host only, dense 16-byte aligned operands assumed) writes the GEMM's plan in the
 *          format of mi355_fp8_blockwise_mm_plan followed by quantizer=fused|launch.
 *   x [M, K] contiguous F32/F16/BF16, K % 128 == 0; w [N, K] e4m3fn row stride ldw; w_scale element (nb, kb) at
 *   w_scale[nb * ws_sn + kb * ws_sk]; bias NULL or [N] in the output dtype; out [M, N] BF16/F16 row stride ldo.
 *   workspace: mi355_fp8_block_linear_workspace_bytes(M, N, K) bytes, 256-byte aligned.
 */
size_t mi355_fp8_block_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_fp8_block_linear(const void* x, int x_dtype, const void* w, const float* w_scale, int64_t ws_sn, int64_t ws_sk,
                           const void* bias, void* out, int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldw,
                           int64_t ldo, void* workspace, size_t workspace_bytes, void* stream);
/* The same with the quantizer's arithmetic chosen: MI355_QUANT_DIV as above (fp8_utils.py:201-203, the M-major-scale path),
 * MI355_QUANT_RCP for q = x * (1 / s), which is what triton_w8a8_block_fp8_linear's quantizer computes (fp8_utils.py:293-295,
 * fp8_kernel.py:156-158).  Either way the result is bit-identical to that wrapper's quantizer followed by the blockwise GEMM. */
int mi355_fp8_block_linear_mode(const void* x, int x_dtype, int quant_mode, const void* w, const float* w_scale, int64_t ws_sn,
                                int64_t ws_sk, const void* bias, void* out, int out_dtype, int64_t M, int64_t N, int64_t K,
                                int64_t ldw, int64_t ldo, void* workspace, size_t workspace_bytes, void* stream);
int mi355_fp8_block_linear_plan(int64_t M, int64_t N, int64_t K, char* buf, size_t buf_len);

/*
 * One INT8 linear layer in one call:  out = int8_scaled_mm(per_token_quant_int8(x), w) with scales and bias in the GEMM epilogue.
 * Replaces the call sequence of W8A8Int8LinearMethod.apply (python/sglang/srt/layers/quantization/w8a8_int8.py:387-417):
 *          per_token_quant_int8 (int8_kernel.py:28-89), then int8_scaled_mm (sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:663-747).
 *          The codes and token scales go to the workspace; the result is that of mi355_per_token_quant_int8 followed by
 *          mi355_int8_scaled_mm, bit for bit (the same two kernels on the same data).
 *   x [M, K] contiguous F32/F16/BF16, K * sizeof(x element) % 16 == 0; w [N, K] int8 row stride ldw (the reference's
 *   column-major [K, N]); w_scale [N] fp32; bias NULL or [N] in the output dtype; out [M, N] BF16/F16 row stride ldo.
 *   workspace: mi355_int8_linear_workspace_bytes(M, N, K) bytes, 256-byte aligned.
 */
size_t mi355_int8_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_int8_linear(const void* x, int x_dtype, const void* w, const float* w_scale, const void* bias, void* out, int out_dtype,
                      int64_t M, int64_t N, int64_t K, int64_t ldw, int64_t ldo, void* workspace, size_t workspace_bytes,
                      void* stream);

/*
 * One per-token x per-channel FP8 linear layer in one call:  out = fp8_scaled_mm(per_token_quant_fp8(x), w).
 * Replaces the dynamic per-token branch of apply_fp8_linear (python/sglang/srt/layers/quantization/fp8_utils.py:786-808):
 *          sglang_per_token_quant_fp8 (fp8_kernel.py:573-589), then fp8_scaled_mm.  Codes and token scales go to the
 *          workspace; the result is that of mi355_per_token_quant_fp8 followed by mi355_fp8_scaled_mm, bit for bit.
 *   x [M, K] contiguous F32/F16/BF16, K * sizeof(x element) % 16 == 0; w [N, K] e4m3fn row stride ldw; w_scale [N] fp32;
 *   bias NULL or [N] in the output dtype; out [M, N] BF16/F16 row stride ldo.
 *   workspace: mi355_fp8_per_token_linear_workspace_bytes(M, N, K) bytes, 256-byte aligned.
 */
size_t mi355_fp8_per_token_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_fp8_per_token_linear(const void* x, int x_dtype, const void* w, const float* w_scale, const void* bias, void* out,
                               int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldw, int64_t ldo, void* workspace,
                               size_t workspace_bytes, void* stream);

/*
 * One block-FP8 linear layer with packed power-of-two scales in one call:
 *   out = mi355_fp8_blockwise_mm_ue8m0(quantize_1x128_ue8m0(x), w).
 * Replaces the call sequence of deepgemm_w8a8_block_fp8_linear_with_fallback (python/sglang/srt/layers/quantization/
 *          fp8_utils.py:217-255): sglang_per_token_group_quant_fp8(column_major_scales, scale_tma_aligned, scale_ue8m0)
 *          (q = x * (448 / amax), scale rounded up to a power of two: per_token_group_quant_8bit_v2.cu:77-78), then the
 *          GEMM.  Codes and packed token words go to the workspace; the result is that of mi355_group_quant_8bit with
 *          those arguments followed by mi355_fp8_blockwise_mm_ue8m0, bit for bit.
 *   x [M, K] contiguous F16/BF16, K % 128 == 0; w [N, K] e4m3fn row stride ldw; sb_words as for mi355_fp8_blockwise_mm_ue8m0;
 *   bias NULL or [N] in the output dtype (added in the epilogue); out [M, N] BF16/F16 row stride ldo.
 *   workspace: mi355_fp8_block_linear_ue8m0_workspace_bytes(M, N, K) bytes, 256-byte aligned.
 */
size_t mi355_fp8_block_linear_ue8m0_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_fp8_block_linear_ue8m0(const void* x, int x_dtype, const void* w, const void* sb_words, int64_t sb_sn, int64_t sb_sk,
                                 const void* bias, void* out, int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldw,
                                 int64_t ldo, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_QLINEAR_H */
