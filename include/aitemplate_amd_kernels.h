/*
 * C ABI of libaitemplate_amd_kernels.so: the gfx950 (MI355X) kernels of the
 * AITemplate ROCm GEMM family and their launch shim.
 *
 * These entry points are what the per-op launch functions emitted by the ROCm
 * GEMM codegen bind to.  In the reference each generated function
 *     void <op_name>(void* in, void* weight, void* out, [void* bias, void* d0,
 *                    void* d1,] int64_t* dims..., hipStream_t stream)
 * (python/aitemplate/backend/rocm/gemm/common.py:107-171, :491-521) builds a
 * Composable Kernel argument and calls `invoker.Run` (common.py:69-86); here the
 * same generated function evaluates M/N/K from the dim pointers and calls one
 * of the launchers below with the algo index its profiler selected.
 *
 * Conventions
 *  - plain pointers and sizes only; all tensor pointers are device pointers;
 *    `stream` is a hipStream_t passed as void* (NULL = default stream);
 *  - row-major, K-contiguous operands ("RCR": A[M,K], B[N,K], C[M,N]);
 *    ld* are row pitches in elements, batch strides are in elements;
 *  - dtype: 0 = fp16, 1 = bf16 (inputs, residuals and output share it);
 *    accumulation and the epilogue are fp32;
 *  - return value 0 on success, non-zero on failure with a thread-local
 *    message available from aitamd_last_error(); nothing throws across the
 *    boundary and no entry point synchronises the stream;
 *  - launchers are re-entrant and stream-ordered: no global mutable state.
 */
#ifndef AITEMPLATE_AMD_KERNELS_H_
#define AITEMPLATE_AMD_KERNELS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AITAMD_API __attribute__((visibility("default")))

/* Epilogue ids == the reference's gemm_flag / element-wise functor table
 * (python/aitemplate/backend/rocm/gemm/common.py:269-309). */
enum {
  AITAMD_EPI_NONE = 0,                  /* gemm_rcr, bmm_rcr          : PassThrough  */
  AITAMD_EPI_BIAS = 1,                  /* gemm_rcr_bias              : Add          */
  AITAMD_EPI_BIAS_RELU = 2,             /* gemm_rcr_bias_relu         : AddRelu      */
  AITAMD_EPI_BIAS_GELU = 3,             /* gemm_rcr_bias_{fast_,}gelu : AddFastGelu  */
  AITAMD_EPI_BIAS_ADD = 4,              /* gemm_rcr_bias_add          : AddAdd       */
  AITAMD_EPI_BIAS_ADD_ADD = 5,          /* gemm_rcr_bias_add_add      : AddAddAdd    */
  AITAMD_EPI_BIAS_ADD_RELU = 6,         /* gemm_rcr_bias_add_relu     : AddAddRelu   */
  AITAMD_EPI_BIAS_ADD_ADD_RELU = 7,     /* gemm_rcr_bias_add_add_relu : AddAddAddRelu*/
  AITAMD_EPI_BIAS_SIGMOID = 8,          /* gemm_rcr_bias_sigmoid      : AddSigmoid   */
  AITAMD_EPI_BIAS_TANH = 9,             /* gemm_rcr_bias_tanh         : AddTanh      */
  AITAMD_EPI_BIAS_SWISH = 10,           /* gemm_rcr_bias_swish        : AddSwish     */
  AITAMD_EPI_BIAS_HARDSWISH = 11,       /* gemm_rcr_bias_hardswish    : AddHardswish */
  AITAMD_EPI_BIAS_MUL = 12,             /* gemm_rcr_bias_mul          : AddMul       */
  AITAMD_EPI_BIAS_MUL_ADD = 13,         /* gemm_rcr_bias_mul_add      : AddMulAdd    */
  AITAMD_EPI_BIAS_SIGMOID_MUL = 14,     /* gemm_rcr_bias_sigmoid_mul  : AddSigmoidMul*/
  AITAMD_EPI_BIAS_SIGMOID_MUL_TANH = 15,/* gemm_rcr_bias_sigmoid_mul_tanh            */
  AITAMD_EPI_BIAS_MUL_TANH = 16,        /* gemm_rcr_bias_mul_tanh     : AddMulTanh   */
  AITAMD_EPI_ADD = 17,                  /* bmm_{rrr,ccr,crr}_add      : acc + D0, no bias */
  AITAMD_NUM_EPILOGUES = 18
};

enum { AITAMD_F16 = 0, AITAMD_BF16 = 1 };

/* Library version string, e.g. "aitemplate_amd 0.1 gfx950". */
AITAMD_API const char* aitamd_version(void);

/* Message of the last failure on the calling thread ("" if none). */
AITAMD_API const char* aitamd_last_error(void);

/* ---- instance ("algo") table: replaces the CK instance manifest the reference
 * profiler iterates (python/aitemplate/utils/mk_ck_lib/generator.py:517-861,
 * consumed at python/aitemplate/backend/rocm/gemm/common.py:945-1020). ------- */

/* Number of compiled tile instances for (epilogue, dtype); 0 if none. */
AITAMD_API int aitamd_gemm_num_algos(int epilogue, int dtype);

/* Name of instance `algo` (stable, used as the profiler's OP:<name>), or NULL. */
AITAMD_API const char* aitamd_gemm_algo_name(int epilogue, int dtype, int algo);

/* Index of the instance called `name`, or -1. */
AITAMD_API int aitamd_gemm_find_algo(int epilogue, int dtype, const char* name);

/* 1 if instance `algo` can run this problem (K / pitch / pointer alignment for
 * its load width), else 0.  `align_bytes` is the smallest power-of-two
 * alignment shared by the A and B base pointers (pass 16 when unknown-but-
 * allocator-aligned).  Mirrors the role of CK's IsSupportedArgument
 * (python/aitemplate/backend/rocm/gemm/common.py:78-82). */
AITAMD_API int aitamd_gemm_algo_supported(int epilogue, int dtype, int algo,
                                          int64_t M, int64_t N, int64_t K,
                                          int64_t lda, int64_t ldb, int align_bytes);

/* Heuristic choice used when no profiling result exists (algo = -1 below);
 * the counterpart of the reference's select_minimal_algo CI shortcut
 * (python/aitemplate/backend/rocm/target_def.py:214-234) but shape-aware. */
AITAMD_API int aitamd_gemm_heuristic_algo(int epilogue, int dtype, int64_t batch,
                                          int64_t M, int64_t N, int64_t K,
                                          int64_t lda, int64_t ldb, int align_bytes);

/* ---- launchers ------------------------------------------------------------ */

/* C[m,n] = epilogue( sum_k A[m,k] * B[n,k], bias[n], d0[m,n], d1[m,n] ).
 * Unused pointers (per the epilogue) may be NULL.  d0/d1 have row pitch ldd.
 * algo = -1 selects the heuristic instance.  M, N or K equal to 0 is a no-op
 * (K == 0 still writes epilogue(0, ...), matching an empty sum).
 * Replaces the generated gemm_rcr* op functions' CK call
 * (python/aitemplate/backend/rocm/gemm/common.py:132-169). */
AITAMD_API int aitamd_gemm_rcr(int epilogue, int dtype, int algo,
                               const void* a, const void* b, const void* bias,
                               const void* d0, const void* d1, void* c,
                               int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd,
                               void* stream);

/* Scratch memory for instances that split tiles between workgroups along K (the "splitk" instances): bytes that
 * instance `algo` needs for this problem on the current device, 0 for every other instance.  The reference's ops
 * carry the same quantity as their `workspace` attribute, filled from the profiler's WS:<bytes> field
 * (python/aitemplate/compiler/ops/gemm_universal/gemm_common.py:201-215, 566-569) and served from the model's one
 * shared workspace (python/aitemplate/compiler/transform/memory_planning.py:155-194). */
AITAMD_API int64_t aitamd_gemm_workspace_bytes(int epilogue, int dtype, int algo, int64_t batch,
                                               int64_t M, int64_t N, int64_t K);

/* aitamd_gemm_rcr with scratch memory: `workspace` is device memory, 16-byte aligned, of `workspace_bytes` bytes.
 * Its first 4096 bytes must be zero before the first launch that uses the buffer; every launch leaves them zero
 * again, so one memset after allocation serves any number of launches.  Launches that overlap in time (different
 * streams) need buffers of their own.  algo = -1 may then choose a splitk instance; a splitk instance that gets no
 * buffer, or one smaller than aitamd_gemm_workspace_bytes says, runs without sharing tiles (as the plain instance of
 * the same tile, touching no scratch memory); instances that need no scratch memory ignore the buffer.
 * Same role as the generated op functions' `workspace` argument in the reference
 * (python/aitemplate/backend/rocm/gemm/common.py:491-521, func_call with the global workspace pointer). */
AITAMD_API int aitamd_gemm_rcr_ws(int epilogue, int dtype, int algo,
                                  const void* a, const void* b, const void* bias,
                                  const void* d0, const void* d1, void* c,
                                  int64_t M, int64_t N, int64_t K,
                                  int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd,
                                  void* workspace, int64_t workspace_bytes, void* stream);

/* aitamd_gemm_rcr_ws for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc): the scratch memory is a 16 MiB array inside the library's device image, one per GPU, held
 * from the first call on that GPU until the process ends; the call itself allocates and frees nothing.  It has no
 * counterpart in the reference (whose ops draw their workspace from the model's allocation).  An instance named by
 * `algo` that needs more than aitamd_gemm_noalloc_scratch_bytes() for this problem is refused with a message;
 * algo = -1 chooses among the instances that fit.  All calls on one GPU share that GPU's array: calls that overlap
 * in time on one GPU (different streams) race - serialise them, or use aitamd_gemm_rcr_ws with separate buffers.
 * The first call on a GPU looks the array's address up (hipGetSymbolAddress, under a lock).  Under stream capture
 * that look-up must already have happened: call aitamd_gemm_noalloc_scratch_bytes() once per GPU at set-up, with
 * that GPU current - it returns the capacity and does the look-up - or make one call outside the capture first. */
AITAMD_API int aitamd_gemm_rcr_noalloc(int epilogue, int dtype, int algo,
                                       const void* a, const void* b, const void* bias,
                                       const void* d0, const void* d1, void* c,
                                       int64_t M, int64_t N, int64_t K,
                                       int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd, void* stream);
AITAMD_API int64_t aitamd_gemm_noalloc_scratch_bytes(void);

/* gemm_rcr[_bias...] whose [M, N] result is written through one of the reference's 5-D output permutations
 * into a contiguous buffer.  Epilogues AITAMD_EPI_NONE and AITAMD_EPI_BIAS only (the ones the permuting ops use);
 * g = (g1, g2, g3) is the op's `shape` attribute.
 *   AITAMD_PERMUTE_M2N3: result viewed as [M/g1, g1, g2, g3, N/(g2*g3)], written as dims (2, 0, 3, 1, 4), i.e.
 *     [g2, M/g1, g3, g1, N/(g2*g3)].  For a packed QKV projection with g = (seq_len, 3, heads) that is
 *     [3, batch, heads, seq_len, head_dim].
 *   AITAMD_PERMUTE_M3N2: result viewed as [M/(g1*g2), g1, g2, g3, N/g3], written as dims (2, 0, 3, 1, 4), i.e.
 *     [g2, M/(g1*g2), g3, g1, N/g3] (what the ROCm backend does for layout "20314" as well).
 * Replaces the GemmPermuteM2N3 / GemmPermute instances behind gemm_rcr_bias_permute_m2n3, gemm_rcr_permute_m2n3,
 * gemm_rcr_bias_permute_m3n2 and gemm_rcr_bias_permute
 * (python/aitemplate/backend/rocm/gemm/gemm_rcr_bias_permute_m2n3.py:59-75, permute_common.py:20-130). */
enum { AITAMD_PERMUTE_M2N3 = 1, AITAMD_PERMUTE_M3N2 = 2 };
AITAMD_API int aitamd_gemm_rcr_permute(int epilogue, int dtype, int algo,
                                       const void* a, const void* b, const void* bias, void* c,
                                       int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                       int layout, int64_t g1, int64_t g2, int64_t g3, void* stream);

/* C[b,m,n] = sum_k A[b,m,k] * B[b,n,k]; a batch stride of 0 broadcasts that
 * operand over the batch (python/aitemplate/compiler/ops/gemm_universal/bmm.py:72-90).
 * Replaces the generated bmm_rcr op function's CK call
 * (python/aitemplate/backend/rocm/gemm/bmm_common.py:72-105, bmm_rcr.py:27-182). */
AITAMD_API int aitamd_bmm_rcr(int dtype, int algo,
                              const void* a, const void* b, void* c,
                              int64_t batch, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb, int64_t ldc,
                              int64_t stride_a, int64_t stride_b, int64_t stride_c,
                              void* stream);

/* Batched GEMM for the reference's other operand layouts; the result is row-major [B, M, N] in all of them.
 *   AITAMD_LAYOUT_RCR: A [B, M, K], B [B, N, K]     AITAMD_LAYOUT_RRR: A [B, M, K], B [B, K, N]
 *   AITAMD_LAYOUT_CCR: A [B, K, M], B [B, N, K]     AITAMD_LAYOUT_CRR: A [B, K, M], B [B, K, N]
 * lda / ldb are the row pitches of the matrices as stored, the strides are per batch (0 broadcasts).  d1 = 0
 * stores plainly with ldc / stride_c; d1 > 0 stores [B/d1, M, d1, N] as aitamd_bmm_rcr_permute does (ldc and
 * stride_c are ignored).  A transposed operand whose row pitch is not a multiple of 8 elements is served by the
 * instance with element-wide loads only.
 * Replaces the DeviceBatchedGemmXdl / DeviceGemm instances behind bmm_rrr, bmm_ccr, bmm_crr, gemm_rrr and
 * bmm_rrr_permute (python/aitemplate/backend/rocm/gemm/bmm_rrr.py, bmm_ccr.py, bmm_crr.py, gemm_rrr.py,
 * bmm_rrr_permute.py; layouts in backend/rocm/gemm/layout.py). */
enum { AITAMD_LAYOUT_RCR = 0, AITAMD_LAYOUT_RRR = 1, AITAMD_LAYOUT_CCR = 2, AITAMD_LAYOUT_CRR = 3 };
AITAMD_API int aitamd_bmm(int layout, int dtype, int algo, const void* a, const void* b, void* c,
                          int64_t batch, int64_t M, int64_t N, int64_t K,
                          int64_t lda, int64_t ldb, int64_t ldc,
                          int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t d1, void* stream);
/* C[b] = A[b] x B[b] + D0[b] (epilogue AITAMD_EPI_ADD) in any of the four operand layouts; D0 is row-major
 * [B, M, N] with row pitch ldd and batch stride stride_d (0 broadcasts one [M, N] residual).
 * Replaces the instances behind bmm_rrr_add, bmm_ccr_add, bmm_crr_add
 * (python/aitemplate/backend/rocm/gemm/bmm_rrr_add.py, bmm_ccr_add.py, bmm_crr_add.py). */
AITAMD_API int aitamd_bmm_add(int layout, int dtype, int algo, const void* a, const void* b, const void* d0, void* c,
                              int64_t batch, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd,
                              int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t stride_d, void* stream);
/* aitamd_gemm_rcr_permute with the operand layout as a parameter: AITAMD_LAYOUT_RCR with epilogues none / bias, or
 * AITAMD_LAYOUT_RRR (B is [K, N]) with the bias epilogue, which is gemm_rrr_bias_permute
 * (python/aitemplate/backend/rocm/gemm/gemm_rrr_bias_permute.py:40-110). */
AITAMD_API int aitamd_gemm_permute(int operands, int epilogue, int dtype, int algo,
                                   const void* a, const void* b, const void* bias, void* c,
                                   int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                   int layout, int64_t g1, int64_t g2, int64_t g3, void* stream);
/* aitamd_gemm_algo_supported / aitamd_gemm_heuristic_algo for a given operand layout (same arguments otherwise) */
AITAMD_API int aitamd_gemm_algo_supported_layout(int epilogue, int dtype, int layout, int algo,
                                                 int64_t M, int64_t N, int64_t K,
                                                 int64_t lda, int64_t ldb, int align_bytes);
AITAMD_API int aitamd_gemm_heuristic_algo_layout(int epilogue, int dtype, int layout, int64_t batch,
                                                 int64_t M, int64_t N, int64_t K,
                                                 int64_t lda, int64_t ldb, int align_bytes);

/* bmm_rcr whose [B, M, N] result, viewed as [B/d1, d1, M, N], is written as [B/d1, M, d1, N] (the reference's
 * "0213" permutation with shape = (d1,)): rows of one (batch, head) pair are d1*N elements apart.
 * Replaces the DeviceBatchedGemmEPermuteXdl instances behind bmm_rcr_permute
 * (python/aitemplate/backend/rocm/gemm/bmm_rcr_permute.py, bmm_permute_common.py:29-56). */
AITAMD_API int aitamd_bmm_rcr_permute(int dtype, int algo, const void* a, const void* b, void* c,
                                      int64_t batch, int64_t M, int64_t N, int64_t K,
                                      int64_t lda, int64_t ldb, int64_t stride_a, int64_t stride_b,
                                      int64_t d1, void* stream);

/* out[b / G, m, b % G, o] = sum_n softmax_n( scale * sum_k Q[b,m,k] K[b,n,k] ) V[b,n,o]
 * Q [B,M,K], K [B,N,K], V [B,N,O] contiguous; out [B/G, M, G, O] (the "0213"
 * permute of [B/G, G, M, O]); G = number of heads, B % G == 0.  `scale` is
 * rounded to the element type first, as the reference does; causal != 0 masks
 * keys n > m.  K and O up to 160; head dims that are not MFMA multiples are
 * padded on chip only.  Rows whose keys are all masked (N == 0) produce 0.
 * Replaces the generated bmm_softmax_bmm_permute op function's CK call
 * (python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:84-110,
 * frontend python/aitemplate/compiler/ops/gemm_universal/bmm_softmax_bmm_permute.py:30-194). */
AITAMD_API int aitamd_bmm_softmax_bmm_permute(int dtype,
                                              const void* q, const void* k, const void* v, void* out,
                                              int64_t B, int64_t M, int64_t N, int64_t K, int64_t O,
                                              int64_t G, float scale, int causal, void* stream);

/* mem_eff_attention: out[b, m, h, :] = sum_n softmax_n( scale * q[b,h,m,:] . k[b,h,n,:] ) v[b,h,n,:]
 * q [batch, heads, seq_q, head_dim], k [batch, heads, seq_kv, head_dim], v [batch, heads, seq_kv, head_dim_v]
 * contiguous; out [batch, seq_q, heads, head_dim_v].  The same kernel as aitamd_bmm_softmax_bmm_permute with
 * B = batch * heads and G = heads.  lengths_kv: null, or device memory with `batch` int32 entries: batch entry b
 * attends to its first lengths_kv[b] keys only (clamped to [0, seq_kv]; later rows of k and v are not read), the
 * key-padding mask of the reference's own test (tests/unittest/ops/test_attention.py:504-523, 593).  A batch entry
 * with no keys is written as zeros.  lengths_q: null, or the same form for query rows: rows m >= lengths_q[b] are
 * written as zeros and blocks of query rows that are all padding visit no keys (the reference leaves such rows
 * unspecified; its test blanks them on both sides, test_attention.py:661-664).
 * Replaces the op function that python/aitemplate/backend/rocm/attention/mem_eff_attention.py:305-365 renders
 * (frontend python/aitemplate/compiler/ops/attention/mem_eff_attention.py:49-263). */
AITAMD_API int aitamd_mem_eff_attention(int dtype,
                                        const void* q, const void* k, const void* v, void* out,
                                        int64_t batch, int64_t heads, int64_t seq_q, int64_t seq_kv,
                                        int64_t head_dim, int64_t head_dim_v, float scale, int causal,
                                        const int32_t* lengths_kv, const int32_t* lengths_q, void* stream);

/* Test and measurement knob of the two attention entry points above: force one of the kernel's four work
 * decompositions wherever the shape allows it (0: four waves per 128 query rows; 1: eight waves per 256 rows;
 * 2: as 1 with two wave groups on alternate key tiles; 3: as 0 with two wave groups), or -1 (the default) to let
 * the launcher choose from the shape.  Process-wide; the results are the same in every variant up to rounding.
 * The environment variable AITAMD_ATTN_MODE sets the initial value and is read once.  No counterpart in the
 * reference (CK instances are chosen by its profiler only). */
AITAMD_API int aitamd_attention_set_variant(int variant);

/* Stand-alone element-wise op: out[i] = f(a[i], b[i % b_period]) over `numel` flattened elements (f(b, a) with
 * swap_operands).  `func` is the reference's FuncEnum value (python/aitemplate/compiler/ops/common/epilogue.py:34-70):
 * binary ADD 1, SUB 2, MUL 3, DIV 4, MAX 13, MIN 14 (NaN if either operand is), LRELU 16 (b: negative slope), POW 22;
 * unary TANH 5, COS 6, SIN 7, SIGN 8, ABS 9, LOGE 10, EXP 11, SQRT 12, SIGMOID 15, RELU 18, SILU 21, GELU 23 (erf form),
 * FASTGELU 24 (tanh form), SOFTSIGN 27, FLOOR 30, LOG1P 31, RECIPROCAL 32.  Arithmetic in fp32, one rounding.  b: a tensor of b_period elements that tiles the output (same shape: b_period =
 * numel; an operand that broadcasts over leading dims: the product of its dims; a one-element tensor: 1), or null with
 * the constant b_value; ignored by the unary functions.  Replaces the single-op case of the kernels the reference
 * generates in python/aitemplate/backend/common/elementwise_common.py (ROCm entry:
 * python/aitemplate/backend/rocm/elementwise/fused_elementwise.py:27-65). */
AITAMD_API int aitamd_elementwise(int func, int dtype, const void* a, const void* b, void* out, int64_t numel,
                                  int64_t b_period, float b_value, int swap_operands, void* stream);
/* 1 when aitamd_elementwise implements FuncEnum value `func` (instance filtering at compile time). */
AITAMD_API int aitamd_elementwise_supported(int func);

/* Strided row copy: `rows` rows of `row_bytes` bytes from src (rows src_pitch_bytes apart) to dst (rows
 * dst_pitch_bytes apart); the two ranges must not overlap.  What a split or a concatenate becomes when no GEMM-family
 * op can take the piece as a view (a piece [..., n_i, inner] of x[..., n, inner] is prod(leading dims) rows of
 * n_i * inner elements out of rows n * inner elements apart).  Replaces the kernels the reference generates in
 * python/aitemplate/backend/common/split_common.py:479-530 and concatenate_common.py:661-800 (ROCm entries:
 * python/aitemplate/backend/rocm/tensor/split.py, concatenate.py). */
AITAMD_API int aitamd_copy_rows(const void* src, void* dst, int64_t rows, int64_t row_bytes, int64_t src_pitch_bytes,
                                int64_t dst_pitch_bytes, void* stream);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* AITEMPLATE_AMD_KERNELS_H_ */
