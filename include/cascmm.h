/*
 * cascmm.h -- C ABI of the MI355X (gfx950) cascaded low-precision matmul library.
 *
 * The library computes  C[M,N] = A[M,K] . B[K,N] (+ bias[N])  where the fp32 operands are
 * split on the fly into `terms` low-precision terms (bf16 / fp16 / fp8-e4m3), the kept
 * partial products run on MFMA and are accumulated in fp32.
 *
 * It is the device side of the Python operator
 *     cascaded_lowp_matmul(a, b, *, out=None, dump_ptx=False)
 * of the reference (basedxl/triton/cascaded_lowp_matmul.py:139-173): the host wrapper
 * does the shape checks / batch flattening / output allocation of :146-161,173 and calls
 * cascmm_gemm() where the reference launches its Triton kernel (:163-168).
 *
 * Conventions
 *  - every pointer named A, B, C, bias, x, out, workspace, tensor_exps is a DEVICE pointer;
 *  - the library never allocates or frees device memory and never synchronises the host;
 *  - all work is enqueued on `stream` (a hipStream_t passed as void*, NULL = default stream);
 *  - every function returns 0 on success or a negative cascmm_status; nothing throws.
 *  - row-major operands, leading dimensions in ELEMENTS.
 */
#ifndef CASCMM_H
#define CASCMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CASCMM_VERSION 100 /* major*10000 + minor*100 + patch */

/* element type of A, B, C and bias as stored in memory (C has the type of A, like
 * `torch.empty((M, N), dtype=a.dtype)` at cascaded_lowp_matmul.py:161).  The cascade kernels
 * take fp32.  fp16 (bf16) tensors multiplied as ONE fp16 (bf16) term have fast kernels too:
 * through cascmm_gemm_prepared, or through cascmm_gemm when K % 64 == 0, the rows of A are
 * 16-byte aligned and the workspace holds cascmm_workspace_bytes(...) (B is re-laid there
 * first).  Other combinations with 16-bit tensors run on bounds-checked kernels (bf16 or
 * fp16 terms, 1 or 2 of them, tri). */
enum cascmm_dtype { CASCMM_DT_F32 = 0, CASCMM_DT_F16 = 1, CASCMM_DT_BF16 = 2 };

/* low-precision format of the cascade terms */
enum cascmm_fmt { CASCMM_FMT_BF16 = 0, CASCMM_FMT_FP16 = 1, CASCMM_FMT_FP8 = 2 };

/* which partial products A_i.B_j are summed: TRI keeps i + j <= terms - 1, FULL keeps all */
enum cascmm_products { CASCMM_PROD_TRI = 0, CASCMM_PROD_FULL = 1 };

enum cascmm_status {
  CASCMM_OK = 0,
  CASCMM_ERR_NULL_POINTER = -1,
  CASCMM_ERR_BAD_SHAPE = -2,     /* negative size, leading dimension smaller than the row */
  CASCMM_ERR_BAD_DTYPE = -3,
  CASCMM_ERR_BAD_FORMAT = -4,    /* unknown fmt / unsupported (fmt, terms, products) */
  CASCMM_ERR_WORKSPACE = -5,     /* workspace missing or smaller than cascmm_workspace_bytes */
  CASCMM_ERR_ALIGNMENT = -6,     /* pointer not aligned to its element size */
  CASCMM_ERR_LAUNCH = -7,        /* the HIP runtime refused the launch */
  CASCMM_ERR_BAD_VARIANT = -8,   /* forced kernel variant unknown or unable to run this problem */
  CASCMM_ERR_TOO_LARGE = -9,     /* a dimension exceeds 2^31 - 1 or a product overflows */
  CASCMM_ERR_SCRATCH_LIMIT = -10 /* cascmm_gemm_noalloc: the problem needs more than CASCMM_NOALLOC_SCRATCH_BYTES */
};

/*
 * The matmul.  Replaces the `_matmul_kernel[grid](...)` launch of
 * basedxl/triton/cascaded_lowp_matmul.py:166-168 and, when `bias` is non-NULL, the
 * separate `x + bias` of basedxl/modules/lowp_linear.py:17-19.
 *
 *   A [M,K] lda>=K, B [K,N] ldb>=N, C [M,N] ldc>=N, bias [N] or NULL; all of `dtype`.
 *   fmt/terms/products: supported combinations are
 *       bf16: terms 1..3;  fp16: terms 1..3;  fp8: terms 1..3.
 *   tensor_exps: fp8 only -- device pointer to two int32 {e_A, e_B}: the operands are
 *       scaled by 2^e before rounding (see cascmm_tensor_exp); NULL means {0, 0}.  (Grouped
 *       launch: 2 * count values, problem i at [2i], [2i + 1].)
 *   workspace: used only when cascmm_workspace_bytes(...) > 0 (K split for problems with too
 *       few tiles to occupy the chip: fp32 partial results); 16-byte aligned, contents need no
 *       initialisation.  When it is NULL or too small, a kernel that needs none is selected.
 *   M, N or K equal to 0 is valid (K == 0 writes bias or zeros).
 */
int cascmm_gemm(const void* A, const void* B, void* C, const void* bias,
                int64_t M, int64_t N, int64_t K,
                int64_t lda, int64_t ldb, int64_t ldc,
                int dtype, int fmt, int terms, int products,
                const int32_t* tensor_exps,
                void* workspace, size_t workspace_bytes, void* stream);

/* Same with the kernel variant forced (index into the variant table, see
 * cascmm_variant_count / cascmm_variant_name); variant < 0 selects automatically.  A forced
 * LDS-tiled kernel runs without K split unless `variant` carries a split count S in 2..4 as
 * index | S << 16 (needs S * M * N * 4 bytes of workspace and S dividing the kernel's K steps).
 * No counterpart in the reference, whose Triton autotuner picks among its two configs
 * (cascaded_lowp_matmul.py:29-51); used by the tests and the tuning sweep. */
int cascmm_gemm_variant(const void* A, const void* B, void* C, const void* bias,
                        int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc,
                        int dtype, int fmt, int terms, int products,
                        const int32_t* tensor_exps,
                        void* workspace, size_t workspace_bytes, void* stream, int variant);

/*
 * cascmm_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments
 * and results as cascmm_gemm called with a workspace of cascmm_workspace_bytes(...) bytes, but the
 * K-split partial results live in a buffer built into the library (CASCMM_NOALLOC_SCRATCH_BYTES of
 * device memory per GPU, held until the process ends); the call allocates and frees nothing.
 * A problem for which the kernel cascmm_gemm would pick (given an unlimited workspace) needs more
 * partial results than that returns CASCMM_ERR_SCRATCH_LIMIT (nothing is launched).  All calls on one GPU share the buffer: calls that may overlap in time on
 * one GPU (different streams, or graphs replayed concurrently) race on it and must be ordered by the
 * caller.  Nothing in the buffer needs initialisation between calls.
 * The device address of the buffer is looked up once per GPU, on the first call there or by cascmm_init;
 * a caller that records its first call on a GPU into a graph calls cascmm_init() before the capture
 * (with that GPU current), so that the lookup is not part of it.
 */
#define CASCMM_NOALLOC_SCRATCH_BYTES (8u << 20)
/* Optional set-up for the current GPU (no counterpart in the reference): resolves what the library
 * otherwise resolves on first use there -- today the address of cascmm_gemm_noalloc's built-in buffer.
 * Allocates nothing, launches nothing; CASCMM_ERR_LAUNCH when no GPU is current. */
int cascmm_init(void);
int cascmm_gemm_noalloc(const void* A, const void* B, void* C, const void* bias,
                        int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc,
                        int dtype, int fmt, int terms, int products,
                        const int32_t* tensor_exps, void* stream);

/* `count` (1..8) independent GEMMs of one shape, layout and cascade in ONE launch: problem i
 * computes C[i] = A[i] . B[i] (+ bias[i]); A, B, C, bias are HOST arrays of device pointers
 * (bias may be NULL, or hold NULL entries).  Pointers may repeat (the same activations times
 * several weights).  The kernels are persistent, so the launch gap and the cold first loads of
 * every GEMM after the first disappear.  Counterpart in the reference: the fused to_k/to_v
 * Linear of basedxl/modules/attn.py:23-39, which gets the same effect by concatenating the
 * weights; here the weights stay separate tensors.  fp16 / bf16 tensors as one term of their
 * own format take their fast path when the workspace holds count * cascmm_workspace_bytes(...)
 * (every distinct B[i] is re-laid there). */
int cascmm_gemm_grouped(int count, const void* const* A, const void* const* B, void* const* C,
                        const void* const* bias,
                        int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc,
                        int dtype, int fmt, int terms, int products,
                        const int32_t* tensor_exps,
                        void* workspace, size_t workspace_bytes, void* stream, int variant);

/*
 * Prepared weights.  A Linear layer's weight is constant, so its split can be done once: the
 * counterpart of the one-time `W.T.contiguous().clone()` of basedxl/modules/lowp_linear.py:12.
 * cascmm_prepare_weight writes B[K,N] (leading dimension ldb, element type `dtype`) as MFMA
 * operand slots -- 16 bytes = 8 consecutive k of one column of one plane, [plane][ceil(K/8)][N];
 * planes = terms (bf16, fp16) or ceil(terms/2) (fp8) -- into `out` (16-byte aligned, at least
 * cascmm_prepared_bytes(K, N, fmt, terms) bytes, allocated by the caller).  fp8: *tensor_exp
 * (device int32, NULL = 0) is the scale exponent applied before the split; pass the same value
 * as e_B in tensor_exps of the GEMM.
 * cascmm_gemm_prepared runs `count` (1..8) GEMMs C[i] = A[i] . B[i] (+ bias[i]) of one shape whose
 * right operands are prepared buffers; arguments as cascmm_gemm_grouped, without ldb (the
 * workspace, which may be NULL, is used for the K split of under-filled single launches and
 * holds cascmm_workspace_bytes(...)).  Only the fast kernels exist for it: A must be fp32 with 16-byte aligned rows
 * (CASCMM_ERR_ALIGNMENT otherwise), K a multiple of 32 or 64 depending on the kernel
 * (CASCMM_ERR_BAD_FORMAT when no kernel fits), the prepared buffer below 2 GiB
 * (CASCMM_ERR_TOO_LARGE).  The results equal cascmm_gemm's bit for bit when the same kernel
 * tile is used (same split, same order of accumulation).
 */
size_t cascmm_prepared_bytes(int64_t K, int64_t N, int fmt, int terms);
int cascmm_prepare_weight(const void* B, int64_t K, int64_t N, int64_t ldb, int dtype, int fmt, int terms,
                          const int32_t* tensor_exp, void* out, size_t out_bytes, void* stream);
int cascmm_gemm_prepared(int count, const void* const* A, const void* const* Bprep, void* const* C,
                         const void* const* bias,
                         int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                         int dtype, int fmt, int terms, int products,
                         const int32_t* tensor_exps,
                         void* workspace, size_t workspace_bytes, void* stream, int variant);
int cascmm_select_variant_prepared(int count, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                                   int dtype, int fmt, int terms, int products);

/*
 * Gated projection (GEGLU) in one kernel.  The feed-forward block of the UNet's transformer layers
 * (diffusers' `GEGLU`, a module of the third-party model the reference patches at
 * basedxl/unet.py:81-87: `proj` is one of the nn.Linear layers it routes) computes
 *     h = x . W + b   (N = 2 * Nh columns);   y = h[:, :Nh] * gelu(h[:, Nh:])   (exact, erf form)
 * and writes h, reads it back and writes y.  Here the product and the gate share one kernel:
 * cascmm_prepare_weight_glu prepares W [K, N] like cascmm_prepare_weight but with the columns
 * reordered so that 32 value columns and their 32 gate columns alternate (N % 64 == 0), and
 * cascmm_gemm_prepared_glu, with the arguments of cascmm_gemm_prepared, writes
 *     C[m][j] = (h[m][j] + bias[j]) * gelu(h[m][Nh + j] + bias[Nh + j]),   C [M, Nh], ldc >= Nh,
 * with `bias` (N entries, or NULL) in the ORIGINAL column order; N is the width of the projection
 * (2 * Nh).  Element types as cascmm_gemm_prepared (fp32, or fp16 / bf16 tensors as one term of
 * their own format; the gate is computed in fp32 on the unrounded accumulators and the result
 * rounded once).  CASCMM_ERR_BAD_FORMAT when no kernel with the gated store fits.
 */
int cascmm_prepare_weight_glu(const void* B, int64_t K, int64_t N, int64_t ldb, int dtype, int fmt, int terms,
                              const int32_t* tensor_exp, void* out, size_t out_bytes, void* stream);
int cascmm_gemm_prepared_glu(int count, const void* const* A, const void* const* Bprep, void* const* C,
                             const void* const* bias,
                             int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                             int dtype, int fmt, int terms, int products,
                             const int32_t* tensor_exps, void* stream, int variant);
/* The same gated product on the RAW weight W [K, N] (row-major, ldb; value columns in the first half,
 * gate columns in the second, as the module holds it): no prepared copy of the weight is needed.  Only
 * the large-tile kernel of the two-term bf16 cascade has this store (fp32 tensors, M % 256 == 0,
 * N % 320 == 0, K % 32 == 0, rows 16-byte aligned): cascmm_select_variant_glu returns its index, or
 * CASCMM_ERR_BAD_FORMAT when it does not take the problem or when the library's cost estimates put the
 * best plain kernel plus a separate gate pass ahead (few tiles on many CUs); the caller then runs
 * cascmm_gemm and applies the gate itself.  cascmm_gemm_glu launches it wherever it takes the problem
 * (variant < 0: automatic).  `bias` as above.  Same place in the reference
 * as above. */
int cascmm_select_variant_glu(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                              int dtype, int fmt, int terms, int products);
int cascmm_gemm_glu(const void* A, const void* B, void* C, const void* bias,
                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                    int dtype, int fmt, int terms, int products, void* stream, int variant);

/*
 * Chained feed-forward: the second GEMM with BOTH operands already split.  The reference runs the two
 * Linear layers of a feed-forward block as two independent calls of its operator
 * (basedxl/modules/lowp_linear.py:15-20 on `ff.net.0.proj` and on `ff.net.2`, installed at
 * basedxl/unet.py:81-87); the result of the first is written as fp32, read back, cast again.  Here the
 * first GEMM's gated store can write its result as the operand slots of the second (two bf16 terms,
 * fp32 tensors), and the second multiplies slots by slots:
 *   left slots  [2 terms][K/8][M] x 16 bytes, K % 16 == 0.  Slot (term, kg, m) holds, with kg = 2 t + g,
 *               A[m][16 t + 4 g + 0..3] at positions 0..3 and A[m][16 t + 8 + 4 g + 0..3] at 4..7 (the
 *               order in which the gated store holds its results in registers);
 *   weight      cascmm_prepare_weight_chained: the layout of cascmm_prepare_weight for two bf16 terms
 *               with the same order of k inside every group of 16 (cascmm_prepared_bytes(K, N, bf16, 2)).
 * cascmm_prepare_left writes the left slots of any fp32 A [M, K] (lda % 4 == 0, 16-byte aligned) in a
 * pass of its own -- what the gated store does on the fly; cascmm_left_slots_bytes gives the size
 * (4 M K).  cascmm_gemm_chained computes C = A . B (+ bias) from the two slot buffers in one launch for
 * any M and N, K % 16 == 0, slot buffers below 2 GiB (cascmm_chained_supported says
 * whether a shape is taken); K is split over the waves of a workgroup, so no workspace is needed.
 * Same terms, same three products as cascmm_gemm with two bf16 terms; the order of summation over k
 * differs (four interleaved partial sums), as it does between any two kernel tiles.
 * cascmm_gemm_glu_chained is the first GEMM of such a block: cascmm_gemm_glu (b_prepared == 0: raw weight
 * W [K, N], ldb) or cascmm_gemm_prepared_glu (b_prepared != 0: B written by cascmm_prepare_weight_glu)
 * whose gated result y [M, N / 2] leaves as left slots at out_slots (cascmm_left_slots_bytes(M, N / 2)
 * bytes) instead of fp32.  Only the large-tile kernel has this store (M % 256 == 0, N % 320 == 0,
 * K % 32 == 0, rows of A 16-byte aligned; CASCMM_ERR_BAD_FORMAT otherwise).  The slots hold exactly the
 * split of the fp32 values cascmm_gemm_glu would have written.
 */
size_t cascmm_left_slots_bytes(int64_t M, int64_t K);
int cascmm_gemm_glu_chained(const void* A, const void* B, int b_prepared, void* out_slots, size_t out_bytes,
                            const void* bias, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, void* stream);
int cascmm_prepare_left(const void* A, int64_t M, int64_t K, int64_t lda, void* out, size_t out_bytes, void* stream);
int cascmm_prepare_weight_chained(const void* B, int64_t K, int64_t N, int64_t ldb, void* out, size_t out_bytes,
                                  void* stream);
int cascmm_chained_supported(int64_t M, int64_t N, int64_t K);
int cascmm_gemm_chained(const void* Aslots, const void* Bslots, void* C, const void* bias,
                        int64_t M, int64_t N, int64_t K, int64_t ldc, void* stream);

/* Bytes of device workspace cascmm_gemm can use for this problem (0 for most shapes).
 * Counterpart of nothing in the reference (its small-M shapes fall back to torch.matmul,
 * cascaded_lowp_matmul.py:155-156); the caller allocates, as it allocates `out` (:161). */
size_t cascmm_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype, int fmt, int terms,
                              int products);

/* Variant the automatic selection would run for this problem (index), or a negative status. */
int cascmm_select_variant(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                          int dtype, int fmt, int terms, int products);
/* Same for a grouped launch of `count` problems (the choice depends on how many tiles the
 * group has in total). */
int cascmm_select_variant_grouped(int count, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                  int64_t ldc, int dtype, int fmt, int terms, int products);
int cascmm_variant_count(void);
/* Static string: the device function name of the variant's kernel is a template
 * instantiation whose text contains this name (for filtering rocprof output), or NULL. */
const char* cascmm_variant_name(int variant);
/* The symbol (mangled device function name) of the GEMM kernel that the variant launches, as the
 * code object, a profiler's kernel trace and an assembly listing of the library's sources spell it;
 * static string, NULL for an index outside the table.  Works without a GPU.  Stands where the
 * reference reads its compiled kernel back from the launch (`kernel.asm["ptx"]`,
 * basedxl/triton/cascaded_lowp_matmul.py:163-171): the wrapper's `dump_ptx` looks this symbol up. */
const char* cascmm_variant_kernel(int variant);

/* fp8 tensor scale: writes to *exp_out (device int32) the exponent e with
 * max|x| * 2^e in (224, 448] (0 for an all-zero tensor).  x is [rows, cols] with leading
 * dimension ld.  *exp_out is overwritten; the call is stream-ordered. */
int cascmm_tensor_exp(const void* x, int64_t rows, int64_t cols, int64_t ld, int dtype,
                      int32_t* exp_out, void* stream);

/* The same search in one kernel launch, for the per-call scale of the activations in front of a
 * layer whose weight scale is kept (the counterpart of a layer's one-time weight preparation,
 * basedxl/modules/lowp_linear.py:12): writes exps_out[0] = e of x and, when second_exp is non-NULL,
 * exps_out[1] = *second_exp, i.e. the {e_A, e_B} pair cascmm_gemm takes.  scratch: two device int32
 * that are zero before the first call; every call leaves them zero again.  Calls that share a
 * scratch must be ordered (one stream). */
int cascmm_tensor_exps(const void* x, int64_t rows, int64_t cols, int64_t ld, int dtype,
                       const int32_t* second_exp, int32_t* exps_out, int32_t* scratch, void* stream);

/* A three-term (or any) fp8 GEMM on fp32 tensors that finds the scale of its left operand itself:
 * the same result, bit for bit, as cascmm_tensor_exps(A, ..., b_exp, exps_out, scratch) followed by
 * cascmm_gemm (b_prepared == 0) or cascmm_gemm_prepared with count 1 (b_prepared != 0: B is a buffer
 * written by cascmm_prepare_weight, ldb is ignored) with tensor_exps = exps_out, for the case every
 * Linear layer of a model is in: activations whose scale changes from call to call times a weight
 * whose scale e_B = *b_exp is kept (b_exp NULL: 0), the counterpart of the per-call cast of the
 * activations at basedxl/triton/cascaded_lowp_matmul.py:101-103 next to the one-time weight
 * preparation of basedxl/modules/lowp_linear.py:12.  exps_out (two device int32) receives
 * {e_A, e_B}.  When the kernel that runs splits A in a pass of its own (the fp8-rate kernel:
 * three terms, K a multiple of 64), the search costs no reduction pass: a first kernel leaves
 * per-workgroup maxima in the workspace and the split reduces them.  Otherwise the function makes
 * exactly the two calls named above.  scratch: as for cascmm_tensor_exps.  workspace: as for
 * cascmm_gemm (cascmm_workspace_bytes covers it). */
int cascmm_gemm_fp8_autoscale(const void* A, const void* B, int b_prepared, void* C, const void* bias,
                              int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                              int terms, int products, const int32_t* b_exp, int32_t* exps_out,
                              int32_t* scratch, void* workspace, size_t workspace_bytes, void* stream);

/* The operand split alone (a test hook for parity of the split with the CPU oracle):
 * out is fp32 [terms][n]; term i holds lowp(r_i * 2^(tensor_exp + shift*i)) upcast to fp32
 * with r_0 = x, r_{i+1} = r_i - t_i / 2^(tensor_exp + shift*i); shift = 0 / 11 / 4 for
 * bf16 / fp16 / fp8.  x is `n` contiguous elements of `dtype`. */
int cascmm_split_terms(const void* x, float* out, int64_t n, int dtype, int fmt, int terms,
                       int tensor_exp, void* stream);

/* Measurement hooks (no counterpart in the reference, whose self-benchmark only times its kernel,
 * basedxl/triton/cascaded_lowp_matmul.py:204-242): what the GPU at hand sustains on the two resources a
 * roofline prices the cascade against.
 * cascmm_probe_mfma: `workgroups` x 4 waves each issue `iters` x 4 independent v_mfma_f32_32x32x16_bf16
 * on registers only (131072 flop per wave and iteration); out: workgroups x 256 floats of device memory.
 * cascmm_probe_stream: one pass over `bytes` (a multiple of 16) of device memory at src with
 * `workgroups` x 256 threads, 16 bytes per thread and step: copied to dst, or, with dst NULL, only read
 * (sums: workgroups x 256 floats).  Timing is the caller's (events on `stream`). */
int cascmm_probe_mfma(int workgroups, int iters, float* out, size_t out_bytes, void* stream);
int cascmm_probe_stream(const void* src, void* dst, size_t bytes, int workgroups, float* sums, size_t sums_bytes,
                        void* stream);

/* Consistency of the library's own tables (no counterpart in the reference): the number of entries of
 * the measured-cost table that do not name exactly one compiled kernel variant, plus the number of
 * variant names that occur twice; 0 for a sound build.  (A cost entry whose kernel was renamed would
 * silently leave that kernel to the analytic cost estimate.)  Host only, launches nothing. */
int cascmm_selftest(void);

const char* cascmm_strerror(int status);
int cascmm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* CASCMM_H */
