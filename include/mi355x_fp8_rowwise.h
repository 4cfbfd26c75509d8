/*
 * mi355x_fp8_rowwise.h -- C ABI of the MI355X (gfx950 / CDNA4) row-wise scaled FP8 GEMM library.
 *
 * The library stands in for the native kernels the tritonbench operator
 * `fp8_gemm_rowwise` reaches through FBGEMM:
 *   - tritonbench/operators/fp8_gemm_rowwise/operator.py:187-199
 *       matmul_fp8_row(xq, wq, x_scale, w_scale, bias=...)          (fused bias)
 *   - tritonbench/operators/fp8_gemm_rowwise/operator.py:201-217
 *       torch.ops.fbgemm.f8f8bf16_rowwise(xq, wq, x_scale, w_scale) (baseline backend)
 *   - tritonbench/operators/fp8_gemm_rowwise/operator.py:136-145
 *       fp8_row_quantize(x)                                         (input preparation)
 * The reference defines no C interface of its own for this path (FBGEMM is reached
 * through torch.ops / Python); the entry points below are what a ctypes / pybind
 * binding on the reference side would call.
 *
 * Conventions
 *   - every data pointer is a DEVICE pointer on the current HIP device;
 *   - matrices are row-major, leading dimensions are in ELEMENTS;
 *   - fp8 is OCP e4m3fn (bias 7, max 448, no inf, NaN = 0x7f/0xff), one byte per element;
 *   - bf16 is the upper 16 bits of an IEEE binary32, rounded to nearest even;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - after mi355x_fp8_rowwise_init() on the device, calls only ENQUEUE work: no allocation, no
 *     host synchronisation, no attribute or query call, so they may be recorded into a HIP graph;
 *     state kept on the host is per device, written with atomics, and the same whichever thread
 *     wrote it (the library is re-entrant per stream);
 *   - the library borrows all pointers for the duration of the enqueued work and owns
 *     no device memory.
 *
 * Status codes: 0 ok, MI355X_FP8_EINVAL bad argument, MI355X_FP8_ENOTSUP shape or
 * alignment outside what the kernels handle, MI355X_FP8_ELAUNCH the HIP runtime
 * reported an error at launch. mi355x_fp8_rowwise_last_error() returns a
 * thread-local, NUL-terminated description of the last non-zero status.
 */
#ifndef MI355X_FP8_ROWWISE_H
#define MI355X_FP8_ROWWISE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355X_FP8_ABI_VERSION 2

#define MI355X_FP8_OK        0
#define MI355X_FP8_EINVAL   (-1)
#define MI355X_FP8_ENOTSUP  (-2)
#define MI355X_FP8_ELAUNCH  (-3)

/* Kernel families. AUTO lets the library pick from (M, N, K). */
#define MI355X_FP8_VARIANT_AUTO    0
#define MI355X_FP8_VARIANT_TILED   1  /* LDS-tiled persistent MFMA kernel (compute-bound shapes) */
#define MI355X_FP8_VARIANT_SKINNY  2  /* kernels that own all of K per workgroup and stream B (HBM-bound): M <= 64, \
                                         and M <= 256 where the narrow-tile form below fits */
#define MI355X_FP8_VARIANT_GENERIC 3  /* byte loads and f32 multiply-adds, no requirement on K, the leading dimensions or \
                                         the alignment of a and b: what AUTO runs for operands the two MFMA families   \
                                         cannot take (a few TFLOP/s) */

/*
 * The `variant` argument is a word: bits 0..7 hold the family above; for the tiled family
 * bits 8..15 may pin the tile configuration and bits 16..23 the split-K factor (0 in a
 * field = chosen by the library from the shape). Tile configurations: 0 = 256x256 tiles,
 * one workgroup per CU; 1 = 128x128 tiles, two workgroups per CU; 2 = 256x128 tiles
 * (256 rows of A, 128 rows of B), one workgroup per CU; 3 = 64x256, 4 = 128x256 and 5 = 192x256 tiles, one
 * workgroup per CU; 6 = 128x128 tiles with a deeper ring of loads in flight, one workgroup per CU
 * (chosen by the library only for launches of at most 256 work items and not split; pinned, it
 * runs any shape). Configurations 3 to 6 are not available in the grouped form. With a split-K factor
 * S > 1 every tile's K range is cut into S parts that run as separate work items; they
 * leave fp32 partial sums in the workspace (S*M*N*4 bytes) and a second kernel adds them
 * in a fixed order, so results do not depend on scheduling. A split factor larger than the
 * number of 128-byte K steps is reduced to it.
 */
/* Skinny family only: bit 8 pins the form with one 16-row tile of B per workgroup (the general
 * one; M <= 64). Without a pin, M <= 16 with N a multiple of 16 runs a form that keeps A on chip for
 * the whole launch (one 16-wave workgroup per CU): the pair form for N <= 8192 and any K <= 8192
 * (at most two tiles of B per CU, A parked in LDS, a tile's loads issued in one burst), the
 * persistent form for larger N with K one of 2048, 4096, 6144, 8192 (a run of tiles per CU, A in
 * registers, rolling prefetch; also M <= 32 at K = 4096) - unless the narrow-tile form below or the
 * general form is expected to be faster (the general form is, by a few per cent, at M <= 8 on most
 * shapes, and by more where K is far from a multiple of 2048); every other shape runs the general
 * form anyway. */
#define MI355X_FP8_SKINNY_ONE_TILE      (1 << 8)
/* Skinny family only: bit 9 pins the narrow-tile form (one workgroup per tile of 4 to 64 columns of C,
 * the columns dealt out evenly over the CUs, owns all of K). It takes M <= 64 and, in row blocks of 64 with 64-column tiles, 64 < M <= 256 when
 * ceil(M/64) * ceil(N/64, rounded up to a multiple of 8) <= 256 (one workgroup per CU); "not
 * supported" otherwise. Without a pin the family runs whichever of its forms is expected to be
 * fastest. */
#define MI355X_FP8_SKINNY_NARROW        (2 << 8)
/* Skinny family only: bit 10 pins the forms that keep A on chip (pair or persistent, whichever takes
 * the shape; "not supported" when neither does). */
#define MI355X_FP8_SKINNY_RESIDENT      (4 << 8)
#define MI355X_FP8_TILED_CONFIG(cfg)    ((((cfg) + 1) & 0xff) << 8)
#define MI355X_FP8_TILED_SPLITS(s)      (((s) & 0xff) << 16)
#define MI355X_FP8_NUM_TILE_CONFIGS     7
#define MI355X_FP8_NUM_GROUPED_TILE_CONFIGS 3

/* Source element types accepted by the quantiser. */
#define MI355X_FP8_SRC_F32   0
#define MI355X_FP8_SRC_BF16  1

int mi355x_fp8_rowwise_abi_version(void);

/*
 * Sets the CURRENT HIP device up for this library: checks that it is the part the kernels are
 * scheduled for (256 compute units), raises the dynamic-LDS limit of every kernel on it and looks
 * up the address of the built-in scratch buffer. It has no counterpart in the reference (PyTorch
 * initialises its own libraries on first use). These are the only HIP calls of the library that
 * are not enqueues; after a successful init on a device every entry point below only launches
 * kernels there, whatever shape, variant or instantiation a call is the first to use, so a call
 * may be recorded into a HIP graph without an eager call of the same kind before it. Idempotent
 * and thread-safe; call it once per device, outside graph capture. An entry point called on a
 * device that was never initialised does the same set-up on the way (not under capture, then).
 */
int mi355x_fp8_rowwise_init(void);

const char* mi355x_fp8_rowwise_last_error(void);

/* Variant AUTO would run for this shape with operands that meet the MFMA families' alignment
 * requirements (one of the MI355X_FP8_VARIANT_* values > 0; GENERIC when K is not a multiple
 * of 16), or a negative status when the shape is not supported. Lets tests pin the dispatch. */
int mi355x_fp8_rowwise_select_variant(int64_t M, int64_t N, int64_t K);

/* Bytes of device workspace `variant` needs for this shape (0 when none). Pure host
 * arithmetic: callable without a device. */
size_t mi355x_fp8_rowwise_workspace_bytes(int64_t M, int64_t N, int64_t K, int variant);

/*
 * C[M,N] (bf16) = bf16( (sum_k A[m,k] * B[n,k]) * a_scale[m] * b_scale[n] + bias[n] )
 *
 * Replaces the timed callables of operator.py:187-199 (bias fused before the single
 * bf16 rounding, as matmul_fp8_row does) and operator.py:201-217.
 *
 *   a        e4m3fn [M, K], row stride lda      b        e4m3fn [N, K], row stride ldb
 *   a_scale  f32 [M]                            b_scale  f32 [N]
 *   bias     bf16 [N] or NULL                   c        bf16 [M, N], row stride ldc
 *
 * Requirements: M, N, K >= 1. The MFMA families (TILED, SKINNY) want K, lda, ldb multiples of
 * 16, a and b 16-byte aligned and lda*256, ldb*256, ldc*512 below 2^31; pinned, they answer
 * ENOTSUP otherwise. AUTO sends operands that miss any of that to the GENERIC family, which
 * takes every K, leading dimension and alignment (M <= 4194240).
 * `workspace` (16-byte aligned) may be NULL when mi355x_fp8_rowwise_workspace_bytes() is 0.
 * A call whose variant leaves the split-K factor to the library and brings less workspace
 * than that runs the best plan that needs none (same results up to fp32 summation order);
 * a call that names a split factor > 1 without enough workspace fails with EINVAL.
 */
int mi355x_fp8_rowwise_gemm(const void* a, const void* b,
                            const float* a_scale, const float* b_scale,
                            const void* bias, void* c,
                            int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb, int64_t ldc,
                            void* workspace, size_t workspace_bytes,
                            int variant, void* stream);

/*
 * The same product with the output element type chosen by the caller: MI355X_FP8_OUT_BF16
 * (identical to mi355x_fp8_rowwise_gemm) or MI355X_FP8_OUT_F16 (IEEE binary16, round to
 * nearest even, values beyond 65504 become infinity; `bias` stays bf16). With constant scale
 * vectors this is the tensor-wise scaled product torch._scaled_mm(a, b, scale_a, scale_b,
 * out_dtype=float16) computes at tritonbench/operators/fp8_gemm/fp8_gemm.py:87-101.
 */
#define MI355X_FP8_OUT_BF16  0
#define MI355X_FP8_OUT_F16   1
int mi355x_fp8_rowwise_gemm_ex(const void* a, const void* b,
                               const float* a_scale, const float* b_scale,
                               const void* bias, void* c, int out_type,
                               int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb, int64_t ldc,
                               void* workspace, size_t workspace_bytes,
                               int variant, void* stream);

/*
 * mi355x_fp8_rowwise_gemm with clock readings, for benchmarks that want to tell a kernel's cycles
 * from the clock it ran at (the sustained clock under matrix load differs from box to box and
 * moves with power). It has no counterpart in the reference. Same operands and results as
 * mi355x_fp8_rowwise_gemm; in addition every workgroup g of a TILED-family launch writes four
 * 64-bit readings to stamps[4*g .. 4*g+3]: the shader clock counter at its first and after its
 * last instruction, and the constant 100 MHz counter at the same two points. Workgroups that had
 * no work, and launches of the other kernel families, write nothing: clear the buffer first and
 * skip groups whose first reading is zero. max(end) - min(start) over the groups is the launch in
 * shader cycles, the same difference of the 100 MHz readings its duration.
 * `stamps` is device memory of at least MI355X_FP8_STAMP_ENTRIES 64-bit entries, 8-byte aligned.
 */
#define MI355X_FP8_STAMP_ENTRIES 2048
int mi355x_fp8_rowwise_gemm_stamped(const void* a, const void* b,
                                    const float* a_scale, const float* b_scale,
                                    const void* bias, void* c,
                                    int64_t M, int64_t N, int64_t K,
                                    int64_t lda, int64_t ldb, int64_t ldc,
                                    void* workspace, size_t workspace_bytes,
                                    int variant, uint64_t* stamps, size_t stamp_entries, void* stream);

/*
 * mi355x_fp8_rowwise_gemm for callers that can neither allocate nor bring a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. It has no
 * counterpart in the reference (there every backend allocates through PyTorch). Same operands,
 * same plan and bit-identical bf16 results as mi355x_fp8_rowwise_gemm called with a workspace of
 * mi355x_fp8_rowwise_workspace_bytes(M, N, K, variant) bytes; the split-K partial sums go to a
 * buffer of MI355X_FP8_NOALLOC_SCRATCH_BYTES built into the library's device code (one copy per
 * GPU, held until the process ends). The call allocates and frees nothing.
 *
 * When the plan the library would choose needs more than the buffer holds, the call runs the
 * cheapest plan whose partial sums fit (as the workspace form does with a workspace that is too
 * small); only a call that names a split-K factor the buffer cannot hold is refused with
 * MI355X_FP8_ENOTSUP (use the workspace form for it). All calls on one GPU
 * share that GPU's buffer: calls that may overlap there (different streams, concurrently
 * replayed graphs) race on it and must be ordered by the caller. The buffer's address is looked
 * up by mi355x_fp8_rowwise_init() (or by the first call on a device that was not initialised:
 * make that call outside graph capture).
 */
#define MI355X_FP8_NOALLOC_SCRATCH_BYTES (64u << 20)
int mi355x_fp8_rowwise_gemm_noalloc(const void* a, const void* b,
                                    const float* a_scale, const float* b_scale,
                                    const void* bias, void* c,
                                    int64_t M, int64_t N, int64_t K,
                                    int64_t lda, int64_t ldb, int64_t ldc,
                                    int variant, void* stream);

/*
 * Grouped form (mixture-of-experts layers): A and C are G row blocks stacked in one
 * matrix, block g holding m_sizes[g] rows; block g is multiplied with rows
 * [g*N, (g+1)*N) of B:
 *
 *   C[r, n] = bf16( (sum_k A[r,k] * B[g*N + n, k]) * a_scale[r] * b_scale[g*N + n] )   r in block g
 *
 * Replaces the timed callables of
 * tritonbench/operators/fp8_gemm_rowwise_grouped/operator.py:400-424
 * (grouped_gemm_fp8_rowwise(group_A, group_B, m_sizes, a_scale, b_scale)) and :426-455.
 *
 *   a        e4m3fn [M, K]                      b        e4m3fn [G*N, K]
 *   a_scale  f32 [M]                            b_scale  f32 [G*N]
 *   m_sizes  int32 [G] in DEVICE memory         c        bf16 [M, N]
 *
 * The sizes are read by the kernel, not by the host (no synchronisation): negative sizes
 * count as 0 and rows past M are cut off, so the kernel never leaves A or C whatever the
 * sizes say. Rows of C past the sum of the sizes are left untouched. `tile_config` is -1
 * (the library picks from M / G and the tile counts) or one of the first three tile configurations listed above.
 * Same alignment requirements as mi355x_fp8_rowwise_gemm.
 */
int mi355x_fp8_rowwise_grouped_gemm(const void* a, const void* b,
                                    const float* a_scale, const float* b_scale,
                                    const int32_t* m_sizes, void* c,
                                    int64_t G, int64_t M, int64_t N, int64_t K,
                                    int64_t lda, int64_t ldb, int64_t ldc,
                                    int tile_config, void* stream);

/*
 * Block-scaled form: one scale per 128x128 block of A and of B,
 *
 *   C[m, n] = bf16( sum_kb (sum_{k in block kb} A[m,k] * B[n,k]) * a_scale[m/128][kb] * b_scale[n/128][kb] )
 *
 * Replaces the timed callables of tritonbench/operators/fp8_gemm_blockwise/operator.py:139-145
 * (matmul_fp8_block(xq, wq, x_scale, w_scale), f8f8bf16_blockwise(...)); the scale layout is
 * the one fp8_block_quantize returns there (:86-118).
 *
 *   a        e4m3fn [M, K]                        b        e4m3fn [N, K]
 *   a_scale  f32 [ceil(M/128)][ceil(K/128)]       b_scale  f32 [ceil(N/128)][ceil(K/128)]
 *   c        bf16 [M, N]
 *
 * Requirements as for the MFMA families of mi355x_fp8_rowwise_gemm, and K <= 32768.
 */
int mi355x_fp8_blockwise_gemm(const void* a, const void* b,
                              const float* a_scale, const float* b_scale, void* c,
                              int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb, int64_t ldc, void* stream);

/*
 * Block-wise e4m3fn quantiser, replacing fp8_block_quantize
 * (tritonbench/operators/fp8_gemm_blockwise/operator.py:86-118): one scale per 128 x 128 block,
 *
 *   amax[i,j]      = max |x| over block (i, j); elements past M or K count as zero
 *   scale[i,j]     = fl(fl(1 / max(amax[i,j], 1e-12)) * 448), +inf replaced by 1     (f32)
 *   xq[m,k]        = e4m3fn( x[m,k] * scale[m/128][k/128] )      (f32 product, round to nearest even)
 *   inv_scale[i,j] = 1 / scale[i,j]                                (f32)
 *
 * The lower bound 1e-12 is taken in the source type (for a bf16 source it is the bf16 nearest to
 * 1e-12), everything after it in f32, as eager PyTorch evaluates that function. A block holding a
 * NaN comes out as NaN codes with a NaN inverse scale; a block holding an infinity gets scale 0
 * and inverse scale +inf, its finite elements become zero and the infinities NaN.
 *
 *   x          [M, K] of `src_type`, row stride ldx (elements)     xq  e4m3fn [M, K], row stride ldq
 *   inv_scale  f32 [ceil(M/128)][ceil(K/128)], contiguous: what mi355x_fp8_blockwise_gemm takes
 *
 * At most 65535 block rows (M <= 8388480). Rows 16-byte aligned with K a whole number of 16-byte
 * source chunks take the one-pass form; anything else a slower element-wise one.
 */
int mi355x_fp8_blockwise_quantize(const void* x, int src_type,
                                  void* xq, float* inv_scale,
                                  int64_t M, int64_t K, int64_t ldx, int64_t ldq,
                                  void* stream);

/*
 * Row-wise e4m3fn quantiser, replacing fp8_row_quantize (operator.py:136-145):
 *   amax[r]      = max_k |x[r,k]|
 *   scale[r]     = fl(fl(1 / max(amax[r], 1e-12)) * 448)   (how PyTorch evaluates 448 / tensor)
 *   xq[r,k]      = e4m3fn( clamp(x[r,k] * scale[r], -448, 448) )     (round to nearest even)
 *   inv_scale[r] = 1 / scale[r]                                      (f32)
 * An f32 source is processed in f32. For a bf16 source every intermediate (scale, scaled
 * value, inverse scale) is rounded to bf16, which is how eager PyTorch evaluates the same
 * expression on a bf16 tensor. Non-finite input behaves as in that program: a row holding a NaN
 * comes out as NaN codes (0x7f / 0xff) with a NaN inverse scale; a row holding an infinity gets
 * scale 0 and inverse scale infinity, its finite elements become (signed) zero and the
 * infinities NaN.
 *
 *   x  [R, K] of `src_type`, row stride ldx (elements)     xq  e4m3fn [R, K], row stride ldq
 */
int mi355x_fp8_rowwise_quantize(const void* x, int src_type,
                                void* xq, float* inv_scale,
                                int64_t R, int64_t K, int64_t ldx, int64_t ldq,
                                void* stream);

/*
 * Fused front ends: normalise or gate the bf16 activation and quantise it row-wise in one pass
 * (the row is read once; only the e4m3fn codes and one f32 scale per row are written). They stand
 * in for rms_norm_fp8_rowwise_quant(x1, wd) and silu_mul_fp8_rowwise_quant(x1, x2) in the timed
 * callables of tritonbench/operators/fp8_fused_quant_gemm_rowwise/operator.py:86-94 and :111-119
 * (those kernels live outside the reference repository; the arithmetic below is this library's):
 *
 *   RMSNorm    y[r,k] = (x[r,k] * rstd[r]) * weight[k],   rstd[r] = 1 / sqrt(mean_k x[r,k]^2 + eps)
 *   SiLU-mul   y[r,k] = (x1[r,k] / (1 + exp(-x1[r,k]))) * x2[r,k]
 *
 * all in f32 on the bf16 inputs, followed by the row-wise quantiser's arithmetic on y as on an
 * f32 tensor (see mi355x_fp8_rowwise_quantize): xq, inv_scale feed mi355x_fp8_rowwise_gemm.
 *
 *   x, x1, x2  bf16 [R, K], row strides ldx / ldx1 / ldx2 (elements, multiples of 8)
 *   weight     bf16 [K]                    xq  e4m3fn [R, K], row stride ldq (multiple of 16)
 *   K a multiple of 8; x, x1, x2, weight and xq 16-byte aligned; eps >= 0.
 */
int mi355x_fp8_rmsnorm_rowwise_quantize(const void* x, const void* weight, float eps,
                                        void* xq, float* inv_scale,
                                        int64_t R, int64_t K, int64_t ldx, int64_t ldq,
                                        void* stream);
int mi355x_fp8_silu_mul_rowwise_quantize(const void* x1, const void* x2,
                                         void* xq, float* inv_scale,
                                         int64_t R, int64_t K, int64_t ldx1, int64_t ldx2, int64_t ldq,
                                         void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_FP8_ROWWISE_H */
