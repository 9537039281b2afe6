/*
 * mi_ns.h - C ABI of libmi_ns.so: bf16 SYRK, GEMM+AXPY, Frobenius normalisation and the
 * Newton-Schulz orthogonalisation driver for AMD MI355X (gfx950).
 *
 * The reference project (NVIDIA-NeMo/Emerging-Optimizers) is pure Python and has no FFI for this
 * path; each entry point below names the Python call site(s) of the reference that it stands
 * in for.  All pointers are DEVICE pointers owned by the caller.  Unless stated otherwise the
 * library allocates nothing, never synchronises the host, and enqueues its kernels on `stream`
 * (a hipStream_t passed as void*; NULL is the legacy default stream).
 *
 * Conventions
 *   - bf16 data are raw 16-bit words (bfloat16 bit patterns).
 *   - Leading dimensions (`*_ld`) and batch strides are in ELEMENTS, not bytes.
 *   - Every bf16 matrix must have its contiguous dimension a multiple of 8 elements, `*_ld` a
 *     multiple of 8 and a 16-byte aligned base pointer (16-byte vector loads).  Violations return
 *     MI_ERR_UNSUPPORTED_SHAPE; the host wrapper turns that into the exception the reference raises.
 *   - Return value: MI_OK (0) or a negative MI_ERR_* code; mi_last_error() gives the text.
 */
#ifndef MI_NS_H_
#define MI_NS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_OK 0
#define MI_ERR_BAD_ARG (-1)
#define MI_ERR_UNSUPPORTED_SHAPE (-2)
#define MI_ERR_LAUNCH (-3)
#define MI_ERR_WORKSPACE (-4)

/* Library version (major*10000 + minor*100 + patch). */
int mi_version(void);

/* Thread-local text of the last error returned on this host thread ("" if none). */
const char* mi_last_error(void);

/*
 * D[b] = alpha * A[b] * A[b]^T + beta * C[b]      (bf16 in, fp32 accumulate, bf16 out)
 *
 * Replaces: tsyrk_ex              emerging_optimizers/triton_kernels/syrk.py:335-408
 *           tsyrk_ex_small_matrix emerging_optimizers/triton_kernels/syrk.py:411-500
 *           batched_tsyrk_ex      emerging_optimizers/triton_kernels/batched_syrk.py:266-363
 * (one kernel family; batch == 1 is the 2-D case).
 *
 * A[b] is logically (n, k).  a_trans == 0: memory holds A[b] row-major, element (i, p) at
 * A + b*a_batch_stride + i*a_ld + p.  a_trans != 0: memory holds A[b]^T row-major, element (i, p)
 * at A + b*a_batch_stride + p*a_ld + i  (the reference's TRANS constexpr, syrk.py:200-207).
 * C[b] is (n, n), must be symmetric, may be NULL iff beta == 0.  D[b] is (n, n) row-major.
 * Only lower-triangle tiles are computed; every strictly-lower element is also stored at its
 * mirrored position unless skip_upper != 0, so D[b] is bitwise symmetric (syrk.py:221-224).
 * With skip_upper != 0 the diagonal and everything below it are stored; an element above the diagonal is either
 * left untouched or, where it shares a diagonal block with stored elements, holds its correct value.
 * D may alias neither A nor C.
 */
int mi_syrk_bf16(const void* A, int64_t batch, int64_t n, int64_t k,
                 int64_t a_batch_stride, int64_t a_ld, int a_trans,
                 const void* C, int64_t c_batch_stride, int64_t c_ld,
                 float alpha, float beta,
                 void* D, int64_t d_batch_stride, int64_t d_ld,
                 int skip_upper, void* stream);

/*
 * mi_syrk_bf16 with a caller-provided scratch buffer.  Same arguments, same result up to the order of the float32
 * additions along K.  The reference's kernels need no scratch (syrk.py:149-224, batched_syrk.py:158-234): they accept
 * that a tile count which is not a multiple of what the GPU holds leaves it partly idle in the last round; this
 * entry does not.  When the 256 x 256 tiles of the call would fill the rounds of the chip badly (batch 16 of
 * 2048 x 8192: 576 tiles on 256 CUs), the whole rounds run as usual, the K range of each left-over tile is shared
 * between several workgroups that park their float32 accumulators in `workspace`, and a last launch adds them, in a
 * fixed order, and writes those tiles (three launches on `stream`; no workgroup waits for another).
 * mi_syrk_workspace_bytes() gives the size needed (0: the call would not use one; any smaller buffer, or NULL,
 * selects the ordinary launch); the buffer must be 256-byte aligned and must not be shared by calls that overlap in
 * time.  The result is deterministic for a given (batch, n, k) and device, but which tiles are split depends on the
 * batch size, so a matrix computed inside a batch and alone may differ in the last bit of float32 accumulation.
 * A transposed operand (a_trans != 0: stored as K rows of N, syrk.py:200-207) is, for n >= 2048 and when the model
 * expects a gain, first copied into `workspace` in the K-contiguous layout (batch * n * k bf16, included in
 * mi_syrk_workspace_bytes) and then multiplied by the K-contiguous kernels, which have a 192 x 192 tile and the faster
 * K loop: 4096 x 14336 transposed runs in 1.15x the time of the K-contiguous call instead of 1.6x.  Bit-identical to
 * the direct route on integer-valued inputs; on general inputs the tile size, hence the order of the float32
 * additions, may differ.
 * Options (mi_set_option): "streamk" = 0 never splits, 1 splits whenever the shape qualifies (n a multiple of 256,
 * n >= 1024, k a multiple of 64, A not transposed or copied, skip_upper == 0) and tiles are left over after the whole
 * rounds; "syrk_transpose" = 0 never copies a transposed operand, 1 always does (n >= 1024, k a multiple of 64).
 * Every argument is checked before the first launch, the transposing copy included.
 */
size_t mi_syrk_workspace_bytes(int64_t batch, int64_t n, int64_t k, int a_trans);
int mi_syrk_bf16_ws(const void* A, int64_t batch, int64_t n, int64_t k,
                    int64_t a_batch_stride, int64_t a_ld, int a_trans,
                    const void* C, int64_t c_batch_stride, int64_t c_ld,
                    float alpha, float beta,
                    void* D, int64_t d_batch_stride, int64_t d_ld,
                    int skip_upper, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Xout[b] = beta * X[b] + alpha * (Bm[b] * X[b])      (bf16 in, fp32 accumulate)
 *
 * Replaces the third product of a Newton-Schulz step:
 *   torch.addmm(X, B, X, alpha=1.0, beta=a) / torch.addmm(X, A, X, alpha=b, beta=a)
 *     emerging_optimizers/orthogonalized_optimizers/muon_utils.py:374-377, 438-441
 *   torch.baddbmm twins   muon_utils.py:407-410, 472-475
 *
 * Bm[b] is (m, m) row-major (b_ld).  X[b] is logically (m, n).  x_trans == 0: X[b] and Xout[b]
 * are row-major (m, n), element (i, j) at i*ld + j.  x_trans != 0: memory holds X[b]^T and
 * Xout[b]^T row-major (n, m), element (i, j) at j*ld + i (the layout a tall parameter has after the
 * `.mT` view of muon_utils.py:207-208).  Bm need not be symmetric.
 * out_fp32 == 0: Xout is bf16.  out_fp32 != 0: Xout is float32 and is additionally multiplied by
 * out_scale (folds the final `.to(float32)` of muon_utils.py:269 and the Muon scale factor of
 * muon.py:131-132 into the epilogue).  Xout must not alias X or Bm.
 */
int mi_gemm_axpy_bf16(const void* Bm, int64_t b_batch_stride, int64_t b_ld,
                      const void* X, int64_t x_batch_stride, int64_t x_ld, int x_trans,
                      void* Xout, int64_t o_batch_stride, int64_t o_ld,
                      int64_t batch, int64_t m, int64_t n,
                      float alpha, float beta, int out_fp32, float out_scale, void* stream);

/*
 * Per-matrix Frobenius normalisation of a float32 batch, result cast to bf16 or kept float32:
 *   accumulate_fp64 == 0:  out[b] = x[b] / max(||x[b]||_F, eps)      (sum of squares in float32)
 *   accumulate_fp64 != 0:  out[b] = x[b] / float(||x[b]||_F in fp64) (no eps clamp)
 *
 * Replaces: torch.nn.functional.normalize(x, p=2, dim=(-2,-1), eps)   muon_utils.py:216
 *           the float64 vector_norm variant                           muon_utils.py:221-222
 *           X.to(torch.bfloat16)                                      muon_utils.py:262
 *
 * x[b] is `numel` contiguous float32 values at x + b*numel (any 2-D shape: the norm does not
 * depend on it).  out has the same element order.  numel must be a multiple of 8.
 * partials: float64 scratch of at least mi_frob_partials_len(batch, numel) elements.
 * dev_norm: optional (may be NULL) float32[batch] that receives the divisor actually used.
 */
int mi_frob_normalize(const float* x, int64_t batch, int64_t numel, float eps, int accumulate_fp64,
                      void* out, int out_bf16, double* partials, float* dev_norm, void* stream);
size_t mi_frob_partials_len(int64_t batch, int64_t numel);

/*
 * Whole Newton-Schulz orthogonalisation of a float32 batch in one call:
 *   normalise -> bf16 -> `steps` x { A = X X^T ; B = b A + c A^2 ; X = a X + B X } -> float32 * out_scale
 * (cubic step X = a X + b A X when c == 0), i.e. the "medium"-precision body of
 *   newton_schulz                     muon_utils.py:149-274
 *   (batched_)newton_schulz_step_tsyrk muon_utils.py:414-476
 * plus the scale multiplication of Muon's closure (muon.py:131-132).
 *
 * x, out: float32, batch matrices of (rows, cols) row-major contiguous.  The iteration always runs on
 * the orientation with the smaller leading dimension (muon_utils.py:205-208): a tall input is transposed
 * while it is cast to bf16 (into the workspace) and the float32 result is written transposed into `out` (by the
 * last product itself, or by a transposing pass over a staging copy in the workspace), so the MFMA kernels
 * always see the wide layout.  out must not alias x.
 * abc: HOST array of 3*steps floats (a, b, c per step, already expanded by the coefficient iterator).
 * steps == 0 returns the normalised input.  rows and cols must be multiples of 8.
 * workspace: device scratch of at least mi_newton_schulz_workspace_bytes(batch, rows, cols) bytes,
 * 256-byte aligned.
 *
 * Two things differ from a literal step-by-step execution, neither of which changes the function computed:
 *  - the input is cast to bf16 by the pass that sums its squares, and 1 / norm enters the first two products
 *    as a device scalar (norms outside [1e-10, 1e10] are divided out before the cast instead);
 *  - for matrices with at least 1024 rows and twice as many columns, consecutive quintic steps share one Gram
 *    matrix (all factors are polynomials of X X^T and commute): the first three when at least two more follow and
 *    (a_1 a_2)^2 <= 400, otherwise two at a time alternating with single steps, so 5 steps run as 3 + 2 or
 *    2 + 1 + 2; the same holds for 128/256-row matrices at least four times as wide.  The option "ns_pairs"
 *    (mi_set_option; read by the call and by mi_newton_schulz_workspace_bytes, so set it before both) overrides
 *    this: 0 = one step at a time, 1 = never three at once, 2 = pairs at every size.
 */
int mi_newton_schulz_bf16(const float* x, float* out, int64_t batch, int64_t rows, int64_t cols,
                          const float* abc, int steps, float eps, int accumulate_fp64,
                          float out_scale, void* workspace, size_t workspace_bytes, void* stream);
size_t mi_newton_schulz_workspace_bytes(int64_t batch, int64_t rows, int64_t cols);

/*
 * mi_newton_schulz_bf16 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same computation with the workspace taken from a buffer of
 * MI_NOALLOC_SCRATCH_BYTES that is part of the loaded library (each GPU the library runs on holds its own copy until
 * the process ends).  No counterpart in the reference.  The call allocates and frees nothing and clears nothing with
 * memset; calls whose mi_newton_schulz_workspace_bytes(batch, rows, cols) exceeds MI_NOALLOC_SCRATCH_BYTES return
 * MI_ERR_WORKSPACE (128 MiB serve e.g. one 2048 x 8192 matrix, 4 x 1024 x 4096, or 32 x 128 x 4096).  All calls on
 * one GPU share that GPU's buffer: calls that overlap in time on one GPU (different streams or host threads) race,
 * and the buffer keeps the previous call's contents (every value the kernels read from it is written earlier in the
 * same call).  The first call on a device looks up the buffer's address (hipGetSymbolAddress) and should be made
 * outside stream capture.  Results are bit-identical to mi_newton_schulz_bf16.
 */
#define MI_NOALLOC_SCRATCH_BYTES ((size_t)128 << 20)
int mi_newton_schulz_bf16_noalloc(const float* x, float* out, int64_t batch, int64_t rows, int64_t cols,
                                  const float* abc, int steps, float eps, int accumulate_fp64, float out_scale,
                                  void* stream);

/*
 * How mi_newton_schulz_bf16 would group the steps of a call with these arguments (pure host code, no GPU needed):
 * writes the group sizes (1 = an ordinary step, 2 or 3 = that many steps on one Gram matrix) to groups[0..] and
 * returns their number (which may exceed max_groups; only max_groups entries are written), or a negative error
 * code.  No counterpart in the reference, whose loop (muon_utils.py:264-272) always takes one step at a time.
 */
int mi_newton_schulz_schedule(int64_t batch, int64_t rows, int64_t cols, const float* abc, int steps, int* groups,
                              int max_groups);

/*
 * One fused Muon update of a float32 parameter batch: momentum, Nesterov direction, Newton-Schulz
 * orthogonalisation and the weight update, without materialising the direction or the update in HBM:
 *   momentum <- momentum + (1 - beta) (grad - momentum)                 buf.lerp_(grad, 1 - beta)
 *   d         = nesterov ? lerp(grad, momentum, beta) : momentum        grad.lerp(buf, beta)
 *   param    <- param_decay * param + update_scale * NewtonSchulz(d)
 *
 * Replaces, for the decoupled / independent / palm weight-decay methods (which only scale the parameter,
 * mixin.py:35-56), the body of the parameter loop of OrthogonalizedOptimizer.step
 *   emerging_optimizers/orthogonalized_optimizers/orthogonalized_optimizer.py:185-210
 * together with Muon's closure (muon.py:117-132): param_decay = 1 - wd*lr (decoupled), 1 - wd (independent),
 * 1 - wd*lr^2 (palm), 1 (no decay); update_scale = -lr * get_muon_scale_factor(...) * extra_scale_factor.
 * The momentum update, the sum of squares and the bf16 cast of d share one pass over grad and momentum, and the
 * last GEMM epilogue (transposed for a tall parameter) updates param in place.  param, grad, momentum: float32 (batch, rows, cols) row-major contiguous, distinct
 * buffers.  Other arguments and the workspace as for mi_newton_schulz_bf16; steps >= 1; param_decay != 0.
 */
int mi_muon_update_bf16(float* param, const float* grad, float* momentum, int64_t batch, int64_t rows, int64_t cols,
                        float beta, int nesterov, float param_decay, float update_scale,
                        const float* abc, int steps, float eps, int accumulate_fp64,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * Per-kernel timing of mi_newton_schulz_bf16 for benchmarks (no counterpart in the reference, whose
 * benchmark brackets whole calls with torch.cuda.profiler.start/stop, benchmarks/newton_schulz_benchmark.py:155-164).
 * Between mi_profile_begin() and mi_profile_end() every kernel group the driver enqueues is bracketed by a
 * HIP event pair on the caller's stream.  mi_profile_end() waits for those events and fills two arrays of
 * 4 entries indexed by kind: 0 = normalise+cast (2 launches per call), 1 = SYRK X X^T, 2 = SYRK c A^2 + b A,
 * 3 = GEMM+AXPY; ms_by_kind = summed milliseconds, launches_by_kind = number of bracketed groups.
 * Profiling is process-wide and meant for single-threaded benchmark loops.
 */
int mi_profile_begin(void);
int mi_profile_end(float* ms_by_kind, int* launches_by_kind);

/*
 * Process-wide switches of kernel choice and step grouping, for A/B measurements and for tests that must reach a
 * particular kernel variant (no counterpart in the reference, whose Triton autotuner is steered by the presence of
 * absl.testing in sys.modules, triton_kernels/syrk.py:138-140).  An option is an integer; -1 means "decide by
 * shape / cost model" where that exists.
 *   "streamk"         -1 | 0 | 1   split-tail launch of mi_syrk_bf16_ws: by the model | never | whenever it applies
 *   "syrk_transpose"  -1 | 0 | 1   transposing copy of a K-strided operand in mi_syrk_bf16_ws: likewise
 *   "head_apply"       0 | 1       slab kernel for the B X product of 128-row matrices (default 1)
 *   "head_front"       0 | 1       input pass of 128-row matrices that also leaves the Gram partials (default 1)
 *   "tall_direct"      0 | 1       last product of a tall input writes the float32 result transposed (default 1)
 *   "ns_pairs"        -1 | 0 | 1 | 2   steps sharing a Gram matrix: by shape | never | never three at once | pairs
 *                                      at every size
 * Initial values come from the environment variables MI_STREAMK, MI_SYRK_TRANSPOSE, MI_HEAD_APPLY, MI_HEAD_FRONT,
 * MI_TALL_DIRECT, MI_NS_PAIRS (numbers as above; MI_NS_PAIRS also "pairs" = 1, "force" = 2), read once when the
 * first option is looked up; no call reads the environment after that.  mi_set_option is atomic per option but not
 * ordered against calls in flight on other host threads: "ns_pairs" and "tall_direct" change the workspace size,
 * so set them before mi_newton_schulz_workspace_bytes and leave them alone until the call that uses that size
 * has returned.  Unknown names and out-of-range values return MI_ERR_BAD_ARG.
 */
int mi_set_option(const char* name, int value);
int mi_get_option(const char* name, int* value);

/*
 * What the last product launched from this host thread used (for tests that must know which kernel variant served
 * a shape; the reference's tests check its autotuner's config pruning instead,
 * tests/test_triton_kernels.py:90-125): workgroups per batch entry, tile rows and columns, and whether it was the
 * direct-to-LDS kernel (1; 2 for its stream-K launch) or the general one (0).  Any pointer may be NULL.
 */
int mi_debug_last_launch(int* tiles, int* tile_m, int* tile_n, int* fast);

#ifdef __cplusplus
}
#endif
#endif /* MI_NS_H_ */
