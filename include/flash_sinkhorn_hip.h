/*
 * C ABI of the MI355X (gfx950) FlashSinkhorn kernels.
 *
 * The reference (ot-triton-lab/flash-sinkhorn) has no FFI layer: its device
 * boundary is the set of Python launcher functions in flash_sinkhorn/kernels/
 * that call Triton kernels.  Each entry point below replaces one of those
 * launchers (cited per function, paths relative to src/flash_sinkhorn/).
 *
 * Conventions
 *  - every pointer is a DEVICE pointer to contiguous row-major fp32 unless
 *    stated otherwise; sizes are element counts
 *  - nothing here allocates or frees device memory; the caller owns inputs,
 *    outputs and the workspace (size from fs_workspace_bytes)
 *  - all work is enqueued on `stream` (a hipStream_t passed as void*) and
 *    returns without synchronising; the library keeps no mutable global state
 *    (fs_symmetric_step_noalloc remembers, per device, the address of its built-in buffer)
 *  - return value: FS_OK or a negative FS_ERR_* code (fs_error_string names it)
 *  - flags: FS_FLAG_EXP2 is accepted for interface parity (the kernels always
 *    work in base 2, which is the same function).  Operand precision (everything
 *    accumulates in fp32):
 *      default                    operands as two fp16 planes (22 significand bits) of
 *                                 the matrix scaled by a power of two, three MFMA
 *                                 products: error at or below that of fp32 MFMA operands
 *      FS_FLAG_FP32_MFMA          fp32 operands on v_mfma_f32_32x32x2_f32
 *      FS_FLAG_REDUCED_OPERANDS   permission to use less precise operands (the counterpart of
 *                                 allow_tf32=True); accepted and not acted on: the default
 *                                 mode is the fastest one on this machine
 *    The d <= 128 log-sum-exp kernel leaves out the exponentials of a 32 x 32 logits tile
 *    whose every entry lies more than 2^40 below its row's running maximum (they cannot
 *    change the fp32 row sums); FS_FLAG_NO_TILE_SKIP computes them all the same.
 *    FS_FLAG_COARSE_TEST (log-sum-exp entry points, default operand mode, d <= 128; the carried
 *    margins described below exist at d <= 64 only) applies the
 *    same 2^40 criterion one stage earlier: the hi*hi plane product of a tile is tested
 *    against the running maximum, lowered by a per-row bound on the two cross products, and a
 *    tile that fails ends there (5 MFMAs instead of 13 at d = 64).  What the test can end
 *    depends on where a row's running maximum starts.  With FS_FLAG_OPERANDS_PREPARED the
 *    workspace keeps one int per row next to the planes: the key that held the row's largest
 *    logit in the last launch over these operands.  The row's current logit at that key, a
 *    lower bound of its new maximum whatever the potentials did in between, is where the
 *    running maximum starts; once the potentials settle it is the maximum, and on a peaked
 *    plan nearly every tile ends at the test, sorted rows or not.  Any content of that array
 *    leaves the results exact (indices are clamped into the key set); fs_prepare_operands
 *    resets it, and a row without a key starts from the largest logit of 64 keys sampled from
 *    the whole key set.  With prepared operands the workspace also carries, per 32 query rows
 *    and 32 keys, by how much a tile that ended at the test stayed clear of mattering, together
 *    with the running sum of the largest key-bias changes of the launches so far: as long as
 *    twice the bias change accumulated since a tile's test is below its margin, the tile would
 *    end again, and the launch does not visit it.  The margins are dropped when the operands'
 *    pairing, eps or the bias coefficients change; overwritten keys only cost visits.  Once the
 *    potentials of a solve move little, more than nine tiles in ten are not visited on a peaked
 *    plan (the launch then runs as wavefronts that take lists of tiles to visit from work
 *    queues in the same workspace).
 *    Results stay within fp32 rounding of the full computation.  On a flat plan, where every
 *    tile matters, the test costs about 20 %.  Ignored where it does not apply.
 *    FS_FLAG_COARSE_AUTO (with FS_FLAG_OPERANDS_PREPARED, same conditions) leaves that choice to
 *    the device: every step enqueues both variants and a word of state next to the prepared
 *    planes says which one runs (the workgroups of the other return at once).  The coarse
 *    variant runs first and counts the tiles that end at its test in workgroups whose rows all
 *    started from a key of the launch before; the third launch with such counts decides: if
 *    fewer than 40 % of its tiles ended, the step's merge kernel switches to the plain variant
 *    while the plan stays as flat.  The plain variant counts in turn the tiles whose
 *    exponentials it left out (all logits 2^40 below their rows' running maxima), and a launch
 *    that left out a clearly larger share than the first plain launch of the stretch (by 4 % of
 *    all tiles) hands the next one back to the coarse variant: a schedule of decreasing eps
 *    starts flat and ends peaked.  The state is reset by fs_prepare_operands,
 *    with FS_FLAG_START_PLAIN among its flags to the plain variant (what a caller passes who
 *    knows that its first steps run at a large eps).  Nothing is read back or timed on the
 *    host: the same inputs take the same path on every run, and the calls can be captured into
 *    a graph.
 *    One more form of a two-sided step lives in the same state (fs_symmetric_step(s) and
 *    fs_self_pair_steps on prepared operands, default operand mode, every matrix of 2048 rows
 *    or more): when the sums of a step show that the potentials have settled, the next step
 *    (under the same eps or another: on a flat plan the sums hardly move with eps) computes
 *    every logit once and takes both sides' sums from the same exponentials (row sums and
 *    column sums of 2^(logit + both biases), no running maximum).
 *    Its merge checks every sum against the range in which that is exact in fp32 and has the
 *    two-sided kernel, enqueued behind it, redo the step otherwise: results stay within fp32
 *    rounding of the two-sided step whatever a caller does to the potentials between steps,
 *    and the same inputs give the same bits on every run.  A problem of a matrix with itself
 *    (fs_self_pair_steps, or fs_symmetric_step with x == y and aliased vectors) has a symmetric
 *    matrix of logits: that form then visits only the tiles on and above the diagonal, a row's
 *    sum being its row sums there plus the column sums the earlier rows took for it.
 *    FS_FLAG_NO_SWEEP keeps every step two-sided.
 *    Every operation runs on the two-plane fp16 operands by default and on fp32 MFMA operands
 *    with FS_FLAG_FP32_MFMA (the c-transform at d > 128: fp16 planes in either case).
 */
#ifndef FLASH_SINKHORN_HIP_H
#define FLASH_SINKHORN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FS_OK 0
#define FS_ERR_NULL_POINTER (-1)
#define FS_ERR_BAD_SIZE (-2)
#define FS_ERR_BAD_ARGUMENT (-3)
#define FS_ERR_WORKSPACE_TOO_SMALL (-4)
#define FS_ERR_LAUNCH_FAILED (-5)
#define FS_ERR_UNSUPPORTED (-6)
#define FS_ERR_SCRATCH_TOO_SMALL (-7)

#define FS_FLAG_EXP2 1u
#define FS_FLAG_REDUCED_OPERANDS 2u
#define FS_FLAG_FP32_MFMA 4u
/* 8u: unused (three-plane bf16 operands in ABI version 1) */
#define FS_FLAG_OPERANDS_PREPARED 16u
#define FS_FLAG_NO_TILE_SKIP 32u
#define FS_FLAG_COARSE_TEST 64u
#define FS_FLAG_COARSE_AUTO 128u
#define FS_FLAG_START_PLAIN 256u
#define FS_FLAG_NO_SWEEP 512u

/* operation ids for fs_workspace_bytes */
#define FS_OP_LSE 0
#define FS_OP_SYMMETRIC_STEP 1
#define FS_OP_GRAD 2
#define FS_OP_APPLY_VEC 3
#define FS_OP_APPLY_MAT 4
#define FS_OP_MAT5 5
#define FS_OP_C_TRANSFORM 6

int fs_version(void);
const char* fs_error_string(int code);

/* Bytes of device scratch the given operation needs for an (n, m, d) problem. */
size_t fs_workspace_bytes(int op, int64_t n, int64_t m, int64_t d);

/*
 * Optional: writes the 16-bit operand planes of x:[n,d] and y:[m,d] that the log-sum-exp
 * kernels multiply (see the precision notes above) into the head of `workspace`.  A solver
 * loop calls it once and then passes FS_FLAG_OPERANDS_PREPARED, the same workspace, the same
 * x / y pointers (in either role) and the same precision flags to every fs_lse,
 * fs_lse_fused and fs_symmetric_step of the loop, which then skip the conversion.  The
 * workspace must be sized for the largest of those operations; without the flag every call
 * converts its operands itself.  No counterpart in the reference: its Triton kernels read
 * the fp32 operands directly (kernels/sinkhorn_flashstyle_sqeuclid.py:194-661).
 */
int fs_prepare_operands(const float* x, const float* y, int64_t n, int64_t m, int64_t d,
                        uint32_t flags, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Byte offset, inside a workspace that fs_prepare_operands(x, y, ...) has filled, of the state
 * FS_FLAG_COARSE_AUTO keeps (0 when the configuration has none).  32-bit words a caller
 * may read for diagnostics once the stream has drained: [0] the variant the steps run now
 * (0: coarse tile test, 1: plain), [1] decisions taken so far, [2..3] a 64-bit count of the
 * 32 x 32 logits tiles that ended at the coarse test or were not visited at all (in launches of
 * the plain variant: whose exponentials were left out), [4..5] of all tiles of those launches,
 * [6..7] of the tiles not visited (carried margins, part of [2..3]); [247] non-zero: the next
 * two-sided step may take both sides' sums from one sweep; [269] how many such steps the
 * two-sided kernel had to redo so far.
 * Host arithmetic only.  No counterpart in the reference.
 */
size_t fs_variant_state_offset(const float* x, const float* y, int64_t n, int64_t m, int64_t d,
                               uint32_t flags);

/*
 * Byte offset, inside the same workspace, of the per-row keys FS_FLAG_COARSE_TEST starts from:
 * one int32 per row of x (which = 0) or of y (which = 1), the key of the other matrix (or of
 * the same one, for a self problem) that held the row's largest logit in the last launch with
 * that matrix as the stationary one; -1: none yet.  0 when the configuration keeps none.
 * Diagnostics and tests only; host arithmetic only.  No counterpart in the reference.
 */
size_t fs_best_keys_offset(const float* x, const float* y, int64_t n, int64_t m, int64_t d,
                           uint32_t flags, int which);

/*
 * out[i] = -eps*damping * LSE_j[ coord_scale * x_i.y_j / eps + bias[j] ]
 * Replaces flashsinkhorn_lse (kernels/sinkhorn_flashstyle_sqeuclid.py:815-955,
 * kernel 194-307).  x:[n,d] y:[m,d] bias:[m] out:[n].
 */
int fs_lse(const float* x, const float* y, const float* bias, float* out,
           int64_t n, int64_t m, int64_t d, float eps, float coord_scale, float damping,
           uint32_t flags, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Same with bias[j] = pot_hat[j]/eps + log_w[j] formed inside the kernel.
 * Replaces flashsinkhorn_lse_fused (kernels/sinkhorn_flashstyle_sqeuclid.py:958-1090,
 * kernel 317-419).
 */
int fs_lse_fused(const float* x, const float* y, const float* pot_hat, const float* log_w,
                 float* out, int64_t n, int64_t m, int64_t d, float eps, float coord_scale,
                 float damping, uint32_t flags, void* workspace, size_t workspace_bytes,
                 void* stream);

/*
 * One Jacobi step on shifted potentials, both halves from the OLD potentials:
 *   f_out = (1-alpha) f_hat + alpha * (-eps*damp_f * LSE_j[(cs2 x.y + g_hat_j)/eps + log_b_j])
 *           - alpha*(1-damp_f)*shift_x      (only when shift_x != NULL)
 *   g_out likewise over i.
 * Replaces flashsinkhorn_symmetric_step (kernels/sinkhorn_flashstyle_sqeuclid.py:1093-1317,
 * kernel 433-661).  shift_x/shift_y (= cost_scale*|x|^2, cost_scale*|y|^2, may be NULL)
 * fold in the unbalanced shift correction the reference's solver applies on the
 * host right after the launch (sinkhorn_solvers.py:509-517).  Outputs must not
 * alias inputs.  Self problem OT(x, x): when x == y, f_hat == g_hat, log_a == log_b,
 * shift_x == shift_y, f_out == g_out (same pointers), n == m and damp_f == damp_g, the two
 * half-updates are the same numbers and are computed once; f_out == g_out otherwise is an
 * error.
 */
int fs_symmetric_step(const float* x, const float* y, const float* f_hat, const float* g_hat,
                      const float* log_a, const float* log_b, float* f_out, float* g_out,
                      const float* shift_x, const float* shift_y,
                      int64_t n, int64_t m, int64_t d, float eps, float alpha, float damp_f,
                      float damp_g, float coord_scale, uint32_t flags, void* workspace,
                      size_t workspace_bytes, void* stream);

/*
 * fs_symmetric_step without a workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference.  The scratch the kernels need (operand planes and
 * partial soft-max rows) lives in a buffer of FS_NOALLOC_SCRATCH_BYTES that is part of the
 * library's code object: every GPU the library runs on holds its own copy until the process
 * ends.  The call allocates and frees nothing; the first call on a device looks up that
 * device's buffer address (callers that will capture make one call before capture starts).
 * Problems with fs_workspace_bytes(FS_OP_SYMMETRIC_STEP, n, m, d) above the buffer size return
 * FS_ERR_SCRATCH_TOO_SMALL.  The device the pointers and the stream belong to must be the
 * current one.  All calls on one GPU share the one buffer: calls that overlap in time on one GPU
 * (two streams, two threads) race; calls ordered on one stream do not.  FS_FLAG_OPERANDS_PREPARED
 * and FS_FLAG_COARSE_AUTO are ignored (every call writes its own operand planes).
 */
#define FS_NOALLOC_SCRATCH_BYTES ((size_t)48 << 20)
int fs_symmetric_step_noalloc(const float* x, const float* y, const float* f_hat,
                              const float* g_hat, const float* log_a, const float* log_b,
                              float* f_out, float* g_out, const float* shift_x,
                              const float* shift_y, int64_t n, int64_t m, int64_t d, float eps,
                              float alpha, float damp_f, float damp_g, float coord_scale,
                              uint32_t flags, void* stream);

/*
 * n_steps Jacobi steps of fs_symmetric_step back to back, enqueued by one call: step s runs
 * with eps[s], alpha[s], damp_f[s], damp_g[s] (HOST arrays of n_steps floats) and reads the
 * potentials step s-1 wrote (step 0 reads f_hat, g_hat).  Even steps write (f_a, g_a), odd
 * steps (f_b, g_b); the result of the call is the pair of parity (n_steps - 1) & 1.  The four
 * work vectors must not alias f_hat / g_hat or each other, except f_a == g_a and f_b == g_b
 * for the self problem (see fs_symmetric_step).  shift_x / shift_y as there; they apply to
 * every step whose damping is below 1.
 * Replaces the iteration of sinkhorn_flashstyle_symmetric (sinkhorn_solvers.py:482-560: the
 * initial step, the averaged steps over eps_list and the extrapolation step are each one
 * flashsinkhorn_symmetric_step call there); the Python mirror batches the steps between two
 * convergence checks into one call.
 */
int fs_symmetric_steps(const float* x, const float* y, const float* f_hat, const float* g_hat,
                       const float* log_a, const float* log_b, float* f_a, float* g_a, float* f_b,
                       float* g_b, const float* shift_x, const float* shift_y, int64_t n,
                       int64_t m, int64_t d, const float* eps, const float* alpha,
                       const float* damp_f, const float* damp_g, int n_steps, float coord_scale,
                       uint32_t flags, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Schur-complement product of the Hessian-vector path: piz = (P z) / diag_x (n values), then
 * out = denom * z - P^T piz (m values), P as in fs_apply_vec.  Two stream-ordered launches with
 * the element-wise factors folded into their epilogues; inv_diag_x holds 1 / diag_x.  out must
 * not alias z.  Workspace: fs_workspace_bytes(FS_OP_APPLY_VEC, n, m, d).
 * Replaces fused_schur_matvec_sqeuclid (kernels/sinkhorn_triton_apply_fused_sqeuclid.py:283-470;
 * the reference's single launch joins its two phases with a spin-wait grid barrier and falls
 * back to two launches when the grid does not fit the device; here the two launches are the
 * design: a kernel that waits for other workgroups must not exist on this machine).
 */
int fs_schur_matvec(const float* x, const float* y, const float* f_hat, const float* g_hat,
                    const float* log_a, const float* log_b, const float* z, const float* inv_diag_x,
                    const float* denom, float* piz, float* out, int64_t n, int64_t m, int64_t d,
                    float eps, float coord_scale, uint32_t flags, void* workspace,
                    size_t workspace_bytes, void* stream);

/*
 * Conjugate gradients with the bookkeeping on the device (no counterpart kernel in the
 * reference: its conjugate_gradient, cg.py:27-121, runs these vector operations as separate
 * PyTorch launches and reads the residual norm back every iteration).
 * fs_cg_init: sol = 0, res = dir = b, state = {r.r, |r0|, tol = max(atol, rtol*|r0|), |r|,
 * done = 0, converged = 0, iterations = 0, -} (8 floats on the device).
 * fs_cg_update, after the caller has computed a_dir = A dir: the curvature dir.a_dir, the step,
 * sol += step*dir, res -= step*a_dir, |res|; stops (done = converged = 1) when |res| <= tol,
 * stops without convergence when the curvature is exactly zero, otherwise
 * dir = res + (|res|^2 / r.r) dir.  Once done is set further updates change nothing, so a
 * caller may enqueue several iterations between two looks at the state and still get the
 * iterate and the iteration count of the step that met the tolerance.  Sums are accumulated in
 * double precision.  One workgroup per launch: meant for the n- and m-vectors of the Schur
 * system, not for large unknowns.
 */
int fs_cg_init(const float* b, float* sol, float* res, float* dir, float* state, int64_t m,
               float rtol, float atol, void* stream);
int fs_cg_update(const float* a_dir, float* sol, float* res, float* dir, float* state, int64_t m,
                 void* stream);

/*
 * The two self problems OT(x, x; a) and OT(y, y; b) of a debiased divergence, n_steps Jacobi
 * steps each, one launch per step for both: in a self problem both potentials stay equal, so a
 * step is one half-update per problem, fx' = (1-alpha) fx + alpha*(-eps_x*damp_x*LSE_j[...]) over
 * the rows of x against x itself, and likewise fy' over y.  eps_x, eps_y, alpha, damp_x, damp_y
 * are HOST arrays of n_steps floats (the two problems may follow different eps schedules; the
 * averaging weight is shared).  Step s reads what step s-1 wrote (step 0 reads fx_hat, fy_hat);
 * even steps write (fx_a, fy_a), odd steps (fx_b, fy_b).  shift_x / shift_y as in
 * fs_symmetric_step.  Workspace: fs_workspace_bytes(FS_OP_SYMMETRIC_STEP, n, n, d) +
 * fs_workspace_bytes(FS_OP_SYMMETRIC_STEP, m, m, d) bytes suffice; with
 * FS_FLAG_OPERANDS_PREPARED the planes are those fs_prepare_operands(x, y, ...) wrote.
 * Replaces the two independent solves sinkhorn_flashstyle_symmetric(x, x, a, a, ...) and
 * (y, y, b, b, ...) that SamplesLoss(debias=True) runs (samples_loss.py:494-512).
 */
int fs_self_pair_steps(const float* x, const float* y, const float* fx_hat, const float* fy_hat,
                       const float* log_a, const float* log_b, float* fx_a, float* fy_a,
                       float* fx_b, float* fy_b, const float* shift_x, const float* shift_y,
                       int64_t n, int64_t m, int64_t d, const float* eps_x, const float* eps_y,
                       const float* alpha, const float* damp_x, const float* damp_y, int n_steps,
                       float coord_scale, uint32_t flags, void* workspace, size_t workspace_bytes,
                       void* stream);

/*
 * Analytic gradient: grad_x[i,:] = 2*cost_scale*gs*a_i*(x_i - sum_j w_ij y_j),
 * w_i. = softmax_j[(g_j - C_ij)/eps + log_b_j]; grad_y symmetric over i.
 * Standard (unshifted) potentials f, g; x2, y2 = row squared norms; gs is read
 * from the 1-element device array grad_scale (NULL means 1).  Either output may
 * be NULL.  Picks the large-d variant internally.
 * Replaces sinkhorn_geomloss_online_grad_sqeuclid
 * (kernels/sinkhorn_triton_grad_sqeuclid.py:891-1207, kernels 101-402 and 405-791).
 */
int fs_grad(const float* x, const float* y, const float* f, const float* g, const float* log_a,
            const float* log_b, const float* a, const float* b, const float* x2, const float* y2,
            const float* grad_scale, float* grad_x, float* grad_y, int64_t n, int64_t m,
            int64_t d, float eps, float cost_scale, uint32_t flags, void* workspace,
            size_t workspace_bytes, void* stream);

/*
 * fs_grad with a hint, no counterpart in the reference: keys_x[i] (keys_y[j]) names a row of y
 * (of x) at which row i of x (row j of y) has a large logit, typically the carried keys that a
 * solve with FS_FLAG_COARSE_TEST left in its prepared workspace (fs_best_keys_offset), or NULL.
 * The rows' running maxima start from their logits at these keys, so that tiles that cannot
 * matter are recognised from the first tile on; any content leaves the results exact (indices
 * are clamped into range, negative ones mean "none").  d <= 128 in the default operand mode;
 * ignored elsewhere.
 */
int fs_grad_seeded(const float* x, const float* y, const float* f, const float* g,
                   const float* log_a, const float* log_b, const float* a, const float* b,
                   const float* x2, const float* y2, const float* grad_scale, float* grad_x,
                   float* grad_y, int64_t n, int64_t m, int64_t d, float eps, float cost_scale,
                   const int* keys_x, const int* keys_y, uint32_t flags, void* workspace,
                   size_t workspace_bytes, void* stream);


/*
 * axis=1: out[i] = sum_j P_ij vec[j];  axis=0: out[j] = sum_i P_ij vec[i], with
 * P_ij = exp(log_a_i + log_b_j + (f_hat_i + g_hat_j + coord_scale x_i.y_j)/eps).
 * Replaces apply_plan_vec_flashstyle (kernels/apply_flash.py:835-951, kernels 594-832).
 */
int fs_apply_vec(const float* x, const float* y, const float* f_hat, const float* g_hat,
                 const float* log_a, const float* log_b, const float* vec, float* out,
                 int64_t n, int64_t m, int64_t d, float eps, float coord_scale, int axis,
                 uint32_t flags, void* workspace, size_t workspace_bytes, void* stream);

/*
 * axis=1: out = P @ (mat * scale[:,None]) (mat:[m,dv], scale:[m] or NULL);
 * axis=0: out = P^T @ mat (mat:[n,dv], scale must be NULL).  out:[n|m, dv].
 * Replaces apply_plan_mat_flashstyle (kernels/apply_flash.py:360-579, kernels 49-343);
 * the reference fixes dv == d.
 */
int fs_apply_mat(const float* x, const float* y, const float* f_hat, const float* g_hat,
                 const float* log_a, const float* log_b, const float* mat, const float* scale,
                 float* out, int64_t n, int64_t m, int64_t d, int64_t dv, float eps,
                 float coord_scale, int axis, uint32_t flags, void* workspace,
                 size_t workspace_bytes, void* stream);

/*
 * out[i,:] = (-4*cost_scale/eps) * sum_j P_ij (A_i.y_j) y_j with
 * P_ij = exp((f_ott_i + g_ott_j - cost_scale*|x_i-y_j|^2)/eps).
 * Replaces mat5_sqeuclid (kernels/apply_ott.py:453-566, kernel 34-168).
 */
int fs_mat5(const float* x, const float* y, const float* f_ott, const float* g_ott,
            const float* A, const float* x2, const float* y2, float* out, int64_t n, int64_t m,
            int64_t d, float eps, float cost_scale, uint32_t flags, void* workspace,
            size_t workspace_bytes, void* stream);

/*
 * Hard c-transform, the eps -> 0 counterpart of fs_lse:
 *   min_out[i] = min_j [-coord_scale x_i.y_j + bias_j],  argmin_out[i] = the smallest j
 * attaining it (int64).  The caller passes bias_j = cost_scale |y_j|^2 - psi_j and adds
 * cost_scale |x_i|^2 to min_out.  Runs on the two-plane fp16 operands (fp32 MFMA operands for
 * d <= 128 with FS_FLAG_FP32_MFMA).
 * Replaces c_transform_kernel (kernels/c_transform_sqeuclid.py:219-354, kernel 117-214).
 */
int fs_c_transform(const float* x, const float* y, const float* bias, float* min_out,
                   int64_t* argmin_out, int64_t n, int64_t m, int64_t d, float coord_scale,
                   uint32_t flags, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_SINKHORN_HIP_H */
