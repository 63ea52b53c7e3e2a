/*
 * kai_hip.h -- C-ABI of libkai_hip.so: the fp32 matrix-multiplication path of
 * the KONAN AI engine (class VMath, source/engine/support/vmath.h of the
 * reference) as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions (they hold for every entry point below)
 *  - Return value: 0 (KAI_OK) or one of the reference's numeric error codes
 *    (source/engine/include/verrors.h).  Nothing is thrown across this boundary;
 *    kai_last_error() returns the calling thread's last message.
 *  - `device`: the reference selects the host loop with device < 0 and the GPU
 *    kernel with device >= 0 (CUDA_CALL, vmath.cu:46-55).  This library is the GPU
 *    side only.  device < 0 returns KAI_ERR_INVALID_ARGUMENT for compute entry
 *    points: the host loops stay in the engine.  For device >= 0 the kernel is
 *    enqueued on the calling thread's CURRENT device, which the caller has already
 *    selected (the engine does it in VDeviceManager::setCurDevice,
 *    local_objects/vdevicemanager.cpp:110-122); kai_set_device() is exported for
 *    that.  Only kai_mem_alloc switches devices itself, as the reference does
 *    (vmath.cu:170-204).
 *  - Pointers are raw device pointers owned by the caller; the library never
 *    allocates, frees or caches them.  Whole buffers from kai_mem_alloc are
 *    16-byte aligned; sub-buffer pointers of any 4-byte alignment are accepted
 *    (slower loads are chosen automatically).  In-place aliasing is legal where the
 *    reference uses it: add_bias (py == pa), activate (py == px), the softmax and
 *    mask ops.  A GEMM output must not alias its inputs.
 *  - Hyper-parameters (`hLeakyAlpha`, `hCoef`) are DEVICE pointers to one float,
 *    read inside the kernel; null reads as 0 (HYPER_ACCESS,
 *    local_objects/vhypermanager.h:9).
 *  - Work is enqueued asynchronously on the stream set by kai_set_stream (the null
 *    stream by default, matching the reference's use of the legacy default
 *    stream); results are ordered by stream order and by the blocking copies.
 *  - `acc` != 0 adds the product to the existing output instead of overwriting it.
 *  - All matrices are dense row-major fp32.  Sizes are int64_t as in the reference
 *    (include/vtypes.h:18-22); each dimension and each leading dimension must be
 *    below 2^31.
 */
#ifndef KAI_HIP_H
#define KAI_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* error codes: the reference's numbers (source/engine/include/verrors.h:4,12,39,52,149,164) */
#define KAI_OK 0
#define KAI_ERR_CONDITIONAL_STATEMENT 8   /* unknown activation code (vmath.cu:3159-3161) */
#define KAI_ERR_INVALID_ARGUMENT 510
#define KAI_ERR_INVALID_POINTER 523
#define KAI_ERR_HOSTMEM_ALLOC_FAILURE 10012
#define KAI_ERR_GPU 50002                 /* VERR_CUDA_ERROR: any HIP runtime or launch error */

/* activation codes, enum class ActFunc (source/engine/include/vtypes.h:37-39) */
#define KAI_ACT_NONE 0
#define KAI_ACT_RELU 1
#define KAI_ACT_LEAKY 2
#define KAI_ACT_SIGMOID 3
#define KAI_ACT_TANH 4
#define KAI_ACT_GELU 5
#define KAI_ACT_SELU 6
#define KAI_ACT_MISH 7
#define KAI_ACT_SWISH 8
#define KAI_ACT_SOFTMAX 9

/* ---- library state --------------------------------------------------------------------------- */

/* Message of the calling thread's last failing call ("" if none).  Replaces the text the
 * reference passes to VP_THROW1(VERR_CUDA_ERROR, "cuda:"+msg) in VMath::cudaCheck (vmath.cu:64-87). */
const char* kai_last_error(void);
/* Number of visible GPUs (reference: cudaGetDeviceCount, local_objects/vdevicemanager.cpp:59-63). */
int kai_device_count(int* count);
/* hipSetDevice for the calling thread (reference: VDeviceManager::setCurDevice, vdevicemanager.cpp:110-122). */
int kai_set_device(int device);
/* Blocks until the current device is idle.  The reference's live path has no such call (it relies
 * on blocking cudaMemcpy); exported for harnesses that time kernels. */
int kai_device_synchronize(void);
/* Stream (a hipStream_t, or null for the null stream) that this THREAD's later calls enqueue on.
 * No counterpart in the reference, which only uses the legacy default stream. */
int kai_set_stream(void* hip_stream);
/* Releases the scratch memory the library allocated for itself (partial sums of reductions cut into parts,
 * of the column sums of long narrow matrices, row norms of kai_cosinesim, the probabilities of a kai_attention_forward call that runs as separate
 * kernels; one buffer per device, created on first need).  Waits for the device first.  The library stays
 * usable: the buffer is created again on demand.  No counterpart in the reference, whose kernels need no
 * scratch. */
int kai_shutdown(void);
/* Makes the current device's scratch at least `bytes` large now, so that later calls find it and allocate
 * nothing: for callers that record calls into a HIP graph (a call whose scratch would have to grow while its
 * stream is being captured fails with KAI_ERR_GPU) or that cannot tolerate an allocation inside a step.  A
 * product never asks for more than 64 MiB of partial sums; kai_attention_forward outside the fused head sizes
 * asks for nbat*ntimes*ntimes*nhead floats on top.  Growing never waits for the device: the smaller buffer is
 * kept until kai_shutdown, so work in flight and recorded graphs stay valid.  No counterpart in the reference. */
int kai_reserve_scratch(int64_t bytes);
/* Current size of the current device's scratch, how many times it was allocated or grown since the last
 * kai_shutdown, and the bytes of replaced buffers still held.  Any pointer may be null.  For tests and
 * diagnostics; no counterpart in the reference. */
int kai_scratch_info(int64_t* bytes, int64_t* growths, int64_t* retired_bytes);
/* Name of the code object's target ("gfx950") and of the current device's architecture. */
int kai_arch_info(char* built_for, char* device_arch, int buflen);

/* ---- memory (VMath::mem_alloc ... get_slice, vmath.h:18-24,40-46,56) ---------------------------- */

/* vmath.cu:170-210: device >= 0 allocates `size` bytes rounded up to a multiple of 16 on that
 * device (saving and restoring the current device); device < 0 allocates host memory. */
int kai_mem_alloc(int device, int64_t size, void** out_ptr);
/* vmath.cu:232-265 */
int kai_mem_free(int device, void* ptr);
/* vmath.cu:278-293: blocking copies */
int kai_memcpy_host_to_host(void* dptr, const void* sptr, int64_t size);
int kai_memcpy_host_to_device(void* dptr, const void* sptr, int64_t size);
int kai_memcpy_device_to_host(void* dptr, const void* sptr, int64_t size);
int kai_memcpy_device_to_device(void* dptr, const void* sptr, int64_t size);
/* vmath.cu:351-360 */
int kai_copy_data(int dest_device, int src_device, void* py, const void* px, int64_t nbytes);
/* vmath.cu:494-530 (`size` counts elements) */
int kai_fill_int(int device, int* ptr, int64_t size, int value);
int kai_fill_float(int device, float* ptr, int64_t size, float value);
/* vmath.cu:534-541 (`size` counts bytes) */
int kai_set_zero(int device, void* ptr, int64_t size);
/* vmath.cu:545-578: py on `device` (host if < 0) <- host px / py host <- px on device / device<-device */
int kai_memcpy_from_host(int device, void* py, const void* px, int64_t size);
int kai_memcpy_to_host(int device, void* py, const void* px, int64_t size);
int kai_memcpy_to_device(int device, void* py, const void* px, int64_t size);
/* vmath.cu:708-715 */
int kai_get_slice(int device, void* py, const void* px, int64_t nbytes);

/* ---- dense layer: VMath::matmul family (vmath.h:137-139) ------------------------------------- */

/* VMath::matmul, vmath.cu:2961-3003.  y[ndat,yvec] (=|+=) x[ndat,xvec] . w[yvec,xvec]^T */
int kai_matmul(int device, float* py, const float* pw, const float* px, int64_t yvec, int64_t ndat, int64_t xvec,
               int acc);
/* VMath::matmul_backward_x, vmath.cu:3007-3047.  gx[ndat,xvec] (=|+=) gy[ndat,yvec] . w[yvec,xvec] */
int kai_matmul_backward_x(int device, float* pgx, const float* pgy, const float* pw, int64_t yvec, int64_t ndat,
                          int64_t xvec, int acc);
/* VMath::matmul_backward_w, vmath.cu:3051-3093.  gw[yvec,xvec] (=|+=) gy[ndat,yvec]^T . x[ndat,xvec] */
int kai_matmul_backward_w(int device, float* pgw, const float* pgy, const float* px, int64_t yvec, int64_t ndat,
                          int64_t xvec, int acc);

/* kai_matmul for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and the same kernels as
 * kai_matmul; it calls no hipMalloc / hipFree and never touches the library's heap scratch.
 * A product whose reduction is cut into parts keeps the partial sums in a fixed 32 MiB array inside the
 * library's code object (each GPU the library runs on holds its copy until the process ends); the number of parts
 * is chosen so that their sums fit the array, so a product that kai_matmul would cut finer runs here with fewer
 * parts (equal to kai_matmul up to the order of the partial sums, bit for bit wherever the part count is the
 * same).  Should a product ever need more than the array holds it is refused with KAI_ERR_INVALID_ARGUMENT and
 * a message that names both sizes.  All calls on one GPU share that array: calls that overlap on one GPU race
 * and must be serialised by the caller.
 * The first use on a device looks up the array's address, which may load the code object there: that must happen
 * BEFORE a stream capture begins.  kai_matmul_noalloc_scratch_bytes() does the look-up for the current device
 * (call it once per device at set-up) and returns the array's size; a first kai_matmul_noalloc made while the
 * thread's stream is being captured fails with KAI_ERR_GPU instead of allocating. */
int kai_matmul_noalloc(int device, float* py, const float* pw, const float* px, int64_t yvec, int64_t ndat,
                       int64_t xvec, int acc);
int64_t kai_matmul_noalloc_scratch_bytes(void);

/* VMath::add_bias, vmath.cu:875-897.  y[r,c] = a[r,c] + b[c]; py may equal pa */
int kai_add_bias(int device, float* py, const float* pa, const float* pb, int64_t nrow, int64_t ncol);
/* VMath::add_bias_backward_b, vmath.cu:901-932.  gb[c] (=|+=) sum_r gy[r,c].  With 6144 rows and more over few
 * columns the rows are summed in runs whose sums pass through the library scratch (at most 128 KiB); where that would have to grow during a stream
 * capture the call takes its single launch instead, which needs none. */
int kai_add_bias_backward_b(int device, float* pgb, const float* pgy, int64_t nrow, int64_t ncol, int acc);

/* VMath::activate, vmath.cu:3097-3243; py may equal px (except for softmax).  The softmax case
 * normalises each row of ncol elements (the reference's row pointer arithmetic at vmath.cu:3146
 * reads outside the buffer; the row-wise meaning is implemented). */
int kai_activate(int device, float* py, const float* px, int64_t nrow, int64_t ncol, int actFunc,
                 const float* hLeakyAlpha);
/* VMath::activate_backward, vmath.cu:3247-3407; px is the pre-activation input.  Codes 0..8 as on the
 * reference's host path plus softmax (9) as on its device path (vmath.cu:3363-3394). */
int kai_activate_backward(int device, float* pgx, const float* pgy, const float* px, int64_t nrow, int64_t ncol,
                          int actFunc, const float* hLeakyAlpha);
/* VMath::activate_backward_with_y, vmath.cu:3411-3486; codes 0..4 only */
int kai_activate_backward_with_y(int device, float* pgx, const float* pgy, const float* py, int64_t nrow,
                                 int64_t ncol, int actFunc, const float* hLeakyAlpha);

/* ---- attention: VMath::mult_on_heads family (vmath.h:234-241) --------------------------------- */

/* VMath::mult_on_heads, vmath.cu:6729-6779.  pp[b,q,k,h] = coef * sum_p K[b,k,h*npiece+p]*Q[b,q,h*npiece+p];
 * K, Q are [nbat, ntimes, nvec]; pp is [nbat, ntimes, ntimes, nhead] (head index innermost). */
int kai_mult_on_heads(int device, float* pp, const float* pK, const float* pQ, int64_t nbat, int64_t ntimes,
                      int64_t nvec, int64_t nhead, int64_t npiece, const float* hCoef);
/* VMath::mult_on_heads_backward, vmath.cu:6783-6829.  g[b,t,h*npiece+p] = sum_k gp[b,t,k,h]*KQ[b,k,h*npiece+p] */
int kai_mult_on_heads_backward(int device, float* pgQKV, const float* pgp, const float* pQKV, int64_t nbat,
                               int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece);
/* VMath::set_mh_attention_mask, vmath.cu:6833-6860.  pp[b,q,k,h] = forward ? -inf : 0 for k > q */
int kai_set_mh_attention_mask(int device, float* pp, int64_t ndat, int64_t ntimes, int64_t nhead, int forward);
/* VMath::softmax_direct_on_axis, vmath.cu:6864-6916.  In place, softmax over the middle axis of
 * [nrow, nvec, ncol]. */
int kai_softmax_direct_on_axis(int device, float* pp, int64_t nrow, int64_t nvec, int64_t ncol);
/* VMath::softmax_direct_on_axis_backward, vmath.cu:6920-6973.  In place on pgp:
 * gp = coef * p * (gp - sum_k p*gp) */
int kai_softmax_direct_on_axis_backward(int device, float* pgp, const float* pp, int64_t nbat, int64_t ntimes,
                                        int64_t nhead, const float* hCoef);
/* VMath::mix_values, vmath.cu:6977-7025.  y[b,q,h,p] = sum_k pp[b,q,k,h] * V[b,k,h*npiece+p] */
int kai_mix_values(int device, float* py, const float* pp, const float* pV, int64_t nbat, int64_t ntimes,
                   int64_t nvec, int64_t nhead, int64_t npiece);
/* VMath::mix_values_backward_prop, vmath.cu:7029-7077.  gp[b,q,k,h] = sum_p gy[b,q,h,p] * V[b,k,h*npiece+p] */
int kai_mix_values_backward_prop(int device, float* pgp, const float* pgy, const float* pV, int64_t nbat,
                                 int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece);
/* VMath::mix_values_backward_value, vmath.cu:7081-7129.  gV[b,k,h*npiece+p] = sum_q pp[b,q,k,h] * gy[b,q,h,p] */
int kai_mix_values_backward_value(int device, float* pgV, const float* pgy, const float* pp, int64_t nbat,
                                  int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece);

/* ---- fused entry points (additive: each equals a fixed sequence of the calls above) ------------ */

/* C[M,N] (=|+=) act( op(A) . op(B) + bias ), row-major.
 *   transA == 0: A is [M,K] with row stride lda;  transA != 0: A is stored [K,M] (lda = its row stride)
 *   transB == 0: B is [K,N] with row stride ldb;  transB != 0: B is stored [N,K]
 * bias (length N) may be null; actFunc is an element-wise code 0..8.  With acc != 0 the order is
 * C = act(C + A.B + bias).  Equals matmul / matmul_backward_x / matmul_backward_w for the operand
 * forms (0,1) / (0,0) / (1,0), followed by add_bias and activate. */
int kai_gemm_f32(int device, int transA, int transB, int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                 const float* B, int64_t ldb, float* C, int64_t ldc, const float* bias, int actFunc,
                 const float* hLeakyAlpha, int acc);

/* No counterpart in the reference (its kernels are one per method).  Writes into `out` which kernel
 * kai_gemm_f32 would launch for 16-byte aligned operands of this shape, as text: "wavesplit 16",
 * "skinny", "shortk_nt", "mfma large whole pipelined split 1", "mfma small general split 4" ...  Host
 * arithmetic only: nothing is launched or allocated and no GPU is needed (without one the choice is made
 * for 256 compute units).  For maintainers and tests of the dispatch rules. */
int kai_gemm_plan(int transA, int transB, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                  int has_bias, int actFunc, int acc, char* out, int buflen);

/* No counterpart in the reference.  A maintainer's override of the dispatcher's choice for every later single
 * (unbatched) product of the process, for audits of the fitted dispatch rules (bench.py --plan-audit times the
 * chosen plan of a shape against every alternative): words in `text`, a tile name ("large", "medium", "small", "flat",
 * "wide") and / or "split N" (N = 1 .. 16 parts of the reduction), or "wavesplit 16" / "wavesplit 32" (the one-launch
 * kernel for small products, where it applies); "stream 16" / "stream 32" / "stream 48" sets only the rows of W
 * that a workgroup of the skinny streaming kernel owns, for the products that kernel takes anyway, and forces no
 * tile; "auto", "" or null clears the override.  A part count that the
 * product cannot take runs as one part.  kai_gemm_plan reports what would run.  Process-wide and not synchronised
 * with calls in flight on other threads: not for production use. */
int kai_gemm_force_plan(const char* text);

/* The engine's `dense` layer formula activate(add(matmul(x,w),b)) (api/vconst.cpp:11) in one launch:
 * py = act(x . w^T + b).  ppre, if not null, receives the pre-activation x . w^T + b that
 * VTensor::activate_backprop needs (vtensor.cpp:5697-5718).  pb may be null (no bias). */
int kai_dense_forward(int device, float* py, float* ppre, const float* pw, const float* pb, const float* px,
                      int64_t yvec, int64_t ndat, int64_t xvec, int actFunc, const float* hLeakyAlpha);

/* Backward of the same layer: ga = activate_backward(gy, ppre) (skipped when ppre is null or
 * actFunc == 0), then gb = colsum(ga), gx = ga . w, gw = ga^T . x: the calls of VTensor::activate_backprop,
 * add_backprop and matmul_backprop (vtensor.cpp:5697-5718, 3470-3479, 1337-1375).  Any of pgx, pgw, pgb may
 * be null.  For none / relu / leaky relu, whole 64 x 64 x 32 tiles, 16-byte aligned operands and the sizes of a
 * mini-batch step (both products together at most four workgroups per compute unit) everything runs in ONE
 * launch, ga never written anywhere (plus a second launch that sums the parts of gx when its reduction is cut);
 * other shapes run the separate kernels with ga in pga_work, a caller buffer of ndat*yvec floats (may equal pgy
 * to overwrite it) or, when pga_work is null, in the library's scratch memory. */
int kai_dense_backward(int device, float* pgx, float* pgw, float* pgb, float* pga_work, const float* pgy,
                       const float* pw, const float* px, const float* ppre, int64_t yvec, int64_t ndat,
                       int64_t xvec, int actFunc, const float* hLeakyAlpha, int acc);

/* ---- cosine similarity (next to the path) ------------------------------------------------------------ */

/* VMath::cosinesim, vmath.cu:6459-6513 (vmath.h:226; driver VTensor::cosinesim, vtensor.cpp:5864-5890).
 * py[nrow1, nrow2] = <x1_i, x2_j> / (|x1_i| |x2_j| + 1e-20): the NT product of the path, the row norms and a
 * scaling pass.  Forward only, as in the reference (its backprop throws VERR_NOT_IMPLEMENTED_YET). */
int kai_cosinesim(int device, float* py, const float* px1, const float* px2, int64_t nrow1, int64_t nrow2,
                  int64_t ncol);

/* ---- recurrent layers (next to the path): the steps between the gate products ---------------------- */
/* VTensor's rnn/lstm/gru loop (vtensor.cpp:2455-2492, 2657-2701) issues, per time step, kai_matmul with
 * acc = 0 and 1 on sub-buffers at t * size offsets, kai_add_bias in place, and the calls below. */

/* VMath::copy, vmath.cu:732-752.  py[n] = pa[n], in stream order. */
int kai_copy(int device, float* py, const float* pa, int64_t ndat);
/* VMath::add, vmath.cu:774-794.  py[n] = pa[n] + pb[n]; py may be pa or pb. */
int kai_add(int device, float* py, const float* pa, const float* pb, int64_t ndat);
/* VMath::lstm_process, vmath.cu:4807-4857.  pa[ndat, 4*nrec] holds the pre-activations of the input, forget,
 * block and output gates; ps = ps1 * f + g * i (ps1 null: 0), pr = tanh(ps) * o.  ninp is unused, as there. */
int kai_lstm_process(int device, float* pr, float* ps, const float* ps1, const float* pa, int64_t ndat, int64_t nrec,
                     int64_t ninp);
/* VMath::lstm_process_backward, vmath.cu:4899-4943 (the device kernel; the host loop, vmath.cu:4860-4897, has the
 * same arithmetic but writes the gate gradients at apos * g + n * nrec, outside the buffer).  pa[ndat, 4*nrec]:
 * this step's gate sums; ps: the state the step started from (null: 0); pgr: gradient of this step's output
 * (read only); pgs: gradient of this step's state on entry, of the previous state on return;
 * pga[ndat, 4*nrec] receives the gate-sum gradients.  ninp is unused, as there. */
int kai_lstm_process_backward(int device, const float* pgr, float* pgs, float* pga, const float* ps, const float* pa,
                              int64_t ndat, int64_t nrec, int64_t ninp);
/* VMath::gru_process, vmath.cu:4946-4996.  pr points at step nt of [ntimes, ndat, nrec] and the previous step is
 * read ndat*nrec floats before it when nt > 0; pai/par[ndat, 3*nrec]: reset, update, candidate. */
int kai_gru_process(int device, float* pr, const float* pai, const float* par, int64_t nt, int64_t ntimes, int64_t ndat,
                    int64_t nrec);
/* VMath::gru_process_backward, vmath.cu:4999-5080.  pgr is replaced by the gradient of the previous step's output. */
int kai_gru_process_backward(int device, float* pgr, float* pgai, float* pgar, const float* pr, const float* pai,
                             const float* par, int64_t nt, int64_t ntimes, int64_t ndat, int64_t nrec);

/* One time step of the loop above in one launch (additive, no counterpart call in the reference):
 *   kai_lstm_step == [pr_prev: kai_matmul(pa, pwr, pr_prev, 4*nrec, ndat, nrec, acc = 1)], [kai_add_bias(pa, pbr)],
 *                    [kai_add_bias(pa, pbi)], kai_lstm_process(pr, ps, ps_prev, pa)
 * with pa[ndat, 4*nrec] holding the input products of this step on entry (kai_matmul over all time steps at
 * once, or per step) and the gate sums the cell saw on return, as the backward pass needs them.  pr_prev null:
 * first step, no recurrent product.  pbi, pbr, ps_prev may be null. */
int kai_lstm_step(int device, float* pr, float* ps, const float* ps_prev, float* pa, const float* pwr,
                  const float* pr_prev, const float* pbi, const float* pbr, int64_t ndat, int64_t nrec);
/*   kai_gru_step == par = pr_prev . pwr^T (zero when pr_prev is null), [kai_add_bias(par, pbr)],
 *                   [kai_add_bias(pai, pbi)], kai_gru_process with ph_prev as the previous output (null: 0).
 * pr_prev and ph_prev are separate because the engine's loop reads the output of step nt - 1 in both
 * directions (vmath.cu:4961) while the product takes the step processed before (vtensor.cpp:2464). */
int kai_gru_step(int device, float* pr, float* pai, float* par, const float* pwr, const float* pr_prev,
                 const float* ph_prev, const float* pbi, const float* pbr, int64_t ndat, int64_t nrec);

/* ---- transposes (next to the path) ----------------------------------------------------------------- */

/* VMath::transpose, vmath.cu:9384-9433 (vmath.h:309).  General axis permutation of a dense tensor of
 * data_size elements.  pn is the DEVICE table of axis_size x 3 ints that VTensor::transpose builds
 * (vtensor.cpp:5391-5417): pn[m*3] = source axis of output axis m, pn[m*3+1] = output elements per step
 * of output axis m, pn[a*3+2] = source elements per step of source axis a.  1 <= axis_size <= 8. */
int kai_transpose(int device, float* py, const float* px, const int* pn, int64_t axis_size, int64_t data_size);
/* VMath::transpose_backward, vmath.cu:9436-9483: pgx[source position] = pgy[n] with the same table. */
int kai_transpose_backward(int device, float* pgx, const float* pgy, const int* pn, int64_t axis_size,
                           int64_t data_size);
/* VMath::transpose_bin, vmath.cu:9487-9510: py[nrow, ncol] = px[ncol, nrow]^T (not in place). */
int kai_transpose_bin(int device, float* py, const float* px, int64_t nrow, int64_t ncol);

/* ---- parameter update: the consumers of the weight and bias gradients (next to the path) ----------- */

/* VMath::accumulate_grad, vmath.cu:364-382 (vmath.h:28).  py[n] += px[n]; sums the gradient shards of
 * data-parallel replicas (vtensor.cpp:433-475). */
int kai_accumulate_grad(int device, float* py, const float* px, int64_t nrow);
/* VMath::subtract_param_grad, vmath.cu:385-404 (vmath.h:29).  pp[n] -= pg[n] * learningRate; the
 * reference runs it on the host only (voptimizer.cpp:524,538), this entry point keeps the update on
 * the device. */
int kai_subtract_param_grad(int device, float* pp, const float* pg, int64_t nrow, const float* hLearningRate);
/* VMath::apply_decay, vmath.cu:408-444 (vmath.h:30).  pd = pg + l2 * pp + l1 * sign(pp), each term only
 * for a positive coefficient. */
int kai_apply_decay(int device, float* pd, const float* pp, const float* pg, int64_t nrow, const float* hL1Decay,
                    const float* hL2Decay);
/* VMath::eval_adam_delta, vmath.cu:449-490 (vmath.h:31).  One Adam step: ps, pt (moments) and pn (step
 * count, a float tensor) are updated in place, pa receives sterm / (sqrt(tterm) + epsilon).  All five tensors
 * hold nrow elements, pn included: the reference keeps one step count per parameter element (pn[n] += 1). */
int kai_eval_adam_delta(int device, float* pa, const float* pg, float* ps, float* pt, float* pn, int64_t nrow,
                        const float* hRo1, const float* hRo2, const float* hEpsilon);

/* Attention for forward-only use in one launch: py[nbat, ntimes, nhead*npiece] =
 * mix_values(softmax_direct_on_axis(mask(mult_on_heads(K, Q, coef))), V), i.e. the middle of
 * VTensor::mh_attention (vtensor.cpp:3036-3043), without materialising the
 * [nbat, ntimes, ntimes, nhead] tensor (training needs that tensor and keeps the separate calls).
 * masked != 0 applies the causal mask of set_mh_attention_mask.  Head sizes that are multiples of 16 up to 128 with
 * nhead * npiece == nvec and 16-byte aligned operands run fused; any other shape runs the four separate kernels with the
 * probabilities in the library's scratch memory.  The softmax is renormalised tile by tile, so the
 * result equals the separate calls up to rounding. */
int kai_attention_forward(int device, float* py, const float* pQ, const float* pK, const float* pV, int64_t nbat,
                          int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece, const float* hCoef,
                          int masked);

/* No counterpart in the reference.  Writes into `out` how the attention entry points would run this geometry with
 * 16-byte aligned operands, as text: which = 0 kai_attention_forward ("fused" or "separate"), 1
 * kai_attention_forward_train ("fused", "fused, four heads per workgroup" or "separate"), 2 kai_attention_backward
 * ("fused rows and value gradient in one launch", "fused rows + value gradient" (two launches) or "separate"), 3
 * kai_mix_values_backward_value, also the value gradient inside kai_attention_backward ("streamed, one head per
 * workgroup", "streamed, four heads per workgroup" or "tiled"), 4 kai_mix_values and kai_mult_on_heads_backward
 * ("streamed, four heads per workgroup" or "tiled").
 * Host arithmetic only, nothing is launched and no GPU is needed.
 * For maintainers and tests. */
int kai_attention_plan(int which, int64_t nbat, int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece, char* out,
                       int buflen);

/* The same block for training: pp[nbat, ntimes, ntimes, nhead] also receives the probabilities, as the separate
 * calls leave them (masked keys exactly 0), for the backward pass (VTensor::mh_attention keeps them,
 * vtensor.cpp:3005, 3048).  One launch for head sizes that are multiples of 16 up to 128 with nhead * npiece == nvec, 16-byte aligned
 * operands and ntimes <= 1024 (a wave keeps the scores of its queries in registers between the maximum and the
 * stores); any other shape runs the four separate kernels, and so do geometries with more than 512 keys, one head
 * per workgroup and workgroups for at most half of the compute units, where those kernels are the faster ones
 * (kai_attention_plan tells).  Equal to the separate calls up to rounding. */
int kai_attention_forward_train(int device, float* py, float* pp, const float* pQ, const float* pK, const float* pV,
                                int64_t nbat, int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece,
                                const float* hCoef, int masked);

/* The backward middle of the same block in one or two launches: the calls of VTensor::multihead_attention_backprop between
 * the output projection and the input projections (vtensor.cpp:3145-3154),
 *   mix_values_backward_prop, mix_values_backward_value, softmax_direct_on_axis_backward,
 *   [set_mh_attention_mask(backward) when masked != 0], mult_on_heads_backward (key gradient from pQ),
 *   mult_on_heads_backward (query gradient from pK),
 * without the [nbat, ntimes, ntimes, nhead] gradient of the probabilities reaching memory.  The reference indexes
 * that gradient by the output row for the key and the query gradient alike (vmath.cu:6790-6797); this entry point
 * follows it as written.  pgm: gradient of the mixed output; pp: the probabilities the forward pass kept; pm: the
 * mixed output of the forward pass (the engine keeps it, vtensor.cpp:3050), or null -- with it the softmax
 * derivative's row sum is one dot product (sum_k P*gP = sum_d gM*M), without it a first pass over the keys forms
 * it.  Outputs: pgQ, pgK, pgV, each [nbat, ntimes, nvec].  Head sizes that are multiples of 16 up to 128 with
 * nhead * npiece == nvec and 16-byte aligned operands run fused -- the value gradient as further workgroups of the
 * same launch with one head and a length in whole fours, or head counts in whole fours with head sizes up to 64
 * (lengths from 32 on), otherwise in a launch of its own; any other
 * shape runs the six calls with the gradient of the probabilities in the library's scratch memory.  Results equal
 * the separate calls up to the order of the sums. */
int kai_attention_backward(int device, float* pgQ, float* pgK, float* pgV, const float* pgm, const float* pp,
                           const float* pm, const float* pQ, const float* pK, const float* pV, int64_t nbat,
                           int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece, const float* hCoef,
                           int masked);

#ifdef __cplusplus
}
#endif
#endif
