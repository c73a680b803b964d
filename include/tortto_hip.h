/*
 * libtortto_hip.so -- C ABI of the MI355X (gfx950) convolution / BatchNorm path for tortto.
 *
 * The reference (samrere/pytortto 1.3.4) is pure Python: its GPU backend is "the same NumPy
 * expression executed by CuPy".  The functions below are what a native backend for that path
 * binds instead; each one names the reference call site it replaces
 * (paths relative to the reference's src/tortto/).
 *
 * Conventions
 *   - every function returns 0 on success, non-zero on failure; tt_last_error() then holds a
 *     message.  Nothing throws or aborts across this boundary.
 *   - all tensor pointers are DEVICE pointers to C-contiguous float32 NCHW data unless a
 *     parameter is documented as a host pointer.  Outputs are caller-allocated.
 *   - tensor pointers of the convolution, BatchNorm, pooling and elementwise entry points must be
 *     16-byte aligned (the kernels use 16-byte vector accesses; tt_malloc blocks are 256-byte
 *     aligned); a misaligned pointer is refused with an error.  Exception: x and dy of
 *     tt_conv2d_wgrad_f32 may have any 4-byte alignment (it falls back to scalar fetches).
 *   - kernels are enqueued on one library-owned HIP stream and return immediately;
 *     tt_sync() / tt_memcpy_d2h() wait for them.  Calls may come from several threads: one lock
 *     inside the library serialises them (allocator, workspace and table caches are shared), and
 *     work enqueued by different threads runs in the order the calls took the lock.
 *   - tensor sizes: the convolution kernels index with 32-bit element offsets, so one image
 *     ([C, H, W] resp. [K, P, Q]) and the weights must each stay below 2^31 elements; a batch
 *     whose tensors have 2^31 elements or more is cut into runs of images inside the library
 *     (forward, input gradient: one set of launches per run; weight gradient: one set of partial
 *     sums per run, added by the one reduce kernel).  BatchNorm and the elementwise kernels use
 *     64-bit offsets; BatchNorm needs a channel's N*HW values and an image's C*HW below 2^31.
 *     Pooling, the classifier head and the spatial extents (< 16384) keep 32-bit limits and
 *     reject what exceeds them.
 */
#ifndef TORTTO_HIP_H
#define TORTTO_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- runtime: device, memory, stream (replaces cupy.ndarray allocation, cparray(x) H2D and
 *      x.get() D2H at autograd/grad_fcn.py:859-865, :873-877; nn/modules/module.py:108-122) ---- */

const char* tt_last_error(void);
int tt_init(int device);
/* name: host buffer of name_len bytes; the other outputs are host pointers and may be NULL. */
int tt_device_info(char* name, int name_len, int* compute_units, int* clock_khz,
                   int* lds_bytes_per_block, size_t* total_mem_bytes);
int tt_malloc(void** ptr, size_t bytes);      /* pooled: freed blocks are reused by size class */
int tt_free(void* ptr);
int tt_empty_cache(void);                     /* return pooled blocks and the workspace to HIP */
int tt_mem_stats(size_t* bytes_in_use, size_t* bytes_pooled, size_t* workspace_bytes);
int tt_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes);   /* synchronous */
int tt_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes);   /* synchronous */
int tt_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes);    /* stream-ordered */
int tt_memset(void* dst_dev, int byte_value, size_t bytes);             /* stream-ordered */
int tt_sync(void);

/* HIP events on the library stream, for timing kernels from the host side. */
int tt_event_create(void** event);
int tt_event_record(void* event);
int tt_event_elapsed_ms(void* start, void* stop, float* ms);   /* waits for `stop` */
int tt_event_destroy(void* event);

/* ---- measurement instrumentation: per-kernel timing and calibration probes.  Used by bench.py
 *      only; a binding of the convolution / BatchNorm path needs nothing from this section. ---- */

/* Per-kernel timing (no counterpart in the reference).  While enabled, the library brackets
 * each launch of its main kernels with HIP events on its stream; tt_profile_read() waits for
 * the stream and returns the number of launches and their summed duration since
 * tt_profile_enable(1).  Event records between kernels cost a few microseconds each, so
 * whole-job throughput is measured with profiling off. */
enum {
  TT_PROF_CONV_IGEMM_FWD = 0,   /* igemm_f32 launched by tt_conv2d_fwd_f32 */
  TT_PROF_CONV_IGEMM_DGRAD = 1, /* igemm_f32 launched by tt_conv2d_dgrad_f32 (all parity classes) */
  TT_PROF_CONV_WGRAD = 2,       /* wgrad_f32 */
  TT_PROF_CONV_WGRAD_REDUCE = 3,
  TT_PROF_CONV_PREP = 4,        /* weight repack + reduction-index table kernels */
  TT_PROF_BN_FWD_REDUCE = 5,
  TT_PROF_BN_FWD_APPLY = 6,
  TT_PROF_BN_BWD_REDUCE = 7,
  TT_PROF_BN_BWD_APPLY = 8,
  TT_PROF_MAXPOOL_FWD = 9,
  TT_PROF_MAXPOOL_BWD = 10,
  TT_PROF_COUNT = 11
};
int tt_profile_enable(int on);
int tt_profile_read(int kernel_id, long long* launches, double* total_ms);

/* Calibration probes (no counterpart in the reference; measurement only): what the device sustains
 * with nothing else in the way.  tt_probe_mfma_f32 runs `launches` back-to-back launches (about 1.3 ms each)
 * of dense v_mfma_f32_32x32x2_f32 with per-lane varying operands and reports TFLOP/s (host
 * pointers); tt_probe_hbm_f32 streams `bytes` (>= 64 MiB) with 16 KiB contiguous chunks per
 * block: read-only GB/s and copy GB/s (read + written bytes). */
int tt_probe_mfma_f32(int launches, double* tflops_mean, double* tflops_min, double* tflops_max);
int tt_probe_hbm_f32(size_t bytes, double* read_gbs, double* copy_gbs);

/* ---- convolution ------------------------------------------------------------------------- */

/* Matrix arithmetic of the three convolution passes (no counterpart in the reference,
 * whose path is float32 throughout).  TT_CONV_MATH_F32 (the default) multiplies in float32 on
 * v_mfma_f32_32x32x2_f32 and is the mode that meets the reference's tolerances.
 * TT_CONV_MATH_BF16 is the optional reduced-precision variant: tensors stay float32 in memory,
 * both operands are rounded to bfloat16 (nearest even) on their way into
 * v_mfma_f32_32x32x16_bf16 and products are accumulated in float32 (the weight gradient's
 * partial sums are still combined in float64); results differ from the float32 ones by about
 * 2^-8 of the operands' magnitude per term.
 * TT_CONV_MATH_BF16X3 is float32 arithmetic on the bf16 matrix pipe, which is sixteen times as wide
 * as the float32 one: inside the kernel every operand element becomes three bfloat16 terms that add
 * up to it exactly (each the bf16 nearest to what the terms before it leave), and six
 * v_mfma_f32_32x32x16_bf16 per product step accumulate in float32 every product of terms except the
 * three smallest, which together stay below 2^-24 of the product (2^-27 in the root mean square):
 * no more than rounding the product to float32 once.  Results meet the same tolerances as TT_CONV_MATH_F32 (they differ from it as two
 * float32 summation orders do); non-finite operands and magnitudes above 3.38e38 (which round to a
 * bf16 infinity) give NaN where float32 would give an infinity.  Forward and input gradient run
 * that way for every geometry; the weight gradient keeps the float32 instructions (its loop is bound
 * by streaming x and dy through LDS, and three-term variants of it measured no faster).
 * The modes apply to tt_conv2d_fwd_f32,
 * tt_conv2d_dgrad_f32 and tt_conv2d_wgrad_f32.  The setting is process-wide and applies to
 * later calls of every caller; the *_bf16 and *_bf16x3 entry points below select a mode per call
 * instead. */
enum { TT_CONV_MATH_F32 = 0, TT_CONV_MATH_BF16 = 1, TT_CONV_MATH_BF16X3 = 2 };
int tt_set_conv_math(int mode);
int tt_get_conv_math(int* mode);   /* host pointer */
/* The same passes with bf16 (*_bf16) or three-term (*_bf16x3: forward and input gradient) matrix
 * arithmetic for one call, whatever the process-wide mode is (arguments as tt_conv2d_fwd_f32 /
 * tt_conv2d_dgrad_f32 / tt_conv2d_wgrad_f32 below; tensors are float32): for callers that must not
 * change what other callers of the library compute. */
int tt_conv2d_fwd_bf16(const float* x, const float* w, const float* bias, float* y,
                       int N, int C, int H, int W, int K, int R, int S,
                       int sh, int sw, int ph, int pw, int dh, int dw, int groups);
int tt_conv2d_dgrad_bf16(const float* dy, const float* w, const float* bias, float* dx,
                         int N, int C, int Hx, int Wx, int K, int R, int S,
                         int sh, int sw, int ph, int pw, int dh, int dw, int groups, int P, int Q);
int tt_conv2d_wgrad_bf16(const float* x, const float* dy, float* dw,
                         int N, int C, int H, int W, int K, int R, int S,
                         int sh, int sw, int ph, int pw, int dh, int dw_, int groups, int P, int Q);
int tt_conv2d_fwd_bf16x3(const float* x, const float* w, const float* bias, float* y,
                         int N, int C, int H, int W, int K, int R, int S,
                         int sh, int sw, int ph, int pw, int dh, int dw, int groups);
int tt_conv2d_dgrad_bf16x3(const float* dy, const float* w, const float* bias, float* dx,
                           int N, int C, int Hx, int Wx, int K, int R, int S,
                           int sh, int sw, int ph, int pw, int dh, int dw, int groups, int P, int Q);


/* Tuning threshold of tt_conv2d_dgrad_f32 for strided layers with very few input channels (the
 * ResNet stem, the output layer of a transposed generator), no counterpart in the reference.
 * Such launches stack the pixel classes of a cell of the output (one period of the stride
 * pattern, or two / four periods side by side) as rows of one matrix product; a larger cell
 * wastes fewer multiplications but leaves fewer tiles.  A larger cell is taken only while at
 * least `tiles` tiles of 256 cells remain (default 1.5 per compute unit, 384 on an MI355X; 0 =
 * always, which lets small inputs reach the larger cells; -1 = back to the default).  Results do
 * not depend on it beyond summation order.  Process-wide, applies to later calls. */
int tt_set_conv_dense_cell_min_tiles(int tiles);

/* y[N,K,P,Q] = conv(x[N,C,H,W], w[K,C/groups,R,S]) (+ bias[K] if not NULL).
 * Replaces _padding + _sliding_window_view + einsum and the bias add:
 * autograd/grad_nn.py:595-643 (called from :709-711).
 * P = floor((H + 2*ph - dh*(R-1) - 1)/sh) + 1, likewise Q (grad_nn.py:565-566). */
int tt_conv2d_fwd_f32(const float* x, const float* w, const float* bias, float* y,
                      int N, int C, int H, int W, int K, int R, int S,
                      int sh, int sw, int ph, int pw, int dh, int dw, int groups);

/* dx[N,C,Hx,Wx] = sum over k,r,s of dy[N,K,P,Q] * w[K,C/groups,R,S] (+ bias[C] if not NULL):
 * the input gradient of the convolution above, and -- with x as `dy`, the [C_in,C_out/g,R,S]
 * transposed-convolution weight as `w`, K = C_in, C = C_out -- the forward pass of
 * ConvTranspose2d.  Hx, Wx are explicit so that output_padding and rows the forward pass
 * never covered (zero-filled) are handled.  Replaces _dilate + flip + _padding + einsum + crop
 * + pad: autograd/grad_nn.py:659-682 (called from :733 and :755-757). */
int tt_conv2d_dgrad_f32(const float* dy, const float* w, const float* bias, float* dx,
                        int N, int C, int Hx, int Wx, int K, int R, int S,
                        int sh, int sw, int ph, int pw, int dh, int dw, int groups,
                        int P, int Q);

/* dw[K,C/groups,R,S] = sum over n,p,q of x~[n,c,p*sh+r*dh-ph,q*sw+s*dw-pw] * dy[n,k,p,q]
 * (x~ = x zero-padded).  Deterministic: fixed split of the reduction, partial sums combined
 * in float64.  Replaces _conv2d_backward_w: autograd/grad_nn.py:646-656 (called from :731
 * and, with the roles of x and dy exchanged by the caller, :776).
 * P, Q are the spatial size of dy; they may be smaller than the geometry's output size (the
 * reference crops x~ to the rows the windows cover, :653-655) but not larger: a dy that does not
 * belong to the geometry is refused. */
int tt_conv2d_wgrad_f32(const float* x, const float* dy, float* dw,
                        int N, int C, int H, int W, int K, int R, int S,
                        int sh, int sw, int ph, int pw, int dh, int dw_, int groups,
                        int P, int Q);

/* Host-only checks of the index tables behind tt_conv2d_fwd_f32 / tt_conv2d_dgrad_f32 /
 * tt_conv2d_wgrad_f32 (no
 * counterpart in the reference; no device is needed and tt_init() need not have been called).
 * The kernels turn a reduction index (c, r, s) -- (k, tap row, tap column) for the input gradient
 * -- into an address through small per-geometry tables, which the library builds on the host,
 * checks once per new geometry and keeps in device buffers of their own.  These calls run exactly
 * that planning and check for a geometry without launching anything: every table entry, replayed
 * for the extreme pixels under the kernel's own bounds rule, must address the element of x (dy)
 * that autograd/grad_nn.py:603-611 (:659-682) pairs with that reduction index, inside the tensor.
 * The weight gradient's table has one entry per output pixel (image, offsets of the pixel in dy
 * and of its window in x, one bit per tap that falls into the padding); every entry is checked:
 * the dy element and, tap by tap, the x element it leads to must be the ones
 * autograd/grad_nn.py:646-656 pairs, inside the tensors, and a tap is blocked exactly when it lies
 * in the padding.
 * tt_conv2d_check_tables_selftest / _selftest_wgrad damage single entries and return 0 when the
 * check refuses each damaged table. */
int tt_conv2d_check_tables_fwd_f32(int N, int C, int H, int W, int K, int R, int S,
                                   int sh, int sw, int ph, int pw, int dh, int dw, int groups);
int tt_conv2d_check_tables_dgrad_f32(int N, int C, int Hx, int Wx, int K, int R, int S,
                                     int sh, int sw, int ph, int pw, int dh, int dw, int groups,
                                     int P, int Q);
int tt_conv2d_check_tables_wgrad_f32(int N, int C, int H, int W, int K, int R, int S,
                                     int sh, int sw, int ph, int pw, int dh, int dw_, int groups,
                                     int P, int Q);
int tt_conv2d_check_tables_selftest(void);
int tt_conv2d_check_tables_selftest_wgrad(void);

/* Instrumentation of the convolution launches (tests only; no counterpart in the reference).
 * Layers whose tile count loads the compute units unevenly run as one persistent grid of two
 * blocks per compute unit (three with bf16 arithmetic) whose blocks hand partial sums to each
 * other; that is safe only while the whole grid is resident, so the library asks the device how
 * many blocks of each such kernel a compute unit holds and launches one tile per block instead
 * where it is too few.
 *   tt_conv2d_stream_k_blocks_per_cu: the smallest answer over all such kernels of one matrix
 *     arithmetic (bf16 = 0: float32 instructions, 1: TT_CONV_MATH_BF16, 3: TT_CONV_MATH_BF16X3, which
 *     like the float32 ones runs two blocks per compute unit; host pointer).
 *   tt_conv2d_stream_k_force_occupancy: pretend the answer is `blocks` (-1: ask the device).
 *   tt_conv2d_selftest_raise_async_error: a one-thread kernel sets the word that a block sets when
 *     its bounded wait for another block runs out; the next tt_sync() / tt_memcpy_d2h() returns
 *     the error, once.  Nothing waits and nothing fails on the device.
 *   tt_conv2d_images_per_run (host-only): images per run when a batch of N images of image_a
 *     (input) and image_b (output) elements is cut into runs below 2^31 elements; every run starts
 *     16-byte aligned; 0 = impossible (the call itself then returns an error). */
int tt_conv2d_stream_k_blocks_per_cu(int bf16, int* blocks);
int tt_conv2d_stream_k_force_occupancy(int blocks);
int tt_conv2d_selftest_raise_async_error(void);
int tt_conv2d_images_per_run(int N, long long image_a, long long image_b, int* per);
/* The plan of the last single matrix-product launch made by tt_conv2d_fwd_f32 / _dgrad_f32 (host
 * pointer to 8 ints): tile rows, tile columns (pixels), tiles, row tiles, blocks of the persistent
 * grid (0 = one tile per block, -1 = one tile per block on the bf16-first kernels), tiles computed
 * whole, blocks sharing the remaining tiles'
 * reductions, addressing mode | terms << 8 with terms = bf16 terms per operand element of the matrix
 * instructions used (0 = float32 instructions, 1 = TT_CONV_MATH_BF16, 3 = TT_CONV_MATH_BF16X3).
 * Tests use it to compare the images where the shared tiles begin. */
int tt_conv2d_last_launch(int* plan8);
/* The same for the weight gradient, whose blocks add each other's partial sums inside the kernel
 * when the device holds the whole grid at once and leave them to a second kernel otherwise:
 *   tt_conv2d_last_wgrad_launch: {tiles, reduction splits, 1 if added inside the kernel, partial-sum
 *     slots} of the last launch (host pointer to 4 ints);
 *   tt_conv2d_wgrad_force_occupancy: pretend the device holds `blocks` blocks per compute unit
 *     (-1: ask the device). */
/* tt_conv2d_bf16_first_enable: with TT_CONV_MATH_BF16 selected, forward and stride-1 input-gradient
 * launches go to kernels built around the bf16 matrix instruction (operands converted on their way
 * into LDS, 32-deep chunks) when they have at least one tile per compute unit or a reduction of at
 * most 1024 (1, the default) or whenever those kernels support the geometry (2: small test shapes);
 * 0 keeps every launch on the float32 kernels' bf16 instantiations, which also serve the launches
 * the former do not take.  Both compute the same thing: the convolution of
 * the bf16-rounded operands in float32. */
int tt_conv2d_bf16_first_enable(int on);
int tt_conv2d_last_wgrad_launch(int* plan4);
int tt_conv2d_wgrad_force_occupancy(int blocks);

/* out[K] = sum over n and the HW plane of t[N,K,HW]: the bias gradient gd0.sum((0,2,3)),
 * autograd/grad_nn.py:728, :774. */
int tt_channel_sum_f32(const float* t, float* out, int N, int K, int HW);

/* ---- BatchNorm (x viewed as [N, C, HW]) ---------------------------------------------------- */

/* Training forward, autograd/grad_nn.py:921-930 and :942-959:
 *   mean/var(biased) over (n,hw); save_mean[C], save_var_eps[C] = var+eps, save_sd[C] = sqrt(var+eps);
 *   y = (x-mean)/sd*gamma+beta (gamma, beta may be NULL);
 *   if running_mean_in/var_in are not NULL:
 *     running_mean_out = (1-momentum)*running_mean_in + momentum*mean
 *     running_var_out  = (1-momentum)*running_var_in  + momentum*var*(M/(M-1)),  M = N*HW
 *   (in/out may alias).  num_batches_tracked (one float, may be NULL) is incremented by one: the
 *   module's `self.num_batches_tracked.data += 1` (nn/modules/batchnorm.py:66) without a launch of
 *   its own.  Returns an error when M == 1 (grad_nn.py:899-904). */
int tt_bn_fwd_train_f32(const float* x, const float* gamma, const float* beta, float* y,
                        float* save_mean, float* save_var_eps, float* save_sd,
                        const float* running_mean_in, const float* running_var_in,
                        float* running_mean_out, float* running_var_out, float* num_batches_tracked,
                        double momentum, double eps, int N, int C, int HW);

/* tt_bn_fwd_train_f32 for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same
 * arguments, same kernels and bit-identical results, but the first sweep's per-channel partial
 * moments go to a fixed 256 KiB array in the library's device image instead of the workspace that
 * grows on demand, launches are never bracketed for tt_profile_read, and the call makes no
 * hipMalloc / hipFree / event creation.  Limit: tt_workspace_size_bn_f32(...) <= 262144 bytes
 * (16384 partial moments; every tensor of at most 2^29 elements fits); beyond that the call fails
 * with a message and launches nothing.  All calls on one device share the array: it needs no
 * clearing between calls (every slot read was written by the same call), but calls that overlap on
 * one device race.  tt_init() looks the array's device address up once per device. */
int tt_bn_fwd_train_noalloc_f32(const float* x, const float* gamma, const float* beta, float* y,
                                float* save_mean, float* save_var_eps, float* save_sd,
                                const float* running_mean_in, const float* running_var_in,
                                float* running_mean_out, float* running_var_out,
                                float* num_batches_tracked,
                                double momentum, double eps, int N, int C, int HW);

/* Normalisation with given statistics (eval mode), autograd/grad_nn.py:931-959:
 * save_* are written from mean[C]/var[C] exactly as in training so that backward can follow. */
int tt_bn_fwd_eval_f32(const float* x, const float* gamma, const float* beta, float* y,
                       const float* mean, const float* var,
                       float* save_mean, float* save_var_eps, float* save_sd,
                       double eps, int N, int C, int HW);

/* Backward, autograd/grad_nn.py:966-989.  dx, dgamma, dbeta may each be NULL (not needed):
 *   dbeta = sum dy; dgamma = sum dy*(x-mean)/sd;
 *   dx = ((M*g - sum g) - (x-mean)/var_eps * sum(g*(x-mean))) / M / sd,  g = dy*gamma. */
int tt_bn_bwd_f32(const float* x, const float* dy, const float* gamma,
                  const float* save_mean, const float* save_var_eps, const float* save_sd,
                  float* dx, float* dgamma, float* dbeta, int N, int C, int HW);

/* BatchNorm followed by ReLU in one pass each way (no single counterpart in the reference, which
 * runs BatchNorm, autograd/grad_nn.py:921-959 and :966-989, and Relu, :56-67, as separate array
 * expressions; the two autograd nodes stay separate on the host side).
 * tt_bn_relu_fwd_train_f32: tt_bn_fwd_train_f32 whose output is y = maximum(bn(x), 0), NaN kept;
 * the normalised values themselves are not stored (the backward pass needs x and the statistics,
 * the ReLU's backward its own output).
 * tt_bn_relu_bwd_f32: tt_bn_bwd_f32 on the gradient g = dy * (relu_y > 0), formed as dy is read in
 * both sweeps instead of by a kernel of its own; relu_y is the output of the forward call. */
int tt_bn_relu_fwd_train_f32(const float* x, const float* gamma, const float* beta, float* y,
                             float* save_mean, float* save_var_eps, float* save_sd,
                             const float* running_mean_in, const float* running_var_in,
                             float* running_mean_out, float* running_var_out, float* num_batches_tracked,
                             double momentum, double eps, int N, int C, int HW);
int tt_bn_relu_bwd_f32(const float* x, const float* dy, const float* relu_y, const float* gamma,
                       const float* save_mean, const float* save_var_eps, const float* save_sd,
                       float* dx, float* dgamma, float* dbeta, int N, int C, int HW);

/* ---- workspace queries (no counterpart in the reference) -------------------------------------- */

/* Bytes of library workspace (repacked weights, index tables, partial sums) the corresponding call
 * asks for with the same geometry arguments; the library grows its workspace to the largest
 * request seen.  Same argument checks as the calls; nothing is launched or allocated.  The small
 * per-geometry tables the library keeps in buffers of their own (index tables of a few KB, 16 bytes
 * per output pixel for the weight gradient; released by tt_empty_cache) are not included. */
int tt_workspace_size_conv2d_fwd_f32(size_t* bytes, int N, int C, int H, int W, int K, int R, int S,
                                     int sh, int sw, int ph, int pw, int dh, int dw, int groups);
int tt_workspace_size_conv2d_dgrad_f32(size_t* bytes, int N, int C, int Hx, int Wx, int K, int R, int S,
                                       int sh, int sw, int ph, int pw, int dh, int dw, int groups, int P, int Q);
int tt_workspace_size_conv2d_wgrad_f32(size_t* bytes, int N, int C, int H, int W, int K, int R, int S,
                                       int sh, int sw, int ph, int pw, int dh, int dw, int groups, int P, int Q);
int tt_workspace_size_bn_f32(size_t* bytes, int N, int C, int HW);   /* training forward and backward alike */

/* ---- MaxPool2d (autograd/grad_nn.py:784-864) ------------------------------------------------ */

/* x: [NC, H, W] planes (N*C of them), y and tap: [NC, P, Q].  Windows are taken over x padded
 * with -inf (padding ph/pw; taps beyond the bottom/right edge, as ceil_mode produces, read -inf
 * too); NaN is ignored, the first maximum in (kernel row, kernel column) order wins and `tap`
 * receives kernel_row * kw + kernel_column (_max_pool2d, :784-808; the reference's `pos` tuple
 * holds the same two indices).  P and Q are chosen by the caller (floor or ceil rule, :566-579);
 * every window must start inside the input or its top/left padding. */
int tt_maxpool2d_fwd_f32(const float* x, float* y, int* tap, int NC, int H, int W, int P, int Q,
                         int kh, int kw, int sh, int sw, int ph, int pw, int dh, int dw);
/* dx[NC, H, W] from dy[NC, P, Q] and the forward's `tap` (_max_pool2d_backward, :811-824): each
 * output gradient is ASSIGNED to its window's arg-max pixel; when overlapping windows chose the
 * same pixel the last window in (p, q) order wins, as NumPy's indexed assignment does -- the
 * reference does not sum them.  Pixels no window chose receive 0. */
int tt_maxpool2d_bwd_f32(const float* dy, const int* tap, float* dx, int NC, int H, int W, int P, int Q,
                         int kh, int kw, int sh, int sw, int ph, int pw, int dh, int dw);

/* ---- classifier head: spatial mean, Linear, LogSoftmax, NLLLoss ------------------------------- */

/* y[r] = mean(x[r, 0..L)) and its gradient dx[r, i] = g[r] / L: `Mean` over trailing dimensions
 * (autograd/grad_fcn.py:1058-1093; `tt.mean(x, (-1, -2), True)` in the ResNet examples). */
int tt_mean_rows_f32(const float* x, float* y, int R, int L);
int tt_mean_rows_bwd_f32(const float* g, float* dx, int R, int L);
/* y[c, r] = x[r, c]: `Transpose` of a matrix, materialised (grad_fcn.py:752-771; `weight.T` in
 * nn/functional.py:59).  The matrix products of `Mm` (grad_fcn.py:907-932) need no entry point of
 * their own: A[M,K] @ B[K,N] is tt_conv2d_fwd_f32 on the image B = [1, K, 1, N] with the 1x1
 * weights A = [M, K, 1, 1]; G @ B^T is tt_conv2d_wgrad_f32 and A^T @ G is tt_conv2d_dgrad_f32 of
 * the same geometry. */
int tt_transpose2d_f32(const float* x, float* y, int R, int C);
/* out[r, c] = a[r, c] + v[c]: `Add` with the bias broadcast over rows (grad_fcn.py:177-203;
 * nn/functional.py:59); the bias gradient is tt_channel_sum_f32(g, db, R, C, 1). */
int tt_add_rowvec_f32(const float* a, const float* v, float* out, int R, int C);
/* Row-wise y = (x - max) - log(sum(exp(x - max))) and dx = g - sum(g) * exp(y)
 * (autograd/grad_nn.py:373-392).  A NaN in a row makes the whole row NaN, as NumPy's max does. */
int tt_log_softmax_fwd_f32(const float* x, float* y, int R, int C);
int tt_log_softmax_bwd_f32(const float* g, const float* y, float* dx, int R, int C);
/* NllLoss on logp[R, C] with int64 targets (autograd/grad_nn.py:287-349).  weight: per-class
 * weights or NULL; ignore_index acts only when >= 0, as in the reference (:301-305).
 * reduction: 0 none (out[R]), 1 sum, 2 mean (out[1]); `count` (device, 1 float) receives the
 * mean's divisor: R without weights, else the number of rows with non-zero weight (:315-319).
 * The backward takes the same `count`; g is [R] for reduction none, else one value.  Targets in
 * [-C, -1] count from the end, as the reference's NumPy indexing does; targets outside [-C, C)
 * raise IndexError in the reference: a kernel cannot raise, so such a row's loss (and a summed or
 * averaged loss with it) is NaN and its gradient row is zero. */
int tt_nll_loss_fwd_f32(const float* logp, const long long* target, const float* weight, float* out,
                        float* count, int R, int C, long long ignore_index, int reduction);
int tt_nll_loss_bwd_f32(const float* g, const long long* target, const float* weight, const float* count,
                        float* dlogp, int R, int C, long long ignore_index, int reduction);

/* ---- optimiser steps (optim/_functional.py:4-119) ---------------------------------------------- */

/* One SGD update of a parameter in place (_functional.py:4-22): d = grad (+ weight_decay * param);
 * with momentum != 0, buf = d on the first step, else buf = buf * momentum + d * (1 - dampening),
 * and d = buf (or d + buf * momentum with nesterov); param += d * (-lr).  Each product and sum is
 * rounded to float32 separately, as NumPy evaluates the reference's expressions. */
int tt_sgd_step_f32(float* param, const float* grad, float* momentum_buf, size_t n, double lr, double momentum,
                    double dampening, double weight_decay, int nesterov, int first_step);
/* The same update for `count` parameters of one group (the loop of _functional.py:5) in a few
 * launches instead of one per parameter.  The tables are host arrays; first_steps[i] != 0 marks a
 * parameter whose momentum buffer is being created by this step. */
int tt_sgd_step_multi_f32(int count, float* const* params, const float* const* grads, float* const* momentum_bufs,
                          const size_t* sizes, const int* first_steps, double lr, double momentum, double dampening,
                          double weight_decay, int nesterov);
/* One Adam (_functional.py:25-65) or AdamW (decoupled_weight_decay != 0, :68-119) update in place;
 * `step` counts from 1; max_exp_avg_sq only with amsgrad.  The moments are float32 with separate
 * roundings; the denominator sqrt(v) / sqrt(1 - beta2^step) + eps and the final update are
 * float64, as the reference's mixed float32-array / float64-scalar expressions evaluate. */
int tt_adam_step_f32(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, float* max_exp_avg_sq,
                     size_t n, int step, double lr, double beta1, double beta2, double eps, double weight_decay,
                     int amsgrad, int decoupled_weight_decay);
/* The same for `count` parameters of one group in a few launches; steps[i] is each parameter's own
 * step count (adam.py:60-63). */
int tt_adam_step_multi_f32(int count, float* const* params, const float* const* grads, float* const* exp_avgs,
                           float* const* exp_avg_sqs, float* const* max_exp_avg_sqs, const size_t* sizes,
                           const int* steps, double lr, double beta1, double beta2, double eps, double weight_decay,
                           int amsgrad, int decoupled_weight_decay);

/* ---- elementwise glue so whole stacks stay on the device ----------------------------------- */

/* y = max(x, 0) (autograd/grad_nn.py:33-69); dx = dy * (y > 0). */
int tt_relu_fwd_f32(const float* x, float* y, size_t n);
int tt_relu_bwd_f32(const float* dy, const float* y, float* dx, size_t n);
/* y = maximum(x * negative_slope, x); dx = dy where x >= 0 (or NaN), dy * negative_slope where
 * x < 0 (autograd/grad_nn.py:71-95).  dx may alias dy: the reference scales the incoming
 * gradient array in place (:94). */
int tt_leaky_relu_fwd_f32(const float* x, float* y, float negative_slope, size_t n);
int tt_leaky_relu_bwd_f32(const float* dy, const float* x, float* dx, float negative_slope, size_t n);
/* out = a + b (residual Add, autograd/grad_fcn.py:177-203). */
int tt_add_f32(const float* a, const float* b, float* out, size_t n);
/* out = maximum(a + b, 0): the residual Add (grad_fcn.py:177-203) with the ReLU behind it
 * (autograd/grad_nn.py:56) in one pass; bit-identical to tt_add_f32 followed by tt_relu_fwd_f32. */
int tt_add_relu_f32(const float* a, const float* b, float* out, size_t n);
/* acc += alpha * v: gradient accumulation `fn.grad[ind] += grad` (tensor.py:596-599,
 * autograd/function.py:88-93). */
int tt_axpy_f32(float alpha, const float* v, float* acc, size_t n);
/* acc[i] += value (a Python scalar added in place, e.g. `num_batches_tracked.data += 1`,
 * nn/modules/batchnorm.py:66). */
int tt_add_scalar_f32(float* acc, float value, size_t n);
/* dst[i] = value */
int tt_fill_f32(float* dst, float value, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* TORTTO_HIP_H */
