/*
 * cnet_hip.h - C ABI of the MI355X (gfx950) device layer for CNet's dense complex-valued hot path.
 *
 * This library takes the place of the device layer of upstream CNet: the CUDA kernels and host launchers in
 * gpu/kernels.cpp, gpu/reduce.cpp, gpu/reducegrad.cpp and the allocator in gpu/allocator.h / gpu/allocator.cu.
 * Each entry point names the upstream interface it replaces (paths under the upstream tree).
 *
 * Conventions
 *  - A complex matrix is two fp32 planes (re, im), row-major, with a leading dimension in ELEMENTS (ld >= cols).
 *    One row = one sample of the batch (one upstream "clone").  Parameters are stored once (no per-sample copy).
 *  - A gradient carrier is four planes: dz_re, dz_im (dL/dz) and dzs_re, dzs_im (dL/d conj z), as in
 *    impl/vars.h:40-46 upstream.
 *  - `accumulate` != 0 adds into the destination (the upstream `+=` into zeroed planes); 0 overwrites, which saves
 *    the zero-fill and the read.
 *  - Every function returns 0 on success and a negative cnet_status otherwise; it never exits the process
 *    (upstream gpuErrchk prints and exits, gpu/kernels.h:18-28).  cnet_last_error() describes the last failure
 *    of the calling thread.
 *  - All work is queued on one HIP stream (cnet_stream()); nothing synchronises except cnet_sync(), the
 *    device-to-host copies and cnet_shutdown().  One host thread per process drives the library.
 *  - Pointers are device pointers unless the parameter name starts with host_.
 */
#ifndef CNET_HIP_H_
#define CNET_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
	CNET_OK = 0,
	CNET_ERR_NOT_INITIALIZED = -1,
	CNET_ERR_INVALID_ARGUMENT = -2,
	CNET_ERR_HIP = -3,          /* a HIP runtime call failed; text in cnet_last_error() */
	CNET_ERR_OUT_OF_MEMORY = -4,
	CNET_ERR_UNSUPPORTED = -5
} cnet_status;

typedef struct {
	char name[256];
	char arch[64];
	int compute_units;
	int clock_khz;            /* maximum engine clock */
	int wavefront_size;
	int lds_bytes_per_block;  /* largest LDS allocation one workgroup may request */
	int64_t hbm_bytes;
	double fp32_matrix_peak_tflops; /* 256 flop/clk/CU x compute_units x clock */
} cnet_device_info;

/* ---- lifetime, memory, stream: replaces GpuHelper (gpu/allocator.h:97-408, gpu/allocator.cu:4-31) ---------- */
int cnet_init(int device);                 /* select device, create the stream; idempotent */
int cnet_shutdown(void);                   /* sync, free library-owned buffers (twiddles, workspace), destroy stream */
int cnet_get_device_info(cnet_device_info *out);   /* getTotalGlobalMem / getMaxThreadsPerBlock / PrintInfo */
const char *cnet_last_error(void);
void *cnet_stream(void);                   /* the hipStream_t all launches use */
int cnet_set_stream(void *hip_stream);     /* adopt a caller-owned stream (NULL restores the library's own) */
int cnet_sync(void);
int cnet_alloc(size_t bytes, void **out);  /* float_allocate_on_gpu & friends (gpu/allocator.h:121-180) */
int cnet_free(void *ptr);
int cnet_memcpy_h2d(void *dst, const void *host_src, size_t bytes);   /* *_copy_to_gpu   (gpu/allocator.h:182-260) */
/* ---- Host batch pipeline: replaces the per-sample copies of GpuNet::batchToGpu (gpu/gpu_func.h:368-427: two pageable
 *      cudaMemcpy per sample) with page-locked [B x dim] planes, one asynchronous copy per plane, and an upload stream
 *      that runs ahead of the compute stream.
 * cnet_host_alloc / cnet_host_free: page-locked host memory (hipHostMalloc).
 * cnet_memcpy_h2d_async: copy on the compute stream, returns at once; the source must be page-locked and stay
 *      untouched until the stream reaches the copy (cnet_sync, or any later blocking call).
 * cnet_memcpy_d2h_async: the other direction on the compute stream (the per-row losses of a step, replacing the blocking
 *      read of CNet::getLoss, impl/cnet.h / gpu/gpu_func.h:928-969 upstream); the page-locked destination is valid once a
 *      ticket taken after the call has been waited for.
 * cnet_upload_async: the same on the library's upload stream, so it overlaps kernels of the compute stream.
 * cnet_upload_zero: clears device memory on the upload stream, in order with the copies queued there (the imaginary plane
 *      of a batch of real samples is cleared on the device instead of travelling as zeros).
 * cnet_upload_wait_compute: uploads queued after this call start only when everything queued on the compute stream so
 *      far has finished (call before overwriting a device buffer that kernels may still read).
 * cnet_mark_compute(m) / cnet_upload_wait_marker(m), m = 0..7: the same in two halves - remember the current tail of the
 *      compute stream under number m now, make later uploads wait for that point when a buffer is about to be refilled
 *      (buffers used in turn: the marker is set when a buffer is retired, the wait is issued when it is reused; a wait for a
 *      point that has been reached already is not queued at all).
 * cnet_compute_wait_upload: kernels queued after this call start only when every upload queued so far has landed.
 * cnet_mark_upload(m) / cnet_compute_wait_upload_marker(m), m = 0..7: the same in two halves - remember the current tail
 *      of the upload stream under number m (right after the copies of one batch were queued), make later kernels wait for
 *      that point and for nothing queued on the upload stream after it (another batch may already be travelling).
 * cnet_upload_sync: host waits for the upload stream (before reusing a page-locked source buffer).
 * cnet_copy_ticket(upload_stream, &t) / cnet_copy_wait(t): the host-side twin of the markers - t names the current tail of
 *      the compute stream (upload_stream = 0) or of the upload stream (1); cnet_copy_wait(t) blocks the host until that
 *      point has been reached and nothing later, so one page-locked buffer can be refilled while the copy out of the
 *      next one is still running.  May wait for a somewhat later point of the same stream once 32 newer tickets exist. */
int cnet_host_alloc(size_t bytes, void **host_ptr);
int cnet_host_free(void *host_ptr);
int cnet_memcpy_h2d_async(void *dst, const void *pinned_src, size_t bytes);
int cnet_memcpy_d2h_async(void *pinned_dst, const void *src, size_t bytes);
int cnet_upload_async(void *dst, const void *pinned_src, size_t bytes);
int cnet_upload_zero(void *dst, size_t bytes);
/* two regions (a batch and its labels) from page-locked memory to the device on the upload stream, sizes in bytes, multiples
 * of 4; up to 1 MiB in all they travel in ONE kernel launch whose lanes read the host memory over the link (half the
 * host time of two queued copies and none of the copy engine's start-up time), beyond that, or when a source does not lie
 * in memory from cnet_host_alloc, as two cnet_upload_async */
int cnet_upload_pair(void *dst0, const void *pinned_src0, size_t bytes0, void *dst1, const void *pinned_src1, size_t bytes1);
/* A batch out of a data set that is kept on the device, on the upload stream, in one launch:
 *   dst[p][r][0 .. cols) = src[p][idx[r]][0 .. cols)  for p < planes (1 or 2; plane p starts p * plane_stride floats in),
 *   dst_labels[r] = src_labels[idx[r]]                 when both label arrays are given (both NULL: samples only).
 * idx: `rows` int32 in memory from cnet_host_alloc, each in [0, src_rows) (checked on the host; the kernel reads them over
 * the link, 4 bytes per sample instead of the sample).  No counterpart upstream, which copies every sample of every batch
 * from host memory (gpu/gpu_func.h:403-419): with the samples resident, a batch moves at the speed of device memory. */
int cnet_upload_gather_rows(float *dst, int64_t ldd, int64_t dst_plane_stride, const float *src, int64_t lds,
                            int64_t src_plane_stride, int planes, int src_rows, const int32_t *pinned_idx,
                            int32_t *dst_labels, const int32_t *src_labels, int rows, int cols);
/* The same on the compute stream, in front of the kernels that read the batch (no hand-over between the streams: what a small
 * batch wants, whose copy is shorter than the hand-over).  Not while recording: the indices are read when the kernel runs. */
int cnet_gather_rows(float *dst, int64_t ldd, int64_t dst_plane_stride, const float *src, int64_t lds,
                     int64_t src_plane_stride, int planes, int src_rows, const int32_t *pinned_idx,
                     int32_t *dst_labels, const int32_t *src_labels, int rows, int cols);
int cnet_upload_wait_compute(void);
int cnet_mark_compute(int marker);
int cnet_upload_wait_marker(int marker);
int cnet_compute_wait_upload(void);
int cnet_mark_upload(int marker);
int cnet_compute_wait_upload_marker(int marker);
int cnet_upload_sync(void);
int cnet_copy_ticket(int upload_stream, int64_t *ticket);
int cnet_copy_wait(int64_t ticket);
/* kernels queued after this call start only when the point of the upload stream that ticket t names has been reached: one
 * recorded point then serves the host (cnet_copy_wait) and the compute stream, instead of a ticket and a marker */
int cnet_compute_wait_ticket(int64_t ticket);

/* ---- Graphs: a training step at small batch sizes is bound by launch overhead (upstream pays a cudaDeviceSynchronize
 *      per layer on top, gpu/kernels.cpp:104-105).  Between cnet_graph_begin and cnet_graph_end the layer entry points
 *      record their kernels on the library's stream instead of running them; cnet_graph_launch replays the recording
 *      with one call.  Pointers, shapes and scalars (learning rate, accumulate flags) are frozen into the recording.
 *      Entry points that allocate, wait or order the two streams (cnet_alloc, cnet_free, cnet_sync, the blocking copies,
 *      the marker / wait calls of the upload stream, the first use of a DFT length or of a larger workspace) return CNET_ERR_UNSUPPORTED while recording, and cnet_graph_end then fails:
 *      run the sequence once before recording it.  Clearing memory inside a recording uses a fill kernel
 *      (cnet_memset_zero), never a memset node.  While a recording exists, a library workspace that has to grow for a
 *      later call is kept instead of freed, so the recording stays valid. */
int cnet_graph_begin(void);
int cnet_graph_end(void **graph_exec);      /* NULL: drop the recording */
int cnet_graph_launch(void *graph_exec);
int cnet_graph_destroy(void *graph_exec);
int cnet_memcpy_d2h(void *host_dst, const void *src, size_t bytes);   /* *_copy_from_gpu (gpu/allocator.h:262-328); synchronises */
int cnet_memcpy_d2d(void *dst, const void *src, size_t bytes);
int cnet_memset_zero(void *dst, size_t bytes);  /* GpuMapping::zeroGradients (gpu/kernels.cpp:444-469) */

/* ---- complex GEMM core -------------------------------------------------------------------------------------
 * C[M x N] (+)= op(A)[M x K] * op(B)[K x N], complex, fp32 MFMA, four real products per complex product.
 *   a_kmajor = 0: A stored [M][lda] (k contiguous)      1: A stored [K][lda] (m contiguous, i.e. A^T in memory)
 *   b_kmajor = 0: B stored [N][ldb] (k contiguous)      1: B stored [K][ldb] (n contiguous)
 *   conj_b  != 0: use conj(B).
 * The layer entry points below are thin shape adapters over this one.  No upstream counterpart (upstream has
 * no GEMM: one thread per multiply and a shared-memory tree, gpu/reduce.cpp:100-158). */
int cnet_cgemm(int a_kmajor, int b_kmajor, int conj_b, int M, int N, int K,
               const float *a_re, const float *a_im, int64_t lda,
               const float *b_re, const float *b_im, int64_t ldb,
               float *c_re, float *c_im, int64_t ldc, int accumulate);

/* Strided batch of the same product: matrix z of the batch starts z * stride_x elements after matrix 0 (stride 0 = the
 * operand is shared by the whole batch); conj_a != 0 uses conj(A).  Used for a transform applied along an inner axis,
 * e.g. a DFT along the sequence axis of [batch][seq][dim] activations: C_z = F * X_z and, backwards, conj(F) * G*_z. */
int cnet_cgemm_batched(int a_kmajor, int b_kmajor, int conj_a, int conj_b, int M, int N, int K,
                       const float *a_re, const float *a_im, int64_t lda, int64_t stride_a,
                       const float *b_re, const float *b_im, int64_t ldb, int64_t stride_b,
                       float *c_re, float *c_im, int64_t ldc, int64_t stride_c, int batch, int accumulate);

/* ---- Linear: replaces LinearGpu::gpu_linear_forward / gpu_linear_backward
 *      (gpu/reduce.cpp:56-77,532-604; gpu/reducegrad.cpp:20-44,288-322), CPU twin impl/linear.h:51-110.
 * x[B][K], w[N][K] (stored once), y[B][N].   y = x * w^T */
int cnet_clinear_fwd(const float *x_re, const float *x_im, int64_t ldx,
                     const float *w_re, const float *w_im, int64_t ldw,
                     float *y_re, float *y_im, int64_t ldy, int B, int K, int N, int accumulate);
/* Linear followed by CGelu in one launch (gpu_linear_forward + gpu_gelu_forward, gpu/reduce.cpp:56-77 and
 * gpu/kernels.cpp:276-300; CPU twins impl/linear.h:51-69, impl/relu.h:119-131): h = x * w^T (the pre-activation, which
 * the backward pass of the CGelu reads) and y = gelu(h), applied to the accumulators when they are stored, so h is not
 * read back.  h and y share the leading dimension ldy.  With accumulate != 0 the product is added to h and y = gelu of
 * the sum.  y has the bits of cnet_cgelu_fwd applied to h. */
int cnet_clinear_cgelu_fwd(const float *x_re, const float *x_im, int64_t ldx,
                           const float *w_re, const float *w_im, int64_t ldw,
                           float *h_re, float *h_im, float *y_re, float *y_im, int64_t ldy,
                           int B, int K, int N, int accumulate);
/* dx.dz = g.dz * w ; dx.dzs = g.dzs * conj(w)            (both products in one launch) */
int cnet_clinear_bwd_input(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im,
                           int64_t ldg, const float *w_re, const float *w_im, int64_t ldw,
                           float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx,
                           int B, int K, int N, int accumulate);
/* dw.dz = g.dz^T * x ; dw.dzs = g.dzs^T * conj(x), summed over the B rows (the upstream sum over clones,
 * gpu/kernels.cpp:566-598, is part of the product here; deterministic, no atomics). */
int cnet_clinear_bwd_weight(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im,
                            int64_t ldg, const float *x_re, const float *x_im, int64_t ldx,
                            float *dw_dz_re, float *dw_dz_im, float *dw_dzs_re, float *dw_dzs_im, int64_t lddw,
                            int B, int K, int N, int accumulate);

/* The same two backward passes for a gradient pair that is conjugate, g.dzs == conj(g.dz), as the loss layers produce it
 * (CrossEntropy impl/crossent.h, L2Out impl/l2out.h: the loss is real) and every layer's backward pass hands it on: then
 * g.dzs * conj(w) == conj(g.dz * w), so one product is computed and written twice, once conjugated.  Same results as
 * cnet_clinear_bwd_input / _bwd_weight on such a pair to rounding (with four real products per complex one the sums are
 * the same and the signs exact, but half as many blocks may take another block shape; with three, see
 * cnet_cgemm_set_products, the imaginary parts of the two halves are rounded differently) at half the matrix work.  Replace the same upstream
 * functions (gpu/reduce.cpp:532-604, gpu/reducegrad.cpp:288-322); the caller vouches for the pair.  The dzs planes of the
 * result may both be NULL (here and in cnet_cdft_bwd_sym / cnet_ctriang_dft_bwd_sym): then only the dz planes are written,
 * which is all a consumer needs that is itself a conjugate-pair entry point. */
int cnet_clinear_bwd_input_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, const float *w_re, const float *w_im,
                               int64_t ldw, float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im,
                               int64_t lddx, int B, int K, int N, int accumulate);
int cnet_clinear_bwd_weight_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, const float *x_re, const float *x_im,
                                int64_t ldx, float *dw_dz_re, float *dw_dz_im, float *dw_dzs_re, float *dw_dzs_im,
                                int64_t lddw, int B, int K, int N, int accumulate);
/* Both of them in one call, as upstream's LinearGpu::gpu_linear_backward forms every gradient of the layer in one call
 * (gpu/reducegrad.cpp:309-322): dx (+)= g w and dw (+)= g^T x with the bits of the two calls above, each with its own
 * accumulate flag.  When both products are small (a narrow layer at a small batch, 64 x 784 -> 10: each a few microseconds of
 * work behind a launch that costs as much) and take the same kernel they go out as ONE launch; otherwise as the launches
 * of the two calls above, one after the other. */
int cnet_clinear_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, const float *x_re, const float *x_im,
                         int64_t ldx, const float *w_re, const float *w_im, int64_t ldw, float *dx_dz_re, float *dx_dz_im,
                         float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int accumulate_dx, float *dw_dz_re,
                         float *dw_dz_im, float *dw_dzs_re, float *dw_dzs_im, int64_t lddw, int accumulate_dw, int B, int K,
                         int N);

/* How many real matrix products the block kernels of every complex product above and below (Linear, FourierTrans,
 * TriangFourier; forward and backward) form one complex product from.  Upstream's CPU path, the parity reference, multiplies
 * complex numbers with four real multiplications (std::complex, impl/linear.h:51-69); its device code with three, number by
 * number (cmplx_::operator*=, gpu/compl.h:57-63: (a - b) d + a (c - d) and (a + b) c - a (c - d)).
 *   4 (default): Cr = Ar Br - Ai Bi, Ci = Ar Bi + Ai Br, the four real products of the complex multiplication.
 *   3: P = Ar Br, Q = Ai Bi, T = (Ar + Ai)(Br + Bi); Cr = P - Q, Ci = T - P - Q (signs of a conjugated operand
 *      applied to its imaginary part in the sums): a quarter of the matrix work less.  The real part is formed as with
 *      4; the imaginary part carries the rounding of all three products, so its error is bounded against the size
 *      of the whole complex entry, not of the imaginary part alone (measured against double precision on normal operands, relative
 *      Frobenius error of C with 3 against 4: 8.1e-7 against 5.8e-7 at K = 1024, 1.6e-6 against 1.1e-6 at K = 4096; of the
 *      imaginary plane alone 1.7 times that of 4, of the real plane the same).  An operand pair
 *      with both imaginary planes zero still gives an imaginary plane of exact zeros (T and P are then the same sums).
 *      Applies to the block kernels for 16-byte aligned operands with K a multiple of 16 (the ones every large product
 *      runs on), except the 128 x 128 block when both operands are stored with k contiguous (no registers for a third
 *      set of accumulators there: the cost model then weighs that block shape at its four products); the small-C
 *      kernel and the kernel for unaligned operands always use 4.
 * Process-wide; takes effect with the next product that is queued (a recorded graph keeps the kernels it was recorded
 * with).  The environment variable CNET_CGEMM_3M=0 / 1 sets the initial value.
 * Returns CNET_ERR_INVALID_ARGUMENT for any other n, and CNET_ERR_UNSUPPORTED for a change between cnet_graph_begin and
 * cnet_graph_end (one recording would otherwise hold products of both kinds). */
int cnet_cgemm_set_products(int n);
int cnet_cgemm_get_products(void);

/* A Linear layer that feeds a CrossEntropy (a classifier head): y = x w^T, then the forward pass of the loss over the rows of y
 * and its gradient, with the arguments and the bits of cnet_clinear_fwd followed by cnet_cross_entropy_fwd_bwd_sym (y takes the
 * place of z there).  Upstream runs LinearGpu::forward and CrossEntGpu::forward / backward one after the other
 * (gpu/reduce.cpp:581-604, 609-655).  One launch when the head is narrow (N <= 16) and the product small enough for the
 * small-C kernel without slices of K: the workgroup that has formed 16 rows of logits goes on to their loss.  Otherwise those
 * two calls. */
int cnet_clinear_cross_entropy_fwd_bwd_sym(const float *x_re, const float *x_im, int64_t ldx, const float *w_re, const float *w_im,
                                           int64_t ldw, float *y_re, float *y_im, int64_t ldy, const int32_t *labels,
                                           float *out_re, float *out_im, int64_t ldo, float *s, float *loss, int32_t *argmax,
                                           float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz,
                                           int B, int K, int N);

/* ---- FourierTrans as dense complex GEMM: replaces FourierGpu::gpu_fft_forward / gpu_fft_backward
 *      (gpu/reduce.cpp:25-35,160-187,382-393; gpu/reducegrad.cpp:45-48,324-336) and the root-table upload
 *      u_roots_allocate_and_copy_on_gpu (gpu/allocator.h:389-407).  CPU twin impl/ft.h:37-80.
 * F[p][q] = exp(-2 pi i p q / n) / sqrt(n), generated on the device with exact integer reduction of p*q mod n. */
int cnet_cdft_plan(int n);      /* build (once) and keep the n x n twiddle planes; called at net allocation time */
int cnet_cdft_twiddle(int n, const float **f_re, const float **f_im);  /* the planes of an existing plan */
/* Diagnostic: replace the FORWARD operator of length n by a caller-supplied matrix f[p][q] (host, row-major, y_p =
 * sum_q f[p][q] x_q); NULL, NULL restores the exact transform.  The upstream CPU forward is a float FFT whose twiddle
 * recurrence (impl/utils.h:204-211, 242-249) makes it a fixed operator up to 9e-5 away from the exact DFT; feeding that
 * operator here reproduces the CPU path to ~1e-6 and so separates its rounding from everything else.  The backward pass
 * keeps the exact twiddles, as upstream's does (impl/ft.h:57-79). */
int cnet_cdft_set_forward_matrix(int n, const float *host_f_re, const float *host_f_im);
int cnet_cdft_fwd(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy,
                  int B, int n, int accumulate);      /* y = x * F */
/* FourierTrans followed by a Hadamard gate with one shared weight row and a CGelu, the first three layers of upstream's README
 * net (README.md:19-30; FourierGpu::gpu_fft_forward gpu/reduce.cpp:382-393, gpu_hadamard_forward gpu/kernels.cpp:204-232,
 * gpu_gelu_forward gpu/kernels.cpp:292-315): y = x F, h = y .* v (v one row of n weights), a = gelu(h), all three written
 * (leading dimension ld each), with the bits of cnet_cdft_fwd followed by cnet_hadamard_cgelu_fwd.  One launch when the
 * product is small enough for the small-C kernel (a small batch: the step is then bound by its launches), else those two
 * calls. */
int cnet_cdft_hadamard_cgelu_fwd(const float *x_re, const float *x_im, int64_t ldx, const float *v_re, const float *v_im,
                                 float *y_re, float *y_im, float *h_re, float *h_im, float *a_re, float *a_im, int64_t ld,
                                 int B, int n);
/* The same transform for REAL samples (upstream's FourierTrans forward, impl/ft.h:37-55, transforms them like any
 * others, and so does gpu_fft_forward, gpu/reduce.cpp:160-187).  The caller vouches that every x_im is +0 (the plane must
 * exist and hold the zeros: the kernels for small and for unaligned shapes read it; the block kernels do not).  The result is
 * conjugate-symmetric, y[n - q] = conj(y[q]), so only columns 0 .. n/2 (rounded up to a multiple of four) go through the
 * matrix product and the rest are written as conjugates by the same kernels as they store their partners (exact conjugates;
 * the up to three columns next to n/2 whose partners the product computes as well agree with them to rounding), and of the
 * four real products of a complex one the two with x_im are left out: a quarter of the
 * matrix work of cnet_cdft_fwd.  Where the block kernels run the product (an even n at a batch beyond the small-C kernel)
 * the samples are folded about n/2 first, e[k] = x[k] + x[n - k] and o[k] = x[k] - x[n - k] (cos is even and sin odd under
 * k -> n - k), so that Re y = e F_re and Im y = o F_im are sums over k = 0 .. n/2 only: an eighth of the matrix work
 * (4096 x 784: 46 us with the pass that folds, 59 without; 1024 x 4096: 150 against 257; against double precision 8.0e-7
 * where the full product has 1.1e-6 at n = 4096); where n/2 is a multiple of 64 that pass also forms column n/2, the
 * alternating sum of the samples over sqrt n, and the product stops before it.  Agrees with cnet_cdft_fwd on such samples to rounding (the stored
 * twiddles are symmetric under q -> n - q up to their last bit; the products that are left out add exact zeros); assigns. */
int cnet_cdft_fwd_real_input(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy,
                             int B, int n);
int cnet_cdft_bwd(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
                  float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx,
                  int B, int n, int accumulate);      /* dx.dz = g.dz * F ; dx.dzs = g.dzs * conj(F) */
/* for a conjugate gradient pair (see cnet_clinear_bwd_input_sym): dx.dz = g.dz * F, dx.dzs = its conjugate
 * (gpu/reducegrad.cpp:324-336 upstream) */
int cnet_cdft_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, float *dx_dz_re, float *dx_dz_im,
                      float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int B, int n, int accumulate);

/* ---- TriangFourier: the DFT sums restricted to in <= out, y_o = (1/sqrt n) sum_{i <= o} x_i w^{i o}; CPU twin
 *      impl/ft.h:139-189 (upstream has no device kernel for it: its GPU tests expect "not supported",
 *      tests/gputests.h:1319-1330).  Runs as the same complex GEMM against an upper-triangular twiddle matrix; blocks of
 *      the matrix that lie wholly below the diagonal are skipped, so it costs about half of cnet_cdft_*. */
int cnet_ctriang_dft_plan(int n);
int cnet_ctriang_dft_fwd(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy,
                         int B, int n, int accumulate);
int cnet_ctriang_dft_bwd(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
                         float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx,
                         int B, int n, int accumulate);
/* for a conjugate gradient pair (see cnet_clinear_bwd_input_sym); CPU twin impl/ft.h:164-189 */
int cnet_ctriang_dft_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, float *dx_dz_re, float *dx_dz_im,
                             float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int B, int n, int accumulate);

/* ---- Hadamard: replaces gpu_hadamard_forward / _backward (gpu/kernels.cpp:204-274), CPU twin impl/hadamard.h:34-68.
 * y = u .* v.  ldv == 0: v is one parameter row shared by all rows and dv is the sum over rows. */
int cnet_hadamard_fwd(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
                      float *y_re, float *y_im, int64_t ldy, int rows, int cols);
int cnet_hadamard_bwd(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
                      const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
                      float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
                      float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv,
                      int rows, int cols, int accumulate);

/* ---- CGelu: replaces gpu_gelu_forward / _backward (gpu/kernels.cpp:276-360), CPU twin impl/relu.h:119-168. */
int cnet_cgelu_fwd(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy,
                   int rows, int cols);
int cnet_cgelu_bwd(const float *x_re, const float *x_im, int64_t ldx,
                   const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
                   float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx,
                   int rows, int cols, int accumulate);

/* ---- CRelu: y = z where Re z > 0 and Im z > 0, else 0; gradients pass under the same test.  CPU twin
 *      impl/relu.h:32-63 (no upstream device kernel either). */
int cnet_crelu_fwd(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy,
                   int rows, int cols);
int cnet_crelu_bwd(const float *x_re, const float *x_im, int64_t ldx,
                   const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
                   float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx,
                   int rows, int cols, int accumulate);

/* ---- Residual: replaces gpu_residual_forward / _backward (gpu/kernels.cpp:145-202), CPU twin impl/residual.h:40-77.
 * Forward: ldu == 0 or ldv == 0 makes that operand one parameter row added to every row (its gradient is then the
 * column sum of g: cnet_batch_sum). */
int cnet_residual_fwd(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
                      float *y_re, float *y_im, int64_t ldy, int rows, int cols);
int cnet_residual_bwd(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
                      float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
                      float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv,
                      int rows, int cols, int accumulate);

/* ---- SoftMax (L2 normalisation y = z/|z|): replaces SoftMaxGpu::gpu_soft_max_forward / _backward
 *      (gpu/reduce.cpp:189-230,449-466; gpu/reducegrad.cpp:10-19,60-66,268-286), CPU twin impl/softmax.h:33-73 with
 *      the chain rule of impl/cfunc.h:290-325 in closed O(n) form.  s[rows] receives sum |z|^2 per row. */
int cnet_l2norm_fwd(const float *z_re, const float *z_im, int64_t ldz, float *y_re, float *y_im, int64_t ldy,
                    float *s, int rows, int cols);
int cnet_l2norm_bwd(const float *z_re, const float *z_im, int64_t ldz, const float *s,
                    const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
                    float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz,
                    int rows, int cols, int accumulate);

/* ---- CrossEntropy: replaces CrossEntropyGpu::gpu_cross_ent_forward / _backward (gpu/reduce.cpp:469-530,609-655)
 *      and the loss read-back of CNet::getLoss (gpu/gpu_func.h:906-926).  CPU twin impl/crossent.h:50-130.
 * labels[rows] int32.  s = clamped sum |z|^2, loss = -log(max(|z_label|^2/s, 1e-15)), argmax = first index of the
 * strict maximum of |z_k/sqrt(s)|^2.  out_re/out_im (normalised z) may be NULL.  A label outside [0, cols) gives a NaN
 * loss for its row (upstream reads out of bounds); the backward pass then treats every entry as a non-label entry.
 * `loss` (here and in cnet_l2out_fwd) may point into page-locked host memory from cnet_host_alloc: the kernel then stores
 * the per-row losses there itself and no copy has to be queued to read them (a point taken with cnet_copy_ticket behind the
 * call tells the host when they have arrived). */
int cnet_cross_entropy_fwd(const float *z_re, const float *z_im, int64_t ldz, const int32_t *labels,
                           float *out_re, float *out_im, int64_t ldo, float *s, float *loss, int32_t *argmax,
                           int rows, int cols);
/* assigns (never accumulates), as impl/crossent.h:82-104 */
int cnet_cross_entropy_bwd(const float *z_re, const float *z_im, int64_t ldz, const float *s, const int32_t *labels,
                           float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz,
                           int rows, int cols);

/* ---- L2Out: replaces L2Gpu::gpu_norm_forward / gpu_norm_backward (gpu/reduce.cpp:232-251,408-446),
 *      CPU twin impl/l2out.h:33-58.  loss[rows] = sum |z|^2 ; dz = conj z, dzs = z. */
int cnet_l2out_fwd(const float *z_re, const float *z_im, int64_t ldz, float *loss, int rows, int cols);
int cnet_l2out_bwd(const float *z_re, const float *z_im, int64_t ldz,
                   float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz,
                   int rows, int cols, int accumulate);

/* ---- CInput and parameter plumbing: replaces gpu_input_forward / _backward (gpu/kernels.cpp:89-143),
 *      gpu_update_input (gpu/kernels.cpp:471-492) and gpu_copy_to_clones / gpu_grad_from_clones
 *      (gpu/kernels.cpp:528-598; with parameters stored once there is nothing to broadcast, and the sum over
 *      clones becomes cnet_batch_sum or is fused into the producing kernel). */
int cnet_copy2d(const float *src, int64_t lds, float *dst, int64_t ldd, int rows, int cols);       /* one plane */
int cnet_add2d(const float *src, int64_t lds, float *dst, int64_t ldd, int rows, int cols);        /* dst += src */
int cnet_batch_sum(const float *src, int64_t lds, float *dst, int rows, int cols, int accumulate); /* dst[c] (+)= sum_r src[r][c] */
/* cnet_batch_sum for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc); it has no counterpart upstream.  Same arguments, same kernels and bit-identical
 * results; the partial sums of its first stage go to a 2 MiB array that is part of the library's image on each device
 * instead of the library workspace, so the call never allocates or frees.  Limit: slabs x cols <= 524288 floats, with
 * slabs = max(1, min(256, w x compute units / ceil(cols / 256))), w = 8 for planes of 2^24 elements and more, else 4, and at
 * most ceil(rows / 4).  On a device with up to 256 compute units that holds for every cols <= 524288; a device with more
 * units refuses some of the widest planes.  Beyond the limit the call returns CNET_ERR_UNSUPPORTED.  All calls on one device share the array: calls that overlap in time (two
 * streams, two host threads) race. */
int cnet_batch_sum_noalloc(const float *src, int64_t lds, float *dst, int rows, int cols, int accumulate);
/* dst[k][0..n[k]) += src[k][0..n[k]) for `count` dense arrays in one launch: what the loop over the input functions in
 * GpuNet::GpuBackward becomes (each CInput gathers the dz* of its consumer, impl/cinput.h:54-65, gpu/kernels.cpp:118-143).
 * The destinations of one call must not overlap (the additions of a call run concurrently). */
int cnet_add_multi(int count, const float *const *src, float *const *dst, const int64_t *n);
/* z -= lr * dzs ; then dzs = 0 when zero_grad != 0   (impl/cfunc.h:147-152 + impl/cnet.h:413-421) */
int cnet_sgd_update(float *z_re, float *z_im, float *dzs_re, float *dzs_im, int64_t n, float lr, int zero_grad);

/* The same step for `count` tensors in one launch (host arrays of device pointers and lengths): a net with many small
 * parameter tensors is otherwise bound by launches. */
int cnet_sgd_update_multi(int count, float *const *z_re, float *const *z_im, float *const *dzs_re, float *const *dzs_im,
                          const int64_t *n, float lr, int zero_grad);
/* Adam-style step: replaces gpu_update_adam_input (gpu/kernels.cpp:494-525), CPU twin impl/cfunc.h:273-287 +
 * impl/cnet.h:423-431.  m = beta m + (1 - beta) dzs ; z -= lr m / (1 - beta^(t+1)) ; then dzs = 0 when zero_grad != 0.
 * m_re / m_im are the first-moment planes (upstream keeps them in the node's dz planes, impl/cfunc.h:341-349). */
int cnet_adam_update(float *z_re, float *z_im, float *m_re, float *m_im, float *dzs_re, float *dzs_im, int64_t n,
                     float lr, float beta, int t, int zero_grad);

/* ---- The elementwise and loss backward passes for a conjugate gradient pair (see cnet_clinear_bwd_input_sym): g.dzs ==
 *      conj(g.dz) is not read, the dz planes of the result are formed with the arithmetic of the general entry point
 *      (same bits on an exactly conjugate pair), and its dzs planes receive the conjugate when they are given; both may be
 *      NULL, which leaves them untouched: 24 bytes per complex element instead of 40 (CGelu, CRelu, Hadamard, SoftMax),
 *      24 instead of 48 (Residual), 16 instead of 24 (the losses).  They replace the same upstream kernels as the general
 *      entry points: gpu/kernels.cpp:204-360, 145-202; gpu/reducegrad.cpp:268-286; gpu/reduce.cpp:408-446, 609-655. */
int cnet_hadamard_bwd_sym(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
                          const float *g_dz_re, const float *g_dz_im, int64_t ldg,
                          float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
                          float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv,
                          int rows, int cols, int accumulate);
int cnet_cgelu_bwd_sym(const float *x_re, const float *x_im, int64_t ldx, const float *g_dz_re, const float *g_dz_im, int64_t ldg,
                       float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx,
                       int rows, int cols, int accumulate);
/* Hadamard followed by CGelu as one pass each way (the pair gpu_hadamard_forward + gpu_gelu_forward and
 * gpu_gelu_backward + gpu_hadamard_backward, gpu/kernels.cpp:204-360; CPU twins impl/hadamard.h:34-68, impl/relu.h:119-168).
 * Forward: h = u .* v and y = gelu(h) are both written, u and v read once: with a shared v 24 bytes per complex element
 * instead of 16 + 16.  Backward: g is the gradient pair that reaches the CGelu; h is recomputed from u and v (the bits of
 * the forward pass), dh = the CGelu's gradient (assigned, never accumulated; its dzs planes optional, and all four NULL
 * when nobody reads it), du and dv as cnet_hadamard_bwd_sym from dh: with a shared v 24 (32 with dh) bytes per complex
 * element instead of 24 + 24.  Every result has the bits of the two separate calls. */
int cnet_hadamard_cgelu_fwd(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
                            float *h_re, float *h_im, int64_t ldh, float *y_re, float *y_im, int64_t ldy, int rows, int cols);
int cnet_hadamard_cgelu_bwd_sym(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
                                const float *g_dz_re, const float *g_dz_im, int64_t ldg,
                                float *dh_dz_re, float *dh_dz_im, float *dh_dzs_re, float *dh_dzs_im, int64_t lddh,
                                float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
                                float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv,
                                int rows, int cols, int accumulate);
/* The backward pass of a narrow Linear whose operand x = gelu(u .* v) came from a Hadamard gate with one shared row of weights
 * v under a CGelu: cnet_clinear_bwd_sym (dx, dw from the gradient g at the Linear's result) followed by
 * cnet_hadamard_cgelu_bwd_sym with ldv = 0 on dx (dh at the CGelu's operand, du, and dv summed over the batch), with the
 * arguments and the bits of those two calls.  Upstream runs LinearGpu::backward, gpu_gelu_backward and
 * gpu_hadamard_backward one after the other (gpu/reducegrad.cpp:324-336, gpu/kernels.cpp:204-360).  One launch when the batch
 * has at most 128 rows and both products fit the small-C kernel without slices of K: the workgroup that has formed 16 columns
 * of dx (all rows) and of dw goes on to the gate's backward pass of those columns and adds their rows into dv in the order of
 * the separate launches.  Otherwise those two calls (three to four launches). */
int cnet_clinear_hadamard_cgelu_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg,
                                        const float *x_re, const float *x_im, int64_t ldx,
                                        const float *w_re, const float *w_im, int64_t ldw,
                                        float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int accumulate_dx,
                                        float *dw_dz_re, float *dw_dz_im, float *dw_dzs_re, float *dw_dzs_im, int64_t lddw, int accumulate_dw,
                                        const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im,
                                        float *dh_dz_re, float *dh_dz_im, float *dh_dzs_re, float *dh_dzs_im, int64_t lddh,
                                        float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
                                        float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int accumulate_gate,
                                        int B, int K, int N);
int cnet_crelu_bwd_sym(const float *x_re, const float *x_im, int64_t ldx, const float *g_dz_re, const float *g_dz_im, int64_t ldg,
                       float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx,
                       int rows, int cols, int accumulate);
int cnet_residual_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg,
                          float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
                          float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv,
                          int rows, int cols, int accumulate);
/* the same for a Residual whose result feeds two consumers: their two gradients are added in the kernel (g1 first: the
 * bits of two cnet_residual_bwd_sym calls, the second accumulating), and du, dv are written once */
int cnet_residual_bwd_sym2(const float *g1_dz_re, const float *g1_dz_im, int64_t ldg1,
                           const float *g2_dz_re, const float *g2_dz_im, int64_t ldg2,
                           float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
                           float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv,
                           int rows, int cols, int accumulate);
/* A Residual one of whose operands is the result of a CGelu, both backward passes in one (gpu_residual_backward +
 * gpu_gelu_backward, gpu/kernels.cpp:170-202, 302-360; CPU twins impl/residual.h:56-77, impl/relu.h:144-166).  g1 (and g2,
 * or NULL for both of its planes: the Residual then feeds one consumer) is the gradient pair that reaches the Residual;
 * du, the gradient of its other operand, receives g1 + g2; dv, the gradient of the CGelu's result, receives the same when
 * its planes are given (all four NULL: nobody reads it); dh, the gradient of the CGelu's operand h, receives the CGelu
 * backward of g1 + g2 at h.  All assigned.  The bits of cnet_residual_bwd_sym2 (or _sym) followed by cnet_cgelu_bwd_sym;
 * 40 bytes per complex element (32 with one consumer) instead of 56 (48). */
int cnet_residual_cgelu_bwd_sym(const float *g1_dz_re, const float *g1_dz_im, int64_t ldg1,
                                const float *g2_dz_re, const float *g2_dz_im, int64_t ldg2,
                                const float *h_re, const float *h_im, int64_t ldh,
                                float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
                                float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv,
                                float *dh_dz_re, float *dh_dz_im, float *dh_dzs_re, float *dh_dzs_im, int64_t lddh,
                                int rows, int cols);
int cnet_l2norm_bwd_sym(const float *z_re, const float *z_im, int64_t ldz, const float *s,
                        const float *g_dz_re, const float *g_dz_im, int64_t ldg,
                        float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz,
                        int rows, int cols, int accumulate);
/* the two losses produce the pair themselves: dz = conj(dzs) */
int cnet_l2out_bwd_sym(const float *z_re, const float *z_im, int64_t ldz,
                       float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz,
                       int rows, int cols, int accumulate);
int cnet_cross_entropy_bwd_sym(const float *z_re, const float *z_im, int64_t ldz, const float *s, const int32_t *labels,
                               float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz,
                               int rows, int cols);
/* cnet_cross_entropy_fwd and cnet_cross_entropy_bwd_sym in one launch (upstream: gpu_cross_ent_forward and
 * gpu_cross_ent_backward, gpu/reduce.cpp:469-530, 609-655, which a training step always runs one after the other with the
 * same labels): every result of the forward call, and the gradient of each row's loss in the dz planes (its conjugate in
 * the dz* planes when those are given), with the bits of the two separate calls.  For rows short enough that a launch
 * costs more than the pass itself (a classifier head: 10 columns). */
int cnet_cross_entropy_fwd_bwd_sym(const float *z_re, const float *z_im, int64_t ldz, const int32_t *labels,
                                   float *out_re, float *out_im, int64_t ldo, float *s, float *loss, int32_t *argmax,
                                   float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz,
                                   int rows, int cols);

/* ---- CEmbedding: replaces gpu_embedding_forward / _backward (gpu/kernels.cpp:362-442), CPU twin impl/embed.h:109-148.
 * tokens[rows][slots] int32, -1 = padding (zero row); an id >= vocab is treated as padding too (upstream asserts on
 * the host; the host side above this ABI rejects it).  y[rows][slots*dim].  The backward adds the dzs rows of equal
 * tokens in (row, slot) order - deterministic, no atomics. */
int cnet_embedding_fwd(const float *table_re, const float *table_im, int dim, int vocab, const int32_t *tokens,
                       float *y_re, float *y_im, int64_t ldy, int rows, int slots);
int cnet_embedding_bwd(const int32_t *tokens, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
                       float *table_dzs_re, float *table_dzs_im, int dim, int vocab, int rows, int slots, int accumulate);

/* ---- Tuning overrides (environment variables).  None is needed for correct results or for the figures this library is
 *      measured with; they exist so that tests and sweeps can send a shape to every kernel that could take it.  Each is
 *      read ONCE per process, when the first launch that consults it is queued; results do not depend on them beyond
 *      rounding (another block shape or cut groups the sums differently), and every path they select is deterministic.
 *   CNET_CGEMM_TILE = 0..4       block shape of the matrix kernels: 128x128, 64x128, 128x64, 64x64, 64x64 with two LDS
 *                                stages (default: cost model)
 *   CNET_CGEMM_TAIL = 0 | 1      never / whenever possible cut the blocks of a partly filled last round along K
 *   CNET_CGEMM_KCUT = 0          cut a product along K only when half of the compute units would idle
 *   CNET_CGEMM_KMODEL = 0        price every K with the efficiency table measured at K = 2048
 *   CNET_CGEMM_COLSPLIT = 0      never split the last few columns of C off into a launch of their own
 *   CNET_CGEMM_KREST = 0         never split the last K % 16 values of k off (the whole product takes the general kernel)
 *   CNET_CGEMM_SKINNY = 0        small products on the block kernels instead of the small-C kernel
 *   CNET_CGEMM_SKINNY_TILES = n  largest number of 16x16 tiles of C the small-C kernel takes (default 4 per compute unit)
 *   CNET_CGEMM_SKINNY_W = 4|8|16 wavefronts per tile of the small-C kernel
 *   CNET_CGEMM_SKINNY_TWO = 0    two small products of one call as two launches (and the gate behind them as launches of its own)
 *   CNET_CGEMM_3M = 0 | 1        initial value of cnet_cgemm_set_products (1: three real products per complex one)
 *   CNET_CGEMM_PACK = 0          large products of misaligned operands on the operands as they are (no aligned copies)
 *   CNET_DFT_FOLD = 0            the transform of real samples without folding them about n/2 first
 *   CNET_STREAM_MIN_MB = n       footprint (MiB) from which an elementwise / row launch counts as streaming (default 256)
 *   CNET_STREAM_POLICY = 0..3    cache policy of every streaming launch: plain, hint on loads and stores, hinted stores,
 *                                hinted loads + device-scope stores (default: per kernel)
 */

#ifdef __cplusplus
}
#endif
#endif /* CNET_HIP_H_ */
