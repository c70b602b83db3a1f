// FourierTrans as a dense complex GEMM against a twiddle matrix generated on the device.
//   F[p][q] = exp(-2 pi i (p*q mod n) / n) / sqrt(n)        (sign and scaling of impl/utils.h:218-221, impl/ft.h:44-47 upstream)
// p*q is reduced mod n in 64-bit integers before the angle is formed, and sin/cos are evaluated in double, so every
// entry is the correctly rounded fp32 value of the exact root of unity; F is symmetric, so y = x * F.
#include "common.hpp"

#include <algorithm>
#include <map>
#include <vector>

namespace cnet {

int cgemm_real_a(int M, int N, int K, const float *a_re, const float *a_im, long lda, const float *b_re, const float *b_im, long ldb, float *c_re,
		float *c_im, long ldc, int herm_n);
int cgemm_folded(int M, int N, int K, const float *ae, const float *ao, long lda, const float *b_re, const float *b_im, long ldb, float *c_re,
		float *c_im, long ldc, int herm_n);
bool cgemm_block_sized(int M, int N);
int cgemm_pair(bool a_mcontig, bool b_ncontig, int nprob, int M, int N, int K, const float *const a_re[2],
		const float *const a_im[2], long lda, const float *const b_re[2], const float *const b_im[2], long ldb,
		const bool conj_b[2], float *const c_re[2], float *const c_im[2], long ldc, int accumulate, int tri, int mirror);

int cgemm_dft_hgelu(int M, int n, const float *x_re, const float *x_im, long ldx, const float *f_re, const float *f_im, long ldf,
		const float *hv_re, const float *hv_im, float *y_re, float *y_im, float *h_re, float *h_im, float *g_re, float *g_im, long ld,
		bool *launched);

struct Twiddle {
	float *re = nullptr;
	float *im = nullptr;
	long ld = 0;
	// optional caller-supplied forward operator, stored transposed ([q][p]) so that y = x * B; the backward pass
	// always uses the exact twiddles above, as the CPU path does (impl/ft.h:57-79 upstream)
	float *fwd_re = nullptr;
	float *fwd_im = nullptr;
	// TriangFourier operator: T[i][o] = F[i][o] for i <= o, zero below the diagonal (impl/ft.h:151-156 upstream);
	// built on first use
	float *tri_re = nullptr;
	float *tri_im = nullptr;
};
static std::map<int, Twiddle> g_twiddles;

void release_twiddles() {
	for (auto &kv : g_twiddles) {
		(void) hipFree(kv.second.re);  // one allocation holds both planes
		if (kv.second.fwd_re) (void) hipFree(kv.second.fwd_re);
		if (kv.second.tri_re) (void) hipFree(kv.second.tri_re);
	}
	g_twiddles.clear();
}

// upper_only: entries with p > q are written as zeros
__global__ void twiddle_kernel(float *__restrict__ fre, float *__restrict__ fim, int n, long ld, int upper_only) {
	const long idx = (long) blockIdx.x * blockDim.x + threadIdx.x;
	if (idx >= (long) n * n) return;
	const int p = (int) (idx / n), q = (int) (idx % n);
	const long e = ((long) p * q) % n;
	double s, c;
	sincospi(-2.0 * (double) e / (double) n, &s, &c);
	const double scale = (upper_only && p > q) ? 0.0 : 1.0 / sqrt((double) n);
	fre[(long) p * ld + q] = (float) (c * scale);
	fim[(long) p * ld + q] = (float) (s * scale);
}

// cos(2 pi k q / n) is even and sin odd under k -> n - k, so for real samples x of even length n
//   Re X[q] = sum_{k = 0 .. n/2} e[k] F_re[k][q],   Im X[q] = sum_{k = 0 .. n/2} o[k] F_im[k][q]
// with e[0] = x[0], e[n/2] = x[n/2], e[k] = x[k] + x[n - k] and o[k] = x[k] - x[n - k] in between (o[0] = o[n/2] = 0): two
// real products over half the k.  This kernel writes e and o as planes [rows][kp], kp = n/2 + 1 rounded up to a multiple
// of 16 (the chunk of the block kernels), zeros beyond n/2; one thread per four k.
template <bool V4>
__device__ __forceinline__ void fold_group(const float *__restrict__ xr, int n, int k0, float ev[4], float ov[4]) {
	float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};  // x[k0 + s] and its partner x[n - k0 - s]
	if (V4 && k0 + 3 < n / 2 && k0 > 0) {
		// (n and ldx multiples of four, x 16-byte aligned: x[k0 .. k0 + 3] is one aligned group, and the partners are the last
		// three values of the aligned group that ends at n - k0, and the first value of the next one)
		const float4 f = *reinterpret_cast<const float4 *>(xr + k0), g = *reinterpret_cast<const float4 *>(xr + n - k0 - 4);
		a[0] = f.x, a[1] = f.y, a[2] = f.z, a[3] = f.w;
		b[0] = xr[n - k0], b[1] = g.w, b[2] = g.z, b[3] = g.y;
	} else {
#pragma unroll
		for (int s = 0; s < 4; ++s) {
			const int k = k0 + s;
			if (k <= n / 2) {
				a[s] = xr[k];
				if (k > 0 && k < n / 2) b[s] = xr[n - k];
			}
		}
	}
#pragma unroll
	for (int s = 0; s < 4; ++s) {
		const int k = k0 + s;
		ev[s] = a[s] + b[s];
		ov[s] = (k > 0 && k < n / 2) ? a[s] - b[s] : 0.f;
	}
}

template <bool V4>
__global__ __launch_bounds__(256) void fold_kernel(const float *__restrict__ x, long ldx, float *__restrict__ e, float *__restrict__ o, int rows,
		int n, int kp) {
	const long idx = (long) blockIdx.x * 256 + threadIdx.x;
	const int groups = kp / 4;
	if (idx >= (long) rows * groups) return;
	const long row = idx / groups;
	const int k0 = (int) (idx - row * groups) * 4;
	float ev[4], ov[4];
	fold_group<V4>(x + row * ldx, n, k0, ev, ov);
	float4 *pe = reinterpret_cast<float4 *>(e + row * kp + k0), *po = reinterpret_cast<float4 *>(o + row * kp + k0);
	*pe = make_float4(ev[0], ev[1], ev[2], ev[3]);
	*po = make_float4(ov[0], ov[1], ov[2], ov[3]);
}

// The same pass with one wavefront per row, which also forms column n/2 of the transform: F[k][n/2] = (-1)^k / sqrt n, so
// Re X[n/2] = (e[0] - e[1] + e[2] - ...) / sqrt n and Im X[n/2] = 0.  The product then stops at column n/2 - 1; where n/2
// is a multiple of the blocks' width that spares it a round of blocks that hold this one column.  The lanes' sums are
// added in a fixed order.
template <bool V4>
__global__ __launch_bounds__(256) void fold_nyquist_kernel(const float *__restrict__ x, long ldx, float *__restrict__ e, float *__restrict__ o,
		int rows, int n, int kp, float *__restrict__ y_re, float *__restrict__ y_im, long ldy, float scale) {
	const long row = (long) blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= rows) return;  // (a whole wavefront: nothing below is shared between wavefronts)
	const int lane = threadIdx.x & 63, groups = kp / 4;
	const float *xr = x + row * ldx;
	float alt = 0.f;
	for (int g = lane; g < groups; g += 64) {
		float ev[4], ov[4];
		fold_group<V4>(xr, n, g * 4, ev, ov);
		float4 *pe = reinterpret_cast<float4 *>(e + row * kp + g * 4), *po = reinterpret_cast<float4 *>(o + row * kp + g * 4);
		*pe = make_float4(ev[0], ev[1], ev[2], ev[3]);
		*po = make_float4(ov[0], ov[1], ov[2], ov[3]);
		alt += (ev[0] - ev[1]) + (ev[2] - ev[3]);
	}
#pragma unroll
	for (int d = 32; d >= 1; d >>= 1) alt += __shfl_xor(alt, d, 64);
	if (lane == 0) {
		y_re[row * ldy + n / 2] = alt * scale;
		y_im[row * ldy + n / 2] = 0.f;
	}
}

static int get_plan(int n, Twiddle *out, bool create) {
	auto it = g_twiddles.find(n);
	if (it != g_twiddles.end()) {
		*out = it->second;
		return CNET_OK;
	}
	if (!create) return fail(CNET_ERR_INVALID_ARGUMENT, "no twiddle plan for n=%d: call cnet_cdft_plan first", n);
	if (rt().capturing)
		return fail(CNET_ERR_UNSUPPORTED, "the twiddle planes for n=%d would have to be built while a graph is being recorded: call cnet_cdft_plan first", n);
	Twiddle t;
	t.ld = (n + 3) / 4 * 4;  // rows start 16-byte aligned
	size_t plane = (size_t) n * t.ld;
	CNET_HIP(hipMalloc((void **) &t.re, 2 * plane * sizeof(float)));
	t.im = t.re + plane;
	if (t.ld != n) {
		const hipError_t e = hipMemsetAsync(t.re, 0, 2 * plane * sizeof(float), rt().stream);
		if (e != hipSuccess) {
			hipFree(t.re);  // not in the table yet: nothing else would free the planes
			return hip_fail(e, "hipMemsetAsync(twiddle planes)");
		}
	}
	const long total = (long) n * n;
	hipLaunchKernelGGL(twiddle_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, rt().stream, t.re, t.im, n, t.ld, 0);
	g_twiddles[n] = t;  // owned by the table from here on, whatever the launch reports
	CNET_LAUNCH_CHECK();
	*out = t;
	return CNET_OK;
}

static int get_triangular(int n, Twiddle *out) {
	int rc = get_plan(n, out, true);
	if (rc || out->tri_re) return rc;
	if (rt().capturing)
		return fail(CNET_ERR_UNSUPPORTED, "the triangular twiddle planes for n=%d would have to be built while a graph is being recorded: call cnet_ctriang_dft_plan first", n);
	Twiddle &slot = g_twiddles[n];
	const size_t plane = (size_t) n * slot.ld;
	CNET_HIP(hipMalloc((void **) &slot.tri_re, 2 * plane * sizeof(float)));
	slot.tri_im = slot.tri_re + plane;
	if (slot.ld != n) {
		const hipError_t e = hipMemsetAsync(slot.tri_re, 0, 2 * plane * sizeof(float), rt().stream);
		if (e != hipSuccess) {
			hipFree(slot.tri_re);  // the slot must not keep planes that were never filled
			slot.tri_re = slot.tri_im = nullptr;
			return hip_fail(e, "hipMemsetAsync(triangular twiddle planes)");
		}
	}
	const long total = (long) n * n;
	hipLaunchKernelGGL(twiddle_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, rt().stream, slot.tri_re, slot.tri_im, n,
			slot.ld, 1);
	CNET_LAUNCH_CHECK();
	*out = slot;
	return CNET_OK;
}

}  // namespace cnet

using namespace cnet;

extern "C" {

int cnet_cdft_plan(int n) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(n > 0 && n <= 46340);  // p*q must fit the upstream int exponent as well (impl/ft.h:66)
	Twiddle t;
	return get_plan(n, &t, true);
}

int cnet_cdft_twiddle(int n, const float **f_re, const float **f_im) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(f_re && f_im);
	Twiddle t;
	int rc = get_plan(n, &t, false);
	if (rc) return rc;
	*f_re = t.re;
	*f_im = t.im;
	return CNET_OK;
}

int cnet_cdft_set_forward_matrix(int n, const float *host_f_re, const float *host_f_im) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_CHECK_ARG(n > 0 && n <= 46340);
	Twiddle t;
	int rc = get_plan(n, &t, true);
	if (rc) return rc;
	Twiddle &slot = g_twiddles[n];
	if (!host_f_re && !host_f_im) {  // back to the exact transform
		if (slot.fwd_re) {
			CNET_HIP(hipStreamSynchronize(rt().stream));
			CNET_HIP(hipFree(slot.fwd_re));
		}
		slot.fwd_re = slot.fwd_im = nullptr;
		return CNET_OK;
	}
	CNET_CHECK_ARG(host_f_re && host_f_im);
	const size_t plane = (size_t) n * t.ld;
	std::vector<float> tr(2 * plane, 0.0f);
	for (int p = 0; p < n; ++p)
		for (int q = 0; q < n; ++q) {
			tr[(size_t) q * t.ld + p] = host_f_re[(size_t) p * n + q];
			tr[plane + (size_t) q * t.ld + p] = host_f_im[(size_t) p * n + q];
		}
	if (!slot.fwd_re) CNET_HIP(hipMalloc((void **) &slot.fwd_re, 2 * plane * sizeof(float)));
	slot.fwd_im = slot.fwd_re + plane;
	CNET_HIP(hipMemcpyAsync(slot.fwd_re, tr.data(), 2 * plane * sizeof(float), hipMemcpyHostToDevice, rt().stream));
	CNET_HIP(hipStreamSynchronize(rt().stream));
	return CNET_OK;
}

int cnet_cdft_fwd(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy, int B, int n,
		int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && n > 0 && n <= 46340);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && y_re && y_im && ldx >= n && ldy >= n);
	Twiddle t;
	int rc = get_plan(n, &t, true);
	if (rc) return rc;
	const float *f_re = t.fwd_re ? t.fwd_re : t.re, *f_im = t.fwd_re ? t.fwd_im : t.im;
	const float *ar[2] = {x_re, x_re}, *ai[2] = {x_im, x_im}, *br[2] = {f_re, f_re}, *bi[2] = {f_im, f_im};
	float *cr[2] = {y_re, y_re}, *ci[2] = {y_im, y_im};
	bool cj[2] = {false, false};
	return cgemm_pair(false, true, 1, B, n, n, ar, ai, ldx, br, bi, t.ld, cj, cr, ci, ldy, accumulate, 0, 0);
}

int cnet_cdft_hadamard_cgelu_fwd(const float *x_re, const float *x_im, int64_t ldx, const float *v_re, const float *v_im, float *y_re,
		float *y_im, float *h_re, float *h_im, float *a_re, float *a_im, int64_t ld, int B, int n) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && n > 0 && n <= 46340);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && v_re && v_im && y_re && y_im && h_re && h_im && a_re && a_im && ldx >= n && ld >= n);
	Twiddle t;
	int rc = get_plan(n, &t, true);
	if (rc) return rc;
	const float *f_re = t.fwd_re ? t.fwd_re : t.re, *f_im = t.fwd_re ? t.fwd_im : t.im;
	bool launched = false;
	rc = cgemm_dft_hgelu(B, n, x_re, x_im, ldx, f_re, f_im, t.ld, v_re, v_im, y_re, y_im, h_re, h_im, a_re, a_im, ld, &launched);
	if (rc || launched) return rc;
	// a product for the block kernels, or one cut along K: the transform, then gate and activation in one pass over its result
	rc = cnet_cdft_fwd(x_re, x_im, ldx, y_re, y_im, ld, B, n, 0);
	return rc ? rc : cnet_hadamard_cgelu_fwd(y_re, y_im, ld, v_re, v_im, 0, h_re, h_im, ld, a_re, a_im, ld, B, n);
}

int cnet_cdft_fwd_real_input(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy, int B, int n) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && n > 0 && n <= 46340);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && y_re && y_im && ldx >= n && ldy >= n);
	Twiddle t;
	int rc = get_plan(n, &t, true);
	if (rc) return rc;
	// a caller-supplied forward operator need not be symmetric under q -> n - q: the whole product then
	if (t.fwd_re) return cnet_cdft_fwd(x_re, x_im, ldx, y_re, y_im, ldy, B, n, 0);
	// Columns 0 .. n/2 by the matrix product, rounded up to a multiple of four columns, which keeps the product on the
	// kernels with 128-bit loads (x_im holds zeros: the block kernels do not read it, the others do).  Columns cols .. n - 1
	// are the partners n - q of columns 1 .. n - cols (cols > n / 2: each of those has its partner outside the product): the
	// product writes them, conjugated, as it stores their partners.
	const int cols = std::min(n, (n / 2 + 1 + 3) / 4 * 4);
	// Folded about n/2 (fold_kernel), the product is half as long: where the block kernels run it (an even n, a batch
	// beyond the small-C kernel), 4096 x 784: 59 -> 46 us with the pass that folds.  The folded samples live in a buffer of
	// the library's own that only grows (not the workspace, where the product may keep partial sums); while a graph is
	// being recorded it cannot, and a batch larger than any before runs the unfolded product.
	const int kp = (n / 2 + 1 + 15) / 16 * 16;
	static const bool fold = [] {
		const char *e = getenv("CNET_DFT_FOLD");  // tuning override: 0 keeps the unfolded product
		return !e || atoi(e) != 0;
	}();
	if (fold && n % 2 == 0 && kp <= n && ldy % 4 == 0 && aligned16(y_re) && aligned16(y_im) && cgemm_block_sized(B, cols)) {
		const size_t need = 2 * (size_t) B * kp * sizeof(float);
		if (need <= rt().operand_workspace_bytes || !rt().capturing) {
			float *e = (float *) operand_workspace(need);
			if (!e) return CNET_ERR_OUT_OF_MEMORY;
			float *o = e + (size_t) B * kp;
			const bool v4 = n % 4 == 0 && ldx % 4 == 0 && aligned16(x_re);
			// n/2 a multiple of 64, the narrowest block: column n/2 would take a round of blocks of its own
			if (n % 128 == 0 && cgemm_block_sized(B, n / 2)) {
				const float scale = (float) (1.0 / sqrt((double) n));
				const dim3 grid((unsigned) ((B + 3) / 4));
				if (v4)
					hipLaunchKernelGGL(fold_nyquist_kernel<true>, grid, dim3(256), 0, rt().stream, x_re, (long) ldx, e, o, B, n, kp, y_re, y_im, (long) ldy, scale);
				else
					hipLaunchKernelGGL(fold_nyquist_kernel<false>, grid, dim3(256), 0, rt().stream, x_re, (long) ldx, e, o, B, n, kp, y_re, y_im, (long) ldy, scale);
				CNET_LAUNCH_CHECK();
				return cgemm_folded(B, n / 2, kp, e, o, kp, t.re, t.im, t.ld, y_re, y_im, ldy, n);
			}
			const long threads = (long) B * (kp / 4);
			if (v4)
				hipLaunchKernelGGL(fold_kernel<true>, dim3((unsigned) ((threads + 255) / 256)), dim3(256), 0, rt().stream, x_re, (long) ldx, e, o, B, n, kp);
			else
				hipLaunchKernelGGL(fold_kernel<false>, dim3((unsigned) ((threads + 255) / 256)), dim3(256), 0, rt().stream, x_re, (long) ldx, e, o, B, n, kp);
			CNET_LAUNCH_CHECK();
			return cgemm_folded(B, cols, kp, e, o, kp, t.re, t.im, t.ld, y_re, y_im, ldy, n);
		}
	}
	return cgemm_real_a(B, cols, n, x_re, x_im, ldx, t.re, t.im, t.ld, y_re, y_im, ldy, n);
}

int cnet_cdft_bwd(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
		float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int B, int n, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && n > 0 && n <= 46340);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && g_dzs_re && g_dzs_im && dx_dz_re && dx_dz_im && dx_dzs_re && dx_dzs_im);
	CNET_CHECK_ARG(ldg >= n && lddx >= n);
	Twiddle t;
	int rc = get_plan(n, &t, true);
	if (rc) return rc;
	// impl/ft.h:57-79 upstream: dz_q += sum_p G_p w^{pq}/sqrt n ; dzs_q += sum_p Gs_p conj(w^{pq})/sqrt n
	const float *ar[2] = {g_dz_re, g_dzs_re}, *ai[2] = {g_dz_im, g_dzs_im}, *br[2] = {t.re, t.re}, *bi[2] = {t.im, t.im};
	float *cr[2] = {dx_dz_re, dx_dzs_re}, *ci[2] = {dx_dz_im, dx_dzs_im};
	bool cj[2] = {false, true};
	return cgemm_pair(false, true, 2, B, n, n, ar, ai, ldg, br, bi, t.ld, cj, cr, ci, lddx, accumulate, 0, 0);
}

int cnet_ctriang_dft_plan(int n) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(n > 0 && n <= 46340);
	Twiddle t;
	return get_triangular(n, &t);
}

// y_o = sum_{i <= o} x_i T[i][o] : T is stored [k = i][n = o]; the column block [n0, n0 + BN) needs k < n0 + BN only
int cnet_ctriang_dft_fwd(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy, int B, int n,
		int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && n > 0 && n <= 46340);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && y_re && y_im && ldx >= n && ldy >= n);
	Twiddle t;
	int rc = get_triangular(n, &t);
	if (rc) return rc;
	const float *ar[2] = {x_re, x_re}, *ai[2] = {x_im, x_im}, *br[2] = {t.tri_re, t.tri_re}, *bi[2] = {t.tri_im, t.tri_im};
	float *cr[2] = {y_re, y_re}, *ci[2] = {y_im, y_im};
	bool cj[2] = {false, false};
	return cgemm_pair(false, true, 1, B, n, n, ar, ai, ldx, br, bi, t.ld, cj, cr, ci, ldy, accumulate, 1, 0);
}

// dz_i = sum_{o >= i} G_o T[i][o], dzs_i = sum_{o >= i} Gs_o conj(T[i][o])  (impl/ft.h:163-189 upstream): the same
// planes read as [n = i][k = o], i.e. contiguous along the reduction index; the block of rows i >= n0 needs k >= n0 only
int cnet_cdft_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re,
		float *dx_dzs_im, int64_t lddx, int B, int n, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && n > 0 && n <= 46340);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && dx_dz_re && dx_dz_im && ((dx_dzs_re == nullptr) == (dx_dzs_im == nullptr)));
	CNET_CHECK_ARG(ldg >= n && lddx >= n);
	Twiddle t;
	int rc = get_plan(n, &t, true);
	if (rc) return rc;
	// the dz product of cnet_cdft_bwd; the dzs product of a conjugate gradient pair is its conjugate and is written with it
	const float *ar[2] = {g_dz_re, g_dz_re}, *ai[2] = {g_dz_im, g_dz_im}, *br[2] = {t.re, t.re}, *bi[2] = {t.im, t.im};
	float *cr[2] = {dx_dz_re, dx_dzs_re}, *ci[2] = {dx_dz_im, dx_dzs_im};
	bool cj[2] = {false, false};
	return cgemm_pair(false, true, 1, B, n, n, ar, ai, ldg, br, bi, t.ld, cj, cr, ci, lddx, accumulate, 0, dx_dzs_re != nullptr ? 1 : 0);
}

int cnet_ctriang_dft_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, float *dx_dz_re, float *dx_dz_im,
		float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int B, int n, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && n > 0 && n <= 46340);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && dx_dz_re && dx_dz_im && ((dx_dzs_re == nullptr) == (dx_dzs_im == nullptr)));
	CNET_CHECK_ARG(ldg >= n && lddx >= n);
	Twiddle t;
	int rc = get_triangular(n, &t);
	if (rc) return rc;
	const float *ar[2] = {g_dz_re, g_dz_re}, *ai[2] = {g_dz_im, g_dz_im}, *br[2] = {t.tri_re, t.tri_re}, *bi[2] = {t.tri_im, t.tri_im};
	float *cr[2] = {dx_dz_re, dx_dzs_re}, *ci[2] = {dx_dz_im, dx_dzs_im};
	bool cj[2] = {false, false};
	return cgemm_pair(false, false, 1, B, n, n, ar, ai, ldg, br, bi, t.ld, cj, cr, ci, lddx, accumulate, 2, dx_dzs_re != nullptr ? 1 : 0);
}

int cnet_ctriang_dft_bwd(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
		float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int B, int n, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && n > 0 && n <= 46340);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && g_dzs_re && g_dzs_im && dx_dz_re && dx_dz_im && dx_dzs_re && dx_dzs_im);
	CNET_CHECK_ARG(ldg >= n && lddx >= n);
	Twiddle t;
	int rc = get_triangular(n, &t);
	if (rc) return rc;
	const float *ar[2] = {g_dz_re, g_dzs_re}, *ai[2] = {g_dz_im, g_dzs_im}, *br[2] = {t.tri_re, t.tri_re}, *bi[2] = {t.tri_im, t.tri_im};
	float *cr[2] = {dx_dz_re, dx_dzs_re}, *ci[2] = {dx_dz_im, dx_dzs_im};
	bool cj[2] = {false, true};
	return cgemm_pair(false, false, 2, B, n, n, ar, ai, ldg, br, bi, t.ld, cj, cr, ci, lddx, accumulate, 2, 0);
}

}  // extern "C"
