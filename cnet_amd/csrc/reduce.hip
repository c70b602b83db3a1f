// Reductions on split complex planes: the row reductions of L2Out / CrossEntropy / SoftMax (sum |z|^2, argmax,
// the two inner products of the SoftMax backward) and the column reduction that sums per-sample parameter
// gradients over the batch.
//
// Row reductions: one row is owned by G wavefronts of one workgroup (G = 1 for short rows, 4 for long ones).
// Each lane strides over the row with 128-bit loads, then the 64 lanes are combined with DPP row operations
// (quad_perm, row_ror) plus one ds_swizzle and one cross-half exchange, always in the same order, and the G
// wavefront results are added through LDS in wavefront order.  No atomics anywhere: results do not depend on
// scheduling.
#include "common.hpp"
#include "rows.hpp"

#include <algorithm>

namespace {

using namespace cnet::rows;

constexpr int TPB = 256;

// Row geometry shared by the row kernels: TPB/(64*G) rows per workgroup.
#define CNET_ROW_SETUP()                                        \
	constexpr int ROWS_PER_BLOCK = TPB / (64 * G);              \
	const int lane = threadIdx.x & 63;                          \
	const int wave = threadIdx.x >> 6;                          \
	const int slot = wave / G;                                  \
	const int wig = wave % G;                                   \
	const int row_raw = blockIdx.x * ROWS_PER_BLOCK + slot;     \
	const bool live = row_raw < rows;                           \
	const int row = live ? row_raw : rows - 1;                  \
	const int t = wig * 64 + lane;                              \
	constexpr int STRIDE = 64 * G;

// sum over one row of f(re, im), 128-bit loads when V == 4
template <int V, int G, class T, class F>
__device__ __forceinline__ T row_accumulate(const float *__restrict__ pr, const float *__restrict__ pi, int cols, int t, F f, int policy = 0) {
	T acc = T();
	constexpr int STRIDE = 64 * G;
	if (V == 4) {
		for (int c = t * 4; c < cols; c += STRIDE * 4) {
			float4 a = ld4(pr + c, policy);
			float4 b = ld4(pi + c, policy);
			acc += f(a.x, b.x);
			acc += f(a.y, b.y);
			acc += f(a.z, b.z);
			acc += f(a.w, b.w);
		}
	} else {
		for (int c = t; c < cols; c += STRIDE) acc += f(pr[c], pi[c]);
	}
	return acc;
}

// ---------------------------------------------------------------------------------------------- L2Out forward
template <int V, int G>
__global__ __launch_bounds__(TPB) void l2out_fwd_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		float *__restrict__ loss, int rows, int cols, int policy) {
	__shared__ float lds[TPB / 64];
	CNET_ROW_SETUP();
	(void) STRIDE;
	float acc = row_accumulate<V, G, float>(zr + (long) row * ldz, zi + (long) row * ldz, cols, t,
			[](float a, float b) { return a * a + b * b; }, policy);
	acc = group_reduce<float, G>(acc, SumF(), lds, slot, wig, lane);
	if (live && t == 0) loss[row] = acc;
}

// ---------------------------------------------------------------------------------------------- CrossEntropy forward
// (the pass over one row is crossent_fwd_row_at in rows.hpp)
template <int V, int G, bool GRAD>
__device__ __forceinline__ void crossent_fwd_row(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		const int *__restrict__ labels, float *__restrict__ outr, float *__restrict__ outi, long ldo, float *__restrict__ s,
		float *__restrict__ loss, int *__restrict__ argmax, int rows, int cols, const GradPlanes &grad, int policy) {
	__shared__ double lds_d[TPB / 64];
	__shared__ ArgMax lds_a[TPB / 64];
	__shared__ Top2 lds_t[TPB / 64];
	CNET_ROW_SETUP();
	(void) STRIDE;
	crossent_fwd_row_at<V, G, GRAD>(zr + (long) row * ldz, zi + (long) row * ldz, row, live, t, lane, slot, wig, lds_d, lds_a, lds_t, labels, outr,
			outi, ldo, s, loss, argmax, cols, grad, policy);
}

template <int V, int G>
__global__ __launch_bounds__(TPB) void crossent_fwd_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		const int *__restrict__ labels, float *__restrict__ outr, float *__restrict__ outi, long ldo, float *__restrict__ s,
		float *__restrict__ loss, int *__restrict__ argmax, int rows, int cols, int policy) {
	crossent_fwd_row<V, G, false>(zr, zi, ldz, labels, outr, outi, ldo, s, loss, argmax, rows, cols, GradPlanes{nullptr, nullptr, nullptr, nullptr, 0}, policy);
}

// the same pass with the gradient of each row's loss written as well
template <int V, int G>
__global__ __launch_bounds__(TPB) void crossent_fwd_grad_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		const int *__restrict__ labels, float *__restrict__ outr, float *__restrict__ outi, long ldo, float *__restrict__ s,
		float *__restrict__ loss, int *__restrict__ argmax, int rows, int cols, GradPlanes grad) {
	crossent_fwd_row<V, G, true>(zr, zi, ldz, labels, outr, outi, ldo, s, loss, argmax, rows, cols, grad, 0);
}

// ---------------------------------------------------------------------------------------------- SoftMax (L2 normalise)
// impl/softmax.h:33-60 upstream
template <int V, int G>
__global__ __launch_bounds__(TPB) void l2norm_fwd_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		float *__restrict__ yr, float *__restrict__ yi, long ldy, float *__restrict__ s, int rows, int cols) {
	__shared__ double lds_d[TPB / 64];
	CNET_ROW_SETUP();
	const float *pr = zr + (long) row * ldz, *pi = zi + (long) row * ldz;
	double sum = row_accumulate<V, G, double>(pr, pi, cols, t,
			[](float a, float b) { return (double) a * (double) a + (double) b * (double) b; });
	sum = group_reduce<double, G>(sum, SumD(), lds_d, slot, wig, lane);
	double nrm = sqrt(sum);
	if (nrm <= 1.0e-15) nrm = 1.0e-15;
	if ((float) (nrm * nrm * nrm) < 1.0e-15f) nrm = 1.0e-15;
	const double inv = 1.0 / nrm;
	if (!live) return;
	float *qr = yr + (long) row * ldy, *qi = yi + (long) row * ldy;
	if (V == 4) {
		for (int c = t * 4; c < cols; c += STRIDE * 4) {
			float4 a = *reinterpret_cast<const float4 *>(pr + c);
			float4 b = *reinterpret_cast<const float4 *>(pi + c);
			*reinterpret_cast<float4 *>(qr + c) =
					make_float4((float) (a.x * inv), (float) (a.y * inv), (float) (a.z * inv), (float) (a.w * inv));
			*reinterpret_cast<float4 *>(qi + c) =
					make_float4((float) (b.x * inv), (float) (b.y * inv), (float) (b.z * inv), (float) (b.w * inv));
		}
	} else {
		for (int c = t; c < cols; c += STRIDE) {
			qr[c] = (float) (pr[c] * inv);
			qi[c] = (float) (pi[c] * inv);
		}
	}
	if (t == 0 && s) s[row] = (float) sum;
}

// Closed form of the chain rule of impl/cfunc.h:290-325 with the Jacobians of impl/softmax.h:62-73 upstream:
//   A = sum_j G_j z_j + sum_j Gs_j conj(z_j)
//   dz_i  = G_i /sqrt(S) - conj(z_i) A / (2 S^1.5)
//   dzs_i = Gs_i/sqrt(S) - z_i       A / (2 S^1.5)
// SYM: the incoming pair is conjugate (gs = conj(g)): the gs planes are not read, and the dz* planes of the result are
// written only when given (ds_re != nullptr).  Same arithmetic otherwise, so the bits agree with the general kernel.
template <int V, int G, bool SYM>
__global__ __launch_bounds__(TPB) void l2norm_bwd_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		const float *__restrict__ s, const float *__restrict__ g_re, const float *__restrict__ g_im,
		const float *__restrict__ gs_re, const float *__restrict__ gs_im, long ldg, float *__restrict__ d_re,
		float *__restrict__ d_im, float *__restrict__ ds_re, float *__restrict__ ds_im, long ldd, int rows, int cols,
		int accumulate) {
	__shared__ Cplx4 lds_c[TPB / 64];
	CNET_ROW_SETUP();
	const float *pzr = zr + (long) row * ldz, *pzi = zi + (long) row * ldz;
	const float *pgr = g_re + (long) row * ldg, *pgi = g_im + (long) row * ldg;
	const float *psr = SYM ? pgr : gs_re + (long) row * ldg, *psi = SYM ? pgi : gs_im + (long) row * ldg;
	const bool stars = !SYM || ds_re != nullptr;
	float *q0 = d_re + (long) row * ldd, *q1 = d_im + (long) row * ldd;
	float *q2 = stars ? ds_re + (long) row * ldd : nullptr, *q3 = stars ? ds_im + (long) row * ldd : nullptr;
	constexpr int W = V;  // columns per thread and step
	Cplx4 acc = {0.f, 0.f, 0.f, 0.f};  // a,b: G z   c,d: Gs conj z
	for (int c = t * W; c < cols; c += STRIDE * W) {
		float a[W], b[W], gr[W], gi[W], sr[W], si[W];
		if (W == 4) {
			*reinterpret_cast<float4 *>(a) = *reinterpret_cast<const float4 *>(pzr + c);
			*reinterpret_cast<float4 *>(b) = *reinterpret_cast<const float4 *>(pzi + c);
			*reinterpret_cast<float4 *>(gr) = *reinterpret_cast<const float4 *>(pgr + c);
			*reinterpret_cast<float4 *>(gi) = *reinterpret_cast<const float4 *>(pgi + c);
			if (!SYM) {
				*reinterpret_cast<float4 *>(sr) = *reinterpret_cast<const float4 *>(psr + c);
				*reinterpret_cast<float4 *>(si) = *reinterpret_cast<const float4 *>(psi + c);
			}
		} else {
			a[0] = pzr[c]; b[0] = pzi[c]; gr[0] = pgr[c]; gi[0] = pgi[c];
			if (!SYM) {
				sr[0] = psr[c]; si[0] = psi[c];
			}
		}
		if (SYM) {
#pragma unroll
			for (int k = 0; k < W; ++k) {
				sr[k] = gr[k];
				si[k] = -gi[k];
			}
		}
#pragma unroll
		for (int k = 0; k < W; ++k) {
			acc.a += gr[k] * a[k] - gi[k] * b[k];
			acc.b += gr[k] * b[k] + gi[k] * a[k];
			acc.c += sr[k] * a[k] + si[k] * b[k];
			acc.d += si[k] * a[k] - sr[k] * b[k];
		}
	}
	acc = group_reduce<Cplx4, G>(acc, SumC4(), lds_c, slot, wig, lane);
	if (!live) return;
	const float S = s[row];
	double nrm = sqrt((double) S);
	if (nrm <= 1.0e-15) nrm = 1.0e-15;
	float cube = (float) (nrm * nrm * nrm);
	const float inv = (float) (1.0 / nrm);
	const float Ar = 0.5f * (acc.a + acc.c) / cube, Ai = 0.5f * (acc.b + acc.d) / cube;
	for (int c = t * W; c < cols; c += STRIDE * W) {
		float a[W], b[W], gr[W], gi[W], sr[W], si[W], o0[W], o1[W], o2[W], o3[W];
		if (W == 4) {
			*reinterpret_cast<float4 *>(a) = *reinterpret_cast<const float4 *>(pzr + c);
			*reinterpret_cast<float4 *>(b) = *reinterpret_cast<const float4 *>(pzi + c);
			*reinterpret_cast<float4 *>(gr) = *reinterpret_cast<const float4 *>(pgr + c);
			*reinterpret_cast<float4 *>(gi) = *reinterpret_cast<const float4 *>(pgi + c);
			if (!SYM) {
				*reinterpret_cast<float4 *>(sr) = *reinterpret_cast<const float4 *>(psr + c);
				*reinterpret_cast<float4 *>(si) = *reinterpret_cast<const float4 *>(psi + c);
			}
		} else {
			a[0] = pzr[c]; b[0] = pzi[c]; gr[0] = pgr[c]; gi[0] = pgi[c];
			if (!SYM) {
				sr[0] = psr[c]; si[0] = psi[c];
			}
		}
		if (SYM) {
#pragma unroll
			for (int k = 0; k < W; ++k) {
				sr[k] = gr[k];
				si[k] = -gi[k];
			}
		}
#pragma unroll
		for (int k = 0; k < W; ++k) {
			// conj(z) A = (a Ar + b Ai) + i (a Ai - b Ar) ;  z A = (a Ar - b Ai) + i (a Ai + b Ar)
			o0[k] = gr[k] * inv - (a[k] * Ar + b[k] * Ai);
			o1[k] = gi[k] * inv - (a[k] * Ai - b[k] * Ar);
			o2[k] = sr[k] * inv - (a[k] * Ar - b[k] * Ai);
			o3[k] = si[k] * inv - (a[k] * Ai + b[k] * Ar);
			if (accumulate) {
				o0[k] += q0[c + k];
				o1[k] += q1[c + k];
				if (stars) {
					o2[k] += q2[c + k];
					o3[k] += q3[c + k];
				}
			}
		}
		if (W == 4) {
			*reinterpret_cast<float4 *>(q0 + c) = *reinterpret_cast<float4 *>(o0);
			*reinterpret_cast<float4 *>(q1 + c) = *reinterpret_cast<float4 *>(o1);
			if (stars) {
				*reinterpret_cast<float4 *>(q2 + c) = *reinterpret_cast<float4 *>(o2);
				*reinterpret_cast<float4 *>(q3 + c) = *reinterpret_cast<float4 *>(o3);
			}
		} else {
			q0[c] = o0[0]; q1[c] = o1[0];
			if (stars) {
				q2[c] = o2[0]; q3[c] = o3[0];
			}
		}
	}
}

// Register-resident variants for rows of at most 64 * G * 4 * NIT columns (128-bit path): the row is read from memory
// once, held in registers across the reduction and written back normalised, so the traffic is the algorithmic one
// (the two-pass kernels above read every operand twice).  Same per-thread summation order as the two-pass kernels.
template <int G, int NIT>
__global__ __launch_bounds__(TPB) void l2norm_fwd_reg_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		float *__restrict__ yr, float *__restrict__ yi, long ldy, float *__restrict__ s, int rows, int cols, int policy) {
	__shared__ double lds_d[TPB / 64];
	CNET_ROW_SETUP();
	const float *pr = zr + (long) row * ldz, *pi = zi + (long) row * ldz;
	float4 a[NIT], b[NIT];
#pragma unroll
	for (int k = 0; k < NIT; ++k) {
		const int c = (t + k * STRIDE) * 4;
		a[k] = b[k] = make_float4(0.f, 0.f, 0.f, 0.f);
		if (c < cols) {
			a[k] = ld4(pr + c, policy);
			b[k] = ld4(pi + c, policy);
		}
	}
	double sum = 0.0;
	auto sq = [](float x, float y) { return (double) x * (double) x + (double) y * (double) y; };
#pragma unroll
	for (int k = 0; k < NIT; ++k) {
		if ((t + k * STRIDE) * 4 < cols) {
			sum += sq(a[k].x, b[k].x);
			sum += sq(a[k].y, b[k].y);
			sum += sq(a[k].z, b[k].z);
			sum += sq(a[k].w, b[k].w);
		}
	}
	sum = group_reduce<double, G>(sum, SumD(), lds_d, slot, wig, lane);
	double nrm = sqrt(sum);
	if (nrm <= 1.0e-15) nrm = 1.0e-15;
	if ((float) (nrm * nrm * nrm) < 1.0e-15f) nrm = 1.0e-15;
	const double inv = 1.0 / nrm;
	if (!live) return;
	float *qr = yr + (long) row * ldy, *qi = yi + (long) row * ldy;
#pragma unroll
	for (int k = 0; k < NIT; ++k) {
		const int c = (t + k * STRIDE) * 4;
		if (c < cols) {
			st4(qr + c, make_float4((float) (a[k].x * inv), (float) (a[k].y * inv), (float) (a[k].z * inv), (float) (a[k].w * inv)), policy);
			st4(qi + c, make_float4((float) (b[k].x * inv), (float) (b[k].y * inv), (float) (b[k].z * inv), (float) (b[k].w * inv)), policy);
		}
	}
	if (t == 0 && s) s[row] = (float) sum;
}

template <int G, int NIT, bool SYM>
__global__ __launch_bounds__(TPB) void l2norm_bwd_reg_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		const float *__restrict__ s, const float *__restrict__ g_re, const float *__restrict__ g_im,
		const float *__restrict__ gs_re, const float *__restrict__ gs_im, long ldg, float *__restrict__ d_re,
		float *__restrict__ d_im, float *__restrict__ ds_re, float *__restrict__ ds_im, long ldd, int rows, int cols,
		int accumulate, int policy) {
	__shared__ Cplx4 lds_c[TPB / 64];
	CNET_ROW_SETUP();
	const float *src[6] = {zr + (long) row * ldz, zi + (long) row * ldz, g_re + (long) row * ldg, g_im + (long) row * ldg,
			SYM ? nullptr : gs_re + (long) row * ldg, SYM ? nullptr : gs_im + (long) row * ldg};
	const bool stars = !SYM || ds_re != nullptr;
	float *dst[4] = {d_re + (long) row * ldd, d_im + (long) row * ldd, stars ? ds_re + (long) row * ldd : nullptr,
			stars ? ds_im + (long) row * ldd : nullptr};
	constexpr int NSRC = SYM ? 4 : 6;
	float v[NIT][6][4];  // [chunk][z_re, z_im, g_re, g_im, gs_re, gs_im][column]
#pragma unroll
	for (int k = 0; k < NIT; ++k) {
		const int c = (t + k * STRIDE) * 4;
#pragma unroll
		for (int p = 0; p < NSRC; ++p) {
			float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
			if (c < cols) x = ld4(src[p] + c, policy);
			v[k][p][0] = x.x;
			v[k][p][1] = x.y;
			v[k][p][2] = x.z;
			v[k][p][3] = x.w;
		}
		if (SYM) {
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				v[k][4][q] = v[k][2][q];
				v[k][5][q] = -v[k][3][q];
			}
		}
	}
	Cplx4 acc = {0.f, 0.f, 0.f, 0.f};  // a,b: G z   c,d: Gs conj z
#pragma unroll
	for (int k = 0; k < NIT; ++k) {
		if ((t + k * STRIDE) * 4 < cols) {
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				const float a = v[k][0][q], b = v[k][1][q], gr = v[k][2][q], gi = v[k][3][q], sr = v[k][4][q], si = v[k][5][q];
				acc.a += gr * a - gi * b;
				acc.b += gr * b + gi * a;
				acc.c += sr * a + si * b;
				acc.d += si * a - sr * b;
			}
		}
	}
	acc = group_reduce<Cplx4, G>(acc, SumC4(), lds_c, slot, wig, lane);
	if (!live) return;
	const float S = s[row];
	double nrm = sqrt((double) S);
	if (nrm <= 1.0e-15) nrm = 1.0e-15;
	float cube = (float) (nrm * nrm * nrm);
	const float inv = (float) (1.0 / nrm);
	const float Ar = 0.5f * (acc.a + acc.c) / cube, Ai = 0.5f * (acc.b + acc.d) / cube;
#pragma unroll
	for (int k = 0; k < NIT; ++k) {
		const int c = (t + k * STRIDE) * 4;
		if (c < cols) {
			float o[4][4];
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				const float a = v[k][0][q], b = v[k][1][q], gr = v[k][2][q], gi = v[k][3][q], sr = v[k][4][q], si = v[k][5][q];
				o[0][q] = gr * inv - (a * Ar + b * Ai);
				o[1][q] = gi * inv - (a * Ai - b * Ar);
				o[2][q] = sr * inv - (a * Ar - b * Ai);
				o[3][q] = si * inv - (a * Ai + b * Ar);
			}
#pragma unroll
			for (int p = 0; p < 4; ++p) {
				if (p >= 2 && !stars) continue;
				float4 w = make_float4(o[p][0], o[p][1], o[p][2], o[p][3]);
				if (accumulate) {
					const float4 old = *reinterpret_cast<const float4 *>(dst[p] + c);
					w.x += old.x;
					w.y += old.y;
					w.z += old.z;
					w.w += old.w;
				}
				st4(dst[p] + c, w, policy);
			}
		}
	}
}

// ---------------------------------------------------------------------------------------------- batch (column) sum
// stage 1: workgroup = 64 column groups (V columns each) x 4 row lanes, blockIdx.y = slab of rows; the four row lanes
// are added through LDS in lane order; partial[slab][cols]
constexpr int CS_X = 64, CS_Y = 4;

template <int V>
__global__ __launch_bounds__(TPB) void colsum_partial_kernel(const float *__restrict__ src, long ld, float *__restrict__ partial,
		int rows, int cols, int rows_per_slab, int policy) {
	__shared__ float red[CS_Y][CS_X * V];
	const int tx = threadIdx.x % CS_X, ty = threadIdx.x / CS_X;
	// the groups of V columns are dealt evenly to the column blocks of the launch (n = 784: four blocks of 49 groups, not
	// three of 64 and one of 4, whose workgroups would sit idle beside full ones)
	const int per_block = ((cols + V - 1) / V + (int) gridDim.x - 1) / (int) gridDim.x;
	const long col = ((long) blockIdx.x * per_block + tx) * V;
	const bool live = tx < per_block && col < cols;
	const int r0 = blockIdx.y * rows_per_slab, r1 = min(rows, r0 + rows_per_slab);
	float acc[V];
#pragma unroll
	for (int k = 0; k < V; ++k) acc[k] = 0.f;
	if (live) {
		int r = r0 + ty;
		if (V == 4) {
			// eight rows are requested before the first is added (same order of additions, more loads in flight)
			constexpr int U = 8;
			for (; r + (U - 1) * CS_Y < r1; r += U * CS_Y) {
				float4 v[U];
#pragma unroll
				for (int u = 0; u < U; ++u) v[u] = ld4(src + (long) (r + u * CS_Y) * ld + col, policy);
#pragma unroll
				for (int u = 0; u < U; ++u) {
					acc[0] += v[u].x;
					acc[1 % V] += v[u].y;
					acc[2 % V] += v[u].z;
					acc[3 % V] += v[u].w;
				}
			}
		}
		for (; r < r1; r += CS_Y) {
			if (V == 4) {
				float4 v = ld4(src + (long) r * ld + col, policy);
				acc[0] += v.x;
				acc[1 % V] += v.y;
				acc[2 % V] += v.z;
				acc[3 % V] += v.w;
			} else {
				acc[0] += src[(long) r * ld + col];
			}
		}
	}
#pragma unroll
	for (int k = 0; k < V; ++k) red[ty][tx * V + k] = acc[k];
	__syncthreads();
	if (ty == 0 && live) {
#pragma unroll
		for (int k = 0; k < V; ++k)
			partial[(long) blockIdx.y * cols + col + k] = ((red[0][tx * V + k] + red[1][tx * V + k]) + red[2][tx * V + k]) + red[3][tx * V + k];
	}
}

// Second stage: FINAL_COLS columns per workgroup x FINAL_LANES lanes that each add one contiguous part of the slabs in order;
// the lanes' sums are then added in lane order.  Few slabs: 64 columns x 4 lanes.  Many (more than 32): 16 columns x 64
// lanes, which for 128 slabs is two loads per lane and, at 4096 columns, 256 workgroups instead of 64 (the kernel is all
// latency: 2 MiB to read behind a launch).
template <int FINAL_LANES, int FINAL_COLS>
__global__ __launch_bounds__(FINAL_LANES * FINAL_COLS) void colsum_final_kernel(const float *__restrict__ partial, int nslabs, int cols,
		float *__restrict__ dst, int accumulate) {
	__shared__ float red[FINAL_LANES][FINAL_COLS];
	const int tx = threadIdx.x % FINAL_COLS, ty = threadIdx.x / FINAL_COLS;
	const int c = blockIdx.x * FINAL_COLS + tx;
	const bool live = c < cols;
	const int per = (nslabs + FINAL_LANES - 1) / FINAL_LANES, k0 = min(nslabs, ty * per), k1 = min(nslabs, k0 + per);
	red[ty][tx] = live ? cnet::ordered_sum(partial + (long) k0 * cols + c, cols, k1 - k0) : 0.f;
	__syncthreads();
	if (ty == 0 && live) {
		float s = red[0][tx];
#pragma unroll 8
		for (int l = 1; l < FINAL_LANES; ++l) s += red[l][tx];
		dst[c] = accumulate ? dst[c] + s : s;
	}
}

inline bool mult4(long a, long b = 0, long c = 0, long d = 0) { return !(a % 4) && !(b % 4) && !(c % 4) && !(d % 4); }

// Slabs of rows for the two-stage column sum: four or eight workgroups per compute unit, at most 256 slabs.
struct ColsumPlan {
	int V, nslabs, rows_per_slab;
	long col_blocks;
};
inline ColsumPlan plan_colsum(int rows, int cols, bool vec) {
	ColsumPlan p;
	p.V = vec ? 4 : 1;
	p.col_blocks = ((long) cols / p.V + CS_X - 1) / CS_X;
	// a large plane (64 MiB and more) is better served by eight workgroups per unit (27 -> 23 us at 8192 x 4096), a small
	// one by fewer slabs for the second stage to add
	const long per_cu = (long) rows * cols >= (1L << 24) ? 8 : 4;
	int nslabs = (int) std::max(1L, std::min(256L, per_cu * cnet::rt().prop.multiProcessorCount / p.col_blocks));
	nslabs = std::min(nslabs, (rows + CS_Y - 1) / CS_Y);
	p.rows_per_slab = (rows + nslabs - 1) / nslabs;
	p.nslabs = (rows + p.rows_per_slab - 1) / p.rows_per_slab;
	return p;
}

// Partial sums of cnet_batch_sum_noalloc: part of the library's image on every device it is loaded on, so the call
// needs no allocation.  In host code the array's name is only a handle for hipGetSymbolAddress: kernels get the device
// address that was looked up once per device (g_static_partial).
constexpr long kStaticPartialFloats = 512 * 1024;  // 2 MiB
__device__ __align__(256) float static_partial[kStaticPartialFloats];
constexpr int kMaxDevices = 64;
float *g_static_partial[kMaxDevices] = {};

}  // namespace

namespace cnet {

// Called by cnet_init with `device` current: looks up this device's copy of the static partial-sum array.
int init_static_scratch(int device) {
	if (device < 0 || device >= kMaxDevices) return fail(CNET_ERR_INVALID_ARGUMENT, "cnet_init: device %d beyond the %d the library keeps state for", device, kMaxDevices);
	if (g_static_partial[device]) return CNET_OK;
	float *ptr = nullptr;
	CNET_HIP(hipGetSymbolAddress((void **) &ptr, HIP_SYMBOL(static_partial)));
	if (!ptr) return fail(CNET_ERR_HIP, "cnet_init: hipGetSymbolAddress returned no address for the static scratch array");
	g_static_partial[device] = ptr;
	return CNET_OK;
}

}  // namespace cnet

using namespace cnet;

// rows short enough for one wavefront each get four rows per workgroup; long rows get the whole workgroup
#define CNET_ROW_LAUNCH(KERNEL, VEC_OK, ...)                                                                          \
	do {                                                                                                              \
		const bool wide = cols > 2048;                                                                                \
		const int rpb = wide ? 1 : TPB / 64;                                                                          \
		dim3 grid((unsigned) ((rows + rpb - 1) / rpb));                                                               \
		if (VEC_OK) {                                                                                                 \
			if (wide) hipLaunchKernelGGL((KERNEL<4, 4>), grid, dim3(TPB), 0, rt().stream, __VA_ARGS__);               \
			else hipLaunchKernelGGL((KERNEL<4, 1>), grid, dim3(TPB), 0, rt().stream, __VA_ARGS__);                    \
		} else {                                                                                                      \
			if (wide) hipLaunchKernelGGL((KERNEL<1, 4>), grid, dim3(TPB), 0, rt().stream, __VA_ARGS__);               \
			else hipLaunchKernelGGL((KERNEL<1, 1>), grid, dim3(TPB), 0, rt().stream, __VA_ARGS__);                    \
		}                                                                                                             \
		CNET_LAUNCH_CHECK();                                                                                          \
	} while (0)

// register-resident row kernels: NIT 128-bit chunks per thread and plane cover the row
#define CNET_ROW_LAUNCH_REG(KERNEL, NIT_, ...)                                                                       \
	do {                                                                                                              \
		const bool wide = cols > 2048;                                                                                \
		const int rpb = wide ? 1 : TPB / 64;                                                                          \
		dim3 grid((unsigned) ((rows + rpb - 1) / rpb));                                                               \
		if (wide) hipLaunchKernelGGL((KERNEL<4, NIT_>), grid, dim3(TPB), 0, rt().stream, __VA_ARGS__);                \
		else hipLaunchKernelGGL((KERNEL<1, NIT_>), grid, dim3(TPB), 0, rt().stream, __VA_ARGS__);                     \
		CNET_LAUNCH_CHECK();                                                                                          \
	} while (0)

// chunks of 4 columns each thread must hold so that its group (64 lanes, x4 wavefronts for wide rows) covers a row
static inline int chunks_per_thread(int cols) { return (cols + (cols > 2048 ? 1024 : 256) - 1) / (cols > 2048 ? 1024 : 256); }

template <bool SYM>
static int l2norm_bwd_dispatch(const float *z_re, const float *z_im, int64_t ldz, const float *s, const float *g_dz_re,
		const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg, float *dz_dz_re, float *dz_dz_im,
		float *dz_dzs_re, float *dz_dzs_im, int64_t lddz, int rows, int cols, int accumulate) {
	const bool vec = mult4(cols, ldz, ldg, lddz) && aligned16(z_re) && aligned16(z_im) && aligned16(g_dz_re) && aligned16(g_dz_im) &&
			aligned16(g_dzs_re) && aligned16(g_dzs_im) && aligned16(dz_dz_re) && aligned16(dz_dz_im) && aligned16(dz_dzs_re) &&
			aligned16(dz_dzs_im);
	const int nit = chunks_per_thread(cols);
	const bool wide = cols > 2048;
	const int rpb = wide ? 1 : TPB / 64;
	dim3 grid((unsigned) ((rows + rpb - 1) / rpb));
	// z, g (both halves unless the pair is conjugate) and the planes of the result
	const int policy = stream_policy(SYM ? ST_LOADS : ST_BOTH, (SYM ? 4 : 6) + (SYM && !dz_dzs_re ? 2 : 4), (long) rows * cols);
#define CNET_L2N_ARGS z_re, z_im, (long) ldz, s, g_dz_re, g_dz_im, g_dzs_re, g_dzs_im, (long) ldg, dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im, (long) lddz, rows, cols, accumulate
	if (vec && nit <= 4) {
		if (nit <= 2) {
			if (wide) hipLaunchKernelGGL((l2norm_bwd_reg_kernel<4, 2, SYM>), grid, dim3(TPB), 0, rt().stream, CNET_L2N_ARGS, policy);
			else hipLaunchKernelGGL((l2norm_bwd_reg_kernel<1, 2, SYM>), grid, dim3(TPB), 0, rt().stream, CNET_L2N_ARGS, policy);
		} else {
			if (wide) hipLaunchKernelGGL((l2norm_bwd_reg_kernel<4, 4, SYM>), grid, dim3(TPB), 0, rt().stream, CNET_L2N_ARGS, policy);
			else hipLaunchKernelGGL((l2norm_bwd_reg_kernel<1, 4, SYM>), grid, dim3(TPB), 0, rt().stream, CNET_L2N_ARGS, policy);
		}
	} else if (vec) {
		if (wide) hipLaunchKernelGGL((l2norm_bwd_kernel<4, 4, SYM>), grid, dim3(TPB), 0, rt().stream, CNET_L2N_ARGS);
		else hipLaunchKernelGGL((l2norm_bwd_kernel<4, 1, SYM>), grid, dim3(TPB), 0, rt().stream, CNET_L2N_ARGS);
	} else {
		if (wide) hipLaunchKernelGGL((l2norm_bwd_kernel<1, 4, SYM>), grid, dim3(TPB), 0, rt().stream, CNET_L2N_ARGS);
		else hipLaunchKernelGGL((l2norm_bwd_kernel<1, 1, SYM>), grid, dim3(TPB), 0, rt().stream, CNET_L2N_ARGS);
	}
#undef CNET_L2N_ARGS
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

extern "C" {

int cnet_l2out_fwd(const float *z_re, const float *z_im, int64_t ldz, float *loss, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols > 0);
	if (!rows) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && loss && ldz >= cols);
	const bool vec = mult4(cols, ldz) && aligned16(z_re) && aligned16(z_im);
	// a pass that only reads: beyond the cache size the loads carry the streaming hint (0.69 -> 0.82 of the peak rate at 2048
	// rows of 32768 columns, 0.77 -> 0.87 at 32768 rows of 2048)
	const int policy = stream_policy(ST_LOADS, 2, (long) rows * cols);
	CNET_ROW_LAUNCH(l2out_fwd_kernel, vec, z_re, z_im, (long) ldz, loss, rows, cols, policy);
	return CNET_OK;
}

int cnet_cross_entropy_fwd(const float *z_re, const float *z_im, int64_t ldz, const int32_t *labels, float *out_re,
		float *out_im, int64_t ldo, float *s, float *loss, int32_t *argmax, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols > 0);
	if (!rows) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && labels && s && loss && argmax && ldz >= cols);
	CNET_CHECK_ARG((out_re == nullptr) == (out_im == nullptr));
	CNET_CHECK_ARG(out_re == nullptr || ldo >= cols);
	const bool vec = mult4(cols, ldz, out_re ? ldo : 0) && aligned16(z_re) && aligned16(z_im) && aligned16(out_re) &&
			aligned16(out_im);
	// without the normalised planes the pass only reads (and reads once unless a row holds a near tie): streaming loads
	const int policy = out_re ? 0 : stream_policy(ST_LOADS, 2, (long) rows * cols);
	CNET_ROW_LAUNCH(crossent_fwd_kernel, vec, z_re, z_im, (long) ldz, labels, out_re, out_im, (long) ldo, s, loss, argmax, rows,
			cols, policy);
	return CNET_OK;
}

int cnet_cross_entropy_fwd_bwd_sym(const float *z_re, const float *z_im, int64_t ldz, const int32_t *labels, float *out_re,
		float *out_im, int64_t ldo, float *s, float *loss, int32_t *argmax, float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re,
		float *dz_dzs_im, int64_t lddz, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols > 0);
	if (!rows) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && labels && s && loss && argmax && ldz >= cols);
	CNET_CHECK_ARG((out_re == nullptr) == (out_im == nullptr));
	CNET_CHECK_ARG(out_re == nullptr || ldo >= cols);
	CNET_CHECK_ARG(dz_dz_re && dz_dz_im && ((dz_dzs_re == nullptr) == (dz_dzs_im == nullptr)) && lddz >= cols);
	const bool vec = mult4(cols, ldz, out_re ? ldo : 0, lddz) && aligned16(z_re) && aligned16(z_im) && aligned16(out_re) &&
			aligned16(out_im) && aligned16(dz_dz_re) && aligned16(dz_dz_im) && aligned16(dz_dzs_re) && aligned16(dz_dzs_im);
	CNET_ROW_LAUNCH(crossent_fwd_grad_kernel, vec, z_re, z_im, (long) ldz, labels, out_re, out_im, (long) ldo, s, loss, argmax, rows,
			cols, GradPlanes{dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im, (long) lddz});
	return CNET_OK;
}

int cnet_l2norm_fwd(const float *z_re, const float *z_im, int64_t ldz, float *y_re, float *y_im, int64_t ldy, float *s,
		int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols > 0);
	if (!rows) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && y_re && y_im && ldz >= cols && ldy >= cols);
	const bool vec = mult4(cols, ldz, ldy) && aligned16(z_re) && aligned16(z_im) && aligned16(y_re) && aligned16(y_im);
	const int nit = chunks_per_thread(cols);
	if (vec && nit <= 8) {
		const int policy = stream_policy(ST_STORES, 4, (long) rows * cols);
		if (nit <= 2) CNET_ROW_LAUNCH_REG(l2norm_fwd_reg_kernel, 2, z_re, z_im, (long) ldz, y_re, y_im, (long) ldy, s, rows, cols, policy);
		else if (nit <= 4) CNET_ROW_LAUNCH_REG(l2norm_fwd_reg_kernel, 4, z_re, z_im, (long) ldz, y_re, y_im, (long) ldy, s, rows, cols, policy);
		else CNET_ROW_LAUNCH_REG(l2norm_fwd_reg_kernel, 8, z_re, z_im, (long) ldz, y_re, y_im, (long) ldy, s, rows, cols, policy);
		return CNET_OK;
	}
	CNET_ROW_LAUNCH(l2norm_fwd_kernel, vec, z_re, z_im, (long) ldz, y_re, y_im, (long) ldy, s, rows, cols);
	return CNET_OK;
}

int cnet_l2norm_bwd(const float *z_re, const float *z_im, int64_t ldz, const float *s, const float *g_dz_re,
		const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg, float *dz_dz_re, float *dz_dz_im,
		float *dz_dzs_re, float *dz_dzs_im, int64_t lddz, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols > 0);
	if (!rows) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && s && g_dz_re && g_dz_im && g_dzs_re && g_dzs_im);
	CNET_CHECK_ARG(dz_dz_re && dz_dz_im && dz_dzs_re && dz_dzs_im && ldz >= cols && ldg >= cols && lddz >= cols);
	return l2norm_bwd_dispatch<false>(z_re, z_im, ldz, s, g_dz_re, g_dz_im, g_dzs_re, g_dzs_im, ldg, dz_dz_re, dz_dz_im, dz_dzs_re,
			dz_dzs_im, lddz, rows, cols, accumulate);
}

int cnet_l2norm_bwd_sym(const float *z_re, const float *z_im, int64_t ldz, const float *s, const float *g_dz_re, const float *g_dz_im,
		int64_t ldg, float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz, int rows, int cols,
		int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols > 0);
	if (!rows) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && s && g_dz_re && g_dz_im && dz_dz_re && dz_dz_im);
	CNET_CHECK_ARG((dz_dzs_re == nullptr) == (dz_dzs_im == nullptr));
	CNET_CHECK_ARG(ldz >= cols && ldg >= cols && lddz >= cols);
	return l2norm_bwd_dispatch<true>(z_re, z_im, ldz, s, g_dz_re, g_dz_im, nullptr, nullptr, ldg, dz_dz_re, dz_dz_im, dz_dzs_re,
			dz_dzs_im, lddz, rows, cols, accumulate);
}

static int batch_sum_launch(const float *src, int64_t lds, float *dst, int rows, int cols, int accumulate, bool vec,
		const ColsumPlan &p, float *partial) {
	dim3 grid((unsigned) p.col_blocks, (unsigned) p.nslabs);
	if (vec)
		hipLaunchKernelGGL(colsum_partial_kernel<4>, grid, dim3(TPB), 0, rt().stream, src, (long) lds, partial, rows, cols, p.rows_per_slab,
				stream_policy(ST_LOADS, 1, (long) rows * cols));  // a pass that only reads: streaming loads beyond the cache size
	else
		hipLaunchKernelGGL(colsum_partial_kernel<1>, grid, dim3(TPB), 0, rt().stream, src, (long) lds, partial, rows, cols, p.rows_per_slab, 0);
	CNET_LAUNCH_CHECK();
	if (p.nslabs > 32)
		hipLaunchKernelGGL((colsum_final_kernel<64, 16>), dim3((unsigned) ((cols + 15) / 16)), dim3(1024), 0, rt().stream, partial, p.nslabs, cols, dst,
				accumulate);
	else
		hipLaunchKernelGGL((colsum_final_kernel<4, 64>), dim3((unsigned) ((cols + 63) / 64)), dim3(256), 0, rt().stream, partial, p.nslabs, cols, dst,
				accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_batch_sum(const float *src, int64_t lds, float *dst, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows > 0 && cols >= 0);
	if (!cols) return CNET_OK;
	CNET_CHECK_ARG(src && dst && lds >= cols);
	const bool vec = mult4(cols, lds) && aligned16(src);
	const ColsumPlan p = plan_colsum(rows, cols, vec);
	float *partial = (float *) workspace((size_t) p.nslabs * cols * sizeof(float));
	if (!partial) return CNET_ERR_OUT_OF_MEMORY;
	return batch_sum_launch(src, lds, dst, rows, cols, accumulate, vec, p, partial);
}

int cnet_batch_sum_noalloc(const float *src, int64_t lds, float *dst, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows > 0 && cols >= 0);
	if (!cols) return CNET_OK;
	CNET_CHECK_ARG(src && dst && lds >= cols);
	const bool vec = mult4(cols, lds) && aligned16(src);
	const ColsumPlan p = plan_colsum(rows, cols, vec);  // the same slabs as cnet_batch_sum: the same sums in the same order
	if ((long) p.nslabs * cols > kStaticPartialFloats)
		return fail(CNET_ERR_UNSUPPORTED, "cnet_batch_sum_noalloc: %d slabs x %d columns of partial sums exceed the static scratch of %ld floats; use cnet_batch_sum",
				p.nslabs, cols, kStaticPartialFloats);
	float *partial = g_static_partial[rt().device];
	if (!partial) return fail(CNET_ERR_NOT_INITIALIZED, "cnet_batch_sum_noalloc: the static scratch of device %d was not looked up", rt().device);
	// every partial sum the second kernel reads is written by the first one of this call: nothing to clear
	return batch_sum_launch(src, lds, dst, rows, cols, accumulate, vec, p, partial);
}

}  // extern "C"
