// HBM-bound elementwise kernels on split complex planes: Hadamard, CGelu, Residual, the loss backward passes,
// CInput copies, SGD update, zero fill.
//
// All of them walk a [rows x cols] region of row-major planes with per-operand leading dimensions.  One thread
// handles one group of V consecutive columns (V = 4 -> 128-bit loads and stores; V = 1 for odd shapes), so a
// wavefront touches 1 KiB of each plane per access and every byte is read and written exactly once.
#include "common.hpp"
#include "gate.hpp"

#include <algorithm>
#include <cmath>

namespace {

using cnet::gelu_slope;
using cnet::gelu_value;

constexpr int TPB = 256;

typedef float f32x4 __attribute__((ext_vector_type(4)));

// NT: the cache policy of the 128-bit accesses of a launch (see stream_policy below for how it is chosen).
//   0  plain loads and stores: launches whose operands fit the 256 MB memory-side cache, where the next kernel finds them
//   1  loads and stores carry the streaming (non-temporal) hint
//   2  plain loads, streaming stores
//   3  streaming loads, stores at device scope (sc1) without the hint
constexpr bool nt_loads(int policy) { return policy == 1 || policy == 3; }
template <int V, int NT>
__device__ __forceinline__ void ldv(float (&d)[V], const float *__restrict__ p) {
	if (V == 4) {
		const f32x4 *q = reinterpret_cast<const f32x4 *>(p);
		f32x4 t = nt_loads(NT) ? __builtin_nontemporal_load(q) : *q;
		d[0] = t.x;
		d[1 % V] = t.y;
		d[2 % V] = t.z;
		d[3 % V] = t.w;
	} else {
		d[0] = *p;
	}
}

template <int V, int NT>
__device__ __forceinline__ void stv(float *__restrict__ p, const float (&d)[V]) {
	if (V == 4) {
		f32x4 t = {d[0], d[1 % V], d[2 % V], d[3 % V]};
		// The hinted stores are written out: when the two arms of an `accumulate` branch end in the same store the compiler
		// merges them and the merged store loses the non-temporal mark (seen in the listing of every kernel that goes through
		// outv), so the builtin gave plain stores exactly where the hint was wanted.  The s_nop covers the wait state between
		// a 128-bit store and a vector instruction that overwrites its data registers, which the compiler cannot see here.
		if (NT == 1 || NT == 2)
			asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" ::"v"(p), "v"(t) : "memory");
		else if (NT == 3)
			asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(t) : "memory");
		else
			*reinterpret_cast<f32x4 *>(p) = t;
	} else {
		*p = d[0];
	}
}

// store or accumulate
template <int V, int NT>
__device__ __forceinline__ void outv(float *__restrict__ p, const float (&d)[V], int accumulate) {
	if (accumulate) {
		float o[V];
		ldv<V, NT>(o, p);
		float s[V];
#pragma unroll
		for (int k = 0; k < V; ++k) s[k] = o[k] + d[k];
		stv<V, NT>(p, s);
	} else {
		stv<V, NT>(p, d);
	}
}

struct Grad4 {
	float *dz_re, *dz_im, *dzs_re, *dzs_im;
};
struct CGrad4 {
	const float *dz_re, *dz_im, *dzs_re, *dzs_im;
};

#define CNET_ELEM_INDEX()                                                        \
	const long cv = cols / V;                                                    \
	const long idx = (long) blockIdx.x * TPB + threadIdx.x;                      \
	if (idx >= (long) rows * cv) return;                                         \
	const long row = idx / cv;                                                   \
	const long col = (idx - row * cv) * V;

// ------------------------------------------------------------------------------------------------ Hadamard
template <int V, int NT>
__global__ __launch_bounds__(TPB) void hadamard_fwd_kernel(const float *__restrict__ ur, const float *__restrict__ ui, long ldu,
		const float *__restrict__ vr, const float *__restrict__ vi, long ldv_, float *__restrict__ yr,
		float *__restrict__ yi, long ldy, int rows, int cols) {
	CNET_ELEM_INDEX();
	float a[V], b[V], c[V], d[V], pr[V], pi[V];
	ldv<V, NT>(a, ur + row * ldu + col);
	ldv<V, NT>(b, ui + row * ldu + col);
	ldv<V, false>(c, vr + row * ldv_ + col);  // may be one row shared by all rows: keep it cached
	ldv<V, false>(d, vi + row * ldv_ + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		pr[k] = a[k] * c[k] - b[k] * d[k];
		pi[k] = a[k] * d[k] + b[k] * c[k];
	}
	stv<V, NT>(yr + row * ldy + col, pr);
	stv<V, NT>(yi + row * ldy + col, pi);
}

// Both operands per-row: du = (G v, Gs conj v), dv = (G u, Gs conj u).
template <int V, int NT>
__global__ __launch_bounds__(TPB) void hadamard_bwd_kernel(const float *__restrict__ ur, const float *__restrict__ ui, long ldu,
		const float *__restrict__ vr, const float *__restrict__ vi, long ldv_, CGrad4 g, long ldg, Grad4 du, long lddu,
		Grad4 dv, long lddv, int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float a[V], b[V], c[V], d[V], gr[V], gi[V], sr[V], si[V], o[V];
	ldv<V, NT>(a, ur + row * ldu + col);
	ldv<V, NT>(b, ui + row * ldu + col);
	ldv<V, NT>(c, vr + row * ldv_ + col);
	ldv<V, NT>(d, vi + row * ldv_ + col);
	ldv<V, NT>(gr, g.dz_re + row * ldg + col);
	ldv<V, NT>(gi, g.dz_im + row * ldg + col);
	ldv<V, NT>(sr, g.dzs_re + row * ldg + col);
	ldv<V, NT>(si, g.dzs_im + row * ldg + col);
	const long ou = row * lddu + col, ov = row * lddv + col;
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = gr[k] * c[k] - gi[k] * d[k];
	outv<V, NT>(du.dz_re + ou, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = gr[k] * d[k] + gi[k] * c[k];
	outv<V, NT>(du.dz_im + ou, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = sr[k] * c[k] + si[k] * d[k];
	outv<V, NT>(du.dzs_re + ou, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = si[k] * c[k] - sr[k] * d[k];
	outv<V, NT>(du.dzs_im + ou, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = gr[k] * a[k] - gi[k] * b[k];
	outv<V, NT>(dv.dz_re + ov, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = gr[k] * b[k] + gi[k] * a[k];
	outv<V, NT>(dv.dz_im + ov, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = sr[k] * a[k] + si[k] * b[k];
	outv<V, NT>(dv.dzs_re + ov, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = si[k] * a[k] - sr[k] * b[k];
	outv<V, NT>(dv.dzs_im + ov, o, accumulate);
}

// v is one shared parameter row.  Workgroup = 64 column groups (V columns each) x 4 row lanes; blockIdx.y selects a slab
// of rows.  Each thread writes du for its rows and keeps the four dv sums of those rows in registers; the four row
// lanes are added through LDS in lane order and partial[slab][plane][cols] goes to the workspace; a second kernel adds
// the slabs in slab order.  Deterministic: no atomics, fixed summation tree.
constexpr int CS_X = cnet::GATE_CS_X, CS_Y = cnet::GATE_CS_Y;

template <int V, int NT>
__global__ __launch_bounds__(TPB) void hadamard_bwd_shared_kernel(const float *__restrict__ ur, const float *__restrict__ ui,
		long ldu, const float *__restrict__ vr, const float *__restrict__ vi, CGrad4 g, long ldg, Grad4 du, long lddu,
		float *__restrict__ partial, int rows, int cols, int rows_per_slab, int accumulate) {
	__shared__ float red[CS_Y][4][CS_X * V];
	const int tx = threadIdx.x % CS_X, ty = threadIdx.x / CS_X;
	// the groups of V columns are dealt evenly to the column blocks of the launch (n = 784: four blocks of 49 groups, not
	// three of 64 and one of 4, whose workgroups would sit idle beside full ones)
	const int per_block = ((cols + V - 1) / V + (int) gridDim.x - 1) / (int) gridDim.x;
	const long col = ((long) blockIdx.x * per_block + tx) * V;
	const bool live = tx < per_block && col < cols;
	const int slab = blockIdx.y;
	const int r0 = slab * rows_per_slab;
	const int r1 = min(rows, r0 + rows_per_slab);
	float acc[4][V];
#pragma unroll
	for (int p = 0; p < 4; ++p)
#pragma unroll
		for (int k = 0; k < V; ++k) acc[p][k] = 0.f;
	if (live) {
		float c[V], d[V];
		ldv<V, false>(c, vr + col);
		ldv<V, false>(d, vi + col);
		for (int row = r0 + ty; row < r1; row += CS_Y) {
			float a[V], b[V], gr[V], gi[V], sr[V], si[V], o[V];
			ldv<V, NT>(a, ur + (long) row * ldu + col);
			ldv<V, NT>(b, ui + (long) row * ldu + col);
			ldv<V, NT>(gr, g.dz_re + (long) row * ldg + col);
			ldv<V, NT>(gi, g.dz_im + (long) row * ldg + col);
			ldv<V, NT>(sr, g.dzs_re + (long) row * ldg + col);
			ldv<V, NT>(si, g.dzs_im + (long) row * ldg + col);
			const long ou = (long) row * lddu + col;
#pragma unroll
			for (int k = 0; k < V; ++k) o[k] = gr[k] * c[k] - gi[k] * d[k];
			outv<V, NT>(du.dz_re + ou, o, accumulate);
#pragma unroll
			for (int k = 0; k < V; ++k) o[k] = gr[k] * d[k] + gi[k] * c[k];
			outv<V, NT>(du.dz_im + ou, o, accumulate);
#pragma unroll
			for (int k = 0; k < V; ++k) o[k] = sr[k] * c[k] + si[k] * d[k];
			outv<V, NT>(du.dzs_re + ou, o, accumulate);
#pragma unroll
			for (int k = 0; k < V; ++k) o[k] = si[k] * c[k] - sr[k] * d[k];
			outv<V, NT>(du.dzs_im + ou, o, accumulate);
#pragma unroll
			for (int k = 0; k < V; ++k) {
				acc[0][k] += gr[k] * a[k] - gi[k] * b[k];
				acc[1][k] += gr[k] * b[k] + gi[k] * a[k];
				acc[2][k] += sr[k] * a[k] + si[k] * b[k];
				acc[3][k] += si[k] * a[k] - sr[k] * b[k];
			}
		}
	}
#pragma unroll
	for (int p = 0; p < 4; ++p)
#pragma unroll
		for (int k = 0; k < V; ++k) red[ty][p][tx * V + k] = acc[p][k];
	__syncthreads();
	if (ty == 0 && live) {
#pragma unroll
		for (int p = 0; p < 4; ++p) {
			float t[V];
#pragma unroll
			for (int k = 0; k < V; ++k) t[k] = ((red[0][p][tx * V + k] + red[1][p][tx * V + k]) + red[2][p][tx * V + k]) + red[3][p][tx * V + k];
			stv<V, NT>(partial + ((long) slab * 4 + p) * cols + col, t);
		}
	}
}

// dst[p][c] (+)= sum over slabs of partial[slab][p][c], slabs added in index order.
// SLAB_COLS (plane, column) pairs per workgroup x SLAB_LANES lanes that each add one contiguous part of the slabs in order; the
// lanes' sums are then added in lane order.  Few slabs: 64 pairs x 4 lanes; more than 32: 16 pairs x 64 lanes (two loads
// per lane for 128 slabs, four times as many workgroups: the kernel is all latency).
template <int SLAB_LANES, int SLAB_COLS>
__global__ __launch_bounds__(SLAB_LANES * SLAB_COLS) void slab_sum_kernel(const float *__restrict__ partial, int nslabs, int nplanes, int cols,
		Grad4 dst, int accumulate) {
	__shared__ float red[SLAB_LANES][SLAB_COLS];
	const int tx = threadIdx.x % SLAB_COLS, ty = threadIdx.x / SLAB_COLS;
	const long idx = (long) blockIdx.x * SLAB_COLS + tx;
	const bool live = idx < (long) nplanes * cols;
	const int p = live ? (int) (idx / cols) : 0;
	const int c = live ? (int) (idx - (long) p * cols) : 0;
	const int per = (nslabs + SLAB_LANES - 1) / SLAB_LANES, k0 = min(nslabs, ty * per), k1 = min(nslabs, k0 + per);
	red[ty][tx] = live ? cnet::ordered_sum(partial + ((long) k0 * nplanes + p) * cols + c, (long) nplanes * cols, k1 - k0) : 0.f;
	__syncthreads();
	if (ty == 0 && live) {
		float s = red[0][tx];
#pragma unroll 8
		for (int l = 1; l < SLAB_LANES; ++l) s += red[l][tx];
		float *out = p == 0 ? dst.dz_re : (p == 1 ? dst.dz_im : (p == 2 ? dst.dzs_re : dst.dzs_im));
		out[c] = accumulate ? out[c] + s : s;
	}
}

// ------------------------------------------------------------------------------------------------ CGelu
// tanh-GELU on each real plane (impl/relu.h:119-131 upstream).
template <int V, int NT>
__global__ __launch_bounds__(TPB) void gelu_fwd_kernel(const float *__restrict__ xr, const float *__restrict__ xi, long ldx,
		float *__restrict__ yr, float *__restrict__ yi, long ldy, int rows, int cols) {
	CNET_ELEM_INDEX();
	float a[V], b[V];
	ldv<V, NT>(a, xr + row * ldx + col);
	ldv<V, NT>(b, xi + row * ldx + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		a[k] = gelu_value(a[k]);
		b[k] = gelu_value(b[k]);
	}
	stv<V, NT>(yr + row * ldy + col, a);
	stv<V, NT>(yi + row * ldy + col, b);
}

// dz = G s + Gs d ; dzs = G d + Gs s ; s = (g'(x)+g'(y))/2, d = (g'(x)-g'(y))/2   (impl/relu.h:144-166 upstream)
template <int V, int NT>
__global__ __launch_bounds__(TPB) void gelu_bwd_kernel(const float *__restrict__ xr, const float *__restrict__ xi, long ldx,
		CGrad4 g, long ldg, Grad4 dx, long lddx, int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float a[V], b[V], gr[V], gi[V], sr[V], si[V], s[V], d[V], o[V];
	ldv<V, NT>(a, xr + row * ldx + col);
	ldv<V, NT>(b, xi + row * ldx + col);
	ldv<V, NT>(gr, g.dz_re + row * ldg + col);
	ldv<V, NT>(gi, g.dz_im + row * ldg + col);
	ldv<V, NT>(sr, g.dzs_re + row * ldg + col);
	ldv<V, NT>(si, g.dzs_im + row * ldg + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		float px = 0.5f * gelu_slope(a[k]), py = 0.5f * gelu_slope(b[k]);
		s[k] = px + py;
		d[k] = px - py;
	}
	const long off = row * lddx + col;
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = gr[k] * s[k] + sr[k] * d[k];
	outv<V, NT>(dx.dz_re + off, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = gi[k] * s[k] + si[k] * d[k];
	outv<V, NT>(dx.dz_im + off, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = gr[k] * d[k] + sr[k] * s[k];
	outv<V, NT>(dx.dzs_re + off, o, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) o[k] = gi[k] * d[k] + si[k] * s[k];
	outv<V, NT>(dx.dzs_im + off, o, accumulate);
}

// Hadamard followed by CGelu in one pass: h = u .* v and a = gelu(h) are both written (the backward pass needs h), u and v
// are read once and h is not read back: 24 bytes per complex element instead of 16 + 16.
template <int V, int NT>
__global__ __launch_bounds__(TPB) void hadamard_gelu_fwd_kernel(const float *__restrict__ ur, const float *__restrict__ ui, long ldu,
		const float *__restrict__ vr, const float *__restrict__ vi, long ldv_, float *__restrict__ hr, float *__restrict__ hi, long ldh,
		float *__restrict__ yr, float *__restrict__ yi, long ldy, int rows, int cols) {
	CNET_ELEM_INDEX();
	float a[V], b[V], c[V], d[V], pr[V], pi[V];
	ldv<V, NT>(a, ur + row * ldu + col);
	ldv<V, NT>(b, ui + row * ldu + col);
	ldv<V, false>(c, vr + row * ldv_ + col);
	ldv<V, false>(d, vi + row * ldv_ + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		pr[k] = a[k] * c[k] - b[k] * d[k];
		pi[k] = a[k] * d[k] + b[k] * c[k];
	}
	stv<V, NT>(hr + row * ldh + col, pr);
	stv<V, NT>(hi + row * ldh + col, pi);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		pr[k] = gelu_value(pr[k]);
		pi[k] = gelu_value(pi[k]);
	}
	stv<V, NT>(yr + row * ldy + col, pr);
	stv<V, NT>(yi + row * ldy + col, pi);
}

// ------------------------------------------------------------------------------------------------ CRelu
// y = z where Re z > 0 and Im z > 0, else 0 (impl/relu.h:32-46 upstream); the gradients pass under the same test
// (impl/relu.h:48-63).
template <int V, int NT>
__global__ __launch_bounds__(TPB) void crelu_fwd_kernel(const float *__restrict__ xr, const float *__restrict__ xi, long ldx,
		float *__restrict__ yr, float *__restrict__ yi, long ldy, int rows, int cols) {
	CNET_ELEM_INDEX();
	float a[V], b[V];
	ldv<V, NT>(a, xr + row * ldx + col);
	ldv<V, NT>(b, xi + row * ldx + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		const bool on = a[k] > 0.f && b[k] > 0.f;
		a[k] = on ? a[k] : 0.f;
		b[k] = on ? b[k] : 0.f;
	}
	stv<V, NT>(yr + row * ldy + col, a);
	stv<V, NT>(yi + row * ldy + col, b);
}

template <int V, int NT>
__global__ __launch_bounds__(TPB) void crelu_bwd_kernel(const float *__restrict__ xr, const float *__restrict__ xi, long ldx,
		CGrad4 g, long ldg, Grad4 dx, long lddx, int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float a[V], b[V], o[V];
	ldv<V, NT>(a, xr + row * ldx + col);
	ldv<V, NT>(b, xi + row * ldx + col);
	const float *src[4] = {g.dz_re, g.dz_im, g.dzs_re, g.dzs_im};
	float *dst[4] = {dx.dz_re, dx.dz_im, dx.dzs_re, dx.dzs_im};
#pragma unroll
	for (int p = 0; p < 4; ++p) {
		ldv<V, NT>(o, src[p] + row * ldg + col);
#pragma unroll
		for (int k = 0; k < V; ++k) o[k] = (a[k] > 0.f && b[k] > 0.f) ? o[k] : 0.f;
		outv<V, NT>(dst[p] + row * lddx + col, o, accumulate);
	}
}

// ------------------------------------------------------------------------------------------------ Residual
template <int V, int NT>
__global__ __launch_bounds__(TPB) void residual_fwd_kernel(const float *__restrict__ ur, const float *__restrict__ ui, long ldu,
		const float *__restrict__ vr, const float *__restrict__ vi, long ldv_, float *__restrict__ yr,
		float *__restrict__ yi, long ldy, int rows, int cols) {
	CNET_ELEM_INDEX();
	float a[V], b[V], c[V], d[V];
	ldv<V, NT>(a, ur + row * ldu + col);
	ldv<V, NT>(b, ui + row * ldu + col);
	ldv<V, false>(c, vr + row * ldv_ + col);
	ldv<V, false>(d, vi + row * ldv_ + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		a[k] += c[k];
		b[k] += d[k];
	}
	stv<V, NT>(yr + row * ldy + col, a);
	stv<V, NT>(yi + row * ldy + col, b);
}

template <int V, int NT>
__global__ __launch_bounds__(TPB) void residual_bwd_kernel(CGrad4 g, long ldg, Grad4 du, long lddu, Grad4 dv, long lddv,
		int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float t[V];
	const long og = row * ldg + col, ou = row * lddu + col, ov = row * lddv + col;
	ldv<V, NT>(t, g.dz_re + og);
	outv<V, NT>(du.dz_re + ou, t, accumulate);
	outv<V, NT>(dv.dz_re + ov, t, accumulate);
	ldv<V, NT>(t, g.dz_im + og);
	outv<V, NT>(du.dz_im + ou, t, accumulate);
	outv<V, NT>(dv.dz_im + ov, t, accumulate);
	ldv<V, NT>(t, g.dzs_re + og);
	outv<V, NT>(du.dzs_re + ou, t, accumulate);
	outv<V, NT>(dv.dzs_re + ov, t, accumulate);
	ldv<V, NT>(t, g.dzs_im + og);
	outv<V, NT>(du.dzs_im + ou, t, accumulate);
	outv<V, NT>(dv.dzs_im + ov, t, accumulate);
}

// ------------------------------------------------------------------------------------------------ loss backward
// L2Out: dz = conj z, dzs = z  (impl/l2out.h:44-58 upstream)
template <int V, int NT>
__global__ __launch_bounds__(TPB) void l2out_bwd_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		Grad4 dz, long lddz, int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float a[V], b[V], nb[V];
	ldv<V, NT>(a, zr + row * ldz + col);
	ldv<V, NT>(b, zi + row * ldz + col);
#pragma unroll
	for (int k = 0; k < V; ++k) nb[k] = -b[k];
	const long off = row * lddz + col;
	outv<V, NT>(dz.dz_re + off, a, accumulate);
	outv<V, NT>(dz.dz_im + off, nb, accumulate);
	outv<V, NT>(dz.dzs_re + off, a, accumulate);
	outv<V, NT>(dz.dzs_im + off, b, accumulate);
}

// CrossEntropy (impl/crossent.h:82-104 upstream): assigns.  label: dzs = -z (S-m)/(m S), m = max(|z_l|^2, 1e-15);
// other entries: dzs = z/S; dz = conj(dzs).
template <int V, int NT>
__global__ __launch_bounds__(TPB) void crossent_bwd_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		const float *__restrict__ s, const int *__restrict__ labels, Grad4 dz, long lddz, int rows, int cols) {
	CNET_ELEM_INDEX();
	float a[V], b[V], o_r[V], o_i[V], n_i[V];
	ldv<V, NT>(a, zr + row * ldz + col);
	ldv<V, NT>(b, zi + row * ldz + col);
	const float S = s[row];
	const int label = labels[row];
#pragma unroll
	for (int k = 0; k < V; ++k) {
		if (col + k == label) {
			float m = (float) ((double) a[k] * (double) a[k] + (double) b[k] * (double) b[k]);
			m = (m < 1e-15f ? 1e-15f : m);
			o_r[k] = -a[k] * (S - m) / (m * S);
			o_i[k] = -b[k] * (S - m) / (m * S);
		} else {
			o_r[k] = a[k] / S;
			o_i[k] = b[k] / S;
		}
		n_i[k] = -o_i[k];
	}
	const long off = row * lddz + col;
	stv<V, NT>(dz.dzs_re + off, o_r);
	stv<V, NT>(dz.dzs_im + off, o_i);
	stv<V, NT>(dz.dz_re + off, o_r);
	stv<V, NT>(dz.dz_im + off, n_i);
}

// ------------------------------------------------------------------------------------------------ conjugate gradient pairs
// Under a real-valued loss the gradient pair of every value is conjugate: dL/dz* = conj(dL/dz).  The kernels below are
// the backward passes above for such a pair: they read the dz planes of the incoming gradient only, form the dz planes of
// the result with the arithmetic of the general kernel (operation for operation, so the bits agree with it on an exactly
// conjugate pair), and write the dz* planes as the conjugate only where the caller passes them (non-NULL): a consumer
// that is itself one of these kernels, or a conjugate-pair matrix product, never reads them.  24 bytes per complex
// element instead of 40 (CGelu, CRelu, Hadamard, SoftMax), 24 instead of 48 (Residual), 16 instead of 24 (the losses).
using cnet::Pair2;  // dz planes, and optionally the planes that receive the conjugate (gate.hpp)

// (o_r, o_i) to the dz planes and, conjugated, to the dz* planes when they are wanted
template <int V, int NT>
__device__ __forceinline__ void out_pair(const Pair2 &d, long off, const float (&o_r)[V], const float (&o_i)[V], int accumulate) {
	outv<V, NT>(d.dz_re + off, o_r, accumulate);
	outv<V, NT>(d.dz_im + off, o_i, accumulate);
	if (d.dzs_re) {
		float n_i[V];
#pragma unroll
		for (int k = 0; k < V; ++k) n_i[k] = -o_i[k];
		outv<V, NT>(d.dzs_re + off, o_r, accumulate);
		outv<V, NT>(d.dzs_im + off, n_i, accumulate);
	}
}

template <int V, int NT>
__global__ __launch_bounds__(TPB) void gelu_bwd_sym_kernel(const float *__restrict__ xr, const float *__restrict__ xi, long ldx,
		const float *__restrict__ g_re, const float *__restrict__ g_im, long ldg, Pair2 dx, long lddx, int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float a[V], b[V], gr[V], gi[V], o_r[V], o_i[V];
	ldv<V, NT>(a, xr + row * ldx + col);
	ldv<V, NT>(b, xi + row * ldx + col);
	ldv<V, NT>(gr, g_re + row * ldg + col);
	ldv<V, NT>(gi, g_im + row * ldg + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		const float px = 0.5f * gelu_slope(a[k]), py = 0.5f * gelu_slope(b[k]);
		const float s = px + py, d = px - py;
		o_r[k] = gr[k] * s + gr[k] * d;      // G s + conj(G) d
		o_i[k] = gi[k] * s + (-gi[k]) * d;
	}
	out_pair<V, NT>(dx, row * lddx + col, o_r, o_i, accumulate);
}

template <int V, int NT>
__global__ __launch_bounds__(TPB) void crelu_bwd_sym_kernel(const float *__restrict__ xr, const float *__restrict__ xi, long ldx,
		const float *__restrict__ g_re, const float *__restrict__ g_im, long ldg, Pair2 dx, long lddx, int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float a[V], b[V], o_r[V], o_i[V];
	ldv<V, NT>(a, xr + row * ldx + col);
	ldv<V, NT>(b, xi + row * ldx + col);
	ldv<V, NT>(o_r, g_re + row * ldg + col);
	ldv<V, NT>(o_i, g_im + row * ldg + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		const bool on = a[k] > 0.f && b[k] > 0.f;
		o_r[k] = on ? o_r[k] : 0.f;
		o_i[k] = on ? o_i[k] : 0.f;
	}
	out_pair<V, NT>(dx, row * lddx + col, o_r, o_i, accumulate);
}

template <int V, int NT>
__global__ __launch_bounds__(TPB) void residual_bwd_sym_kernel(const float *__restrict__ g_re, const float *__restrict__ g_im, long ldg,
		Pair2 du, long lddu, Pair2 dv, long lddv, int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float o_r[V], o_i[V];
	ldv<V, NT>(o_r, g_re + row * ldg + col);
	ldv<V, NT>(o_i, g_im + row * ldg + col);
	out_pair<V, NT>(du, row * lddu + col, o_r, o_i, accumulate);
	out_pair<V, NT>(dv, row * lddv + col, o_r, o_i, accumulate);
}

// A Residual whose result feeds two consumers: the two incoming gradients are added here (g1 first, as two passes with
// accumulation would), so du and dv are written once instead of written, read and written again
template <int V, int NT>
__global__ __launch_bounds__(TPB) void residual_bwd_sym2_kernel(const float *__restrict__ g1_re, const float *__restrict__ g1_im, long ldg1,
		const float *__restrict__ g2_re, const float *__restrict__ g2_im, long ldg2, Pair2 du, long lddu, Pair2 dv, long lddv, int rows,
		int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float o_r[V], o_i[V], p_r[V], p_i[V];
	ldv<V, NT>(o_r, g1_re + row * ldg1 + col);
	ldv<V, NT>(o_i, g1_im + row * ldg1 + col);
	ldv<V, NT>(p_r, g2_re + row * ldg2 + col);
	ldv<V, NT>(p_i, g2_im + row * ldg2 + col);
	if (accumulate) {
		// the order of two accumulating passes: (old + g1) + g2, for each destination
		const Pair2 *dst[2] = {&du, &dv};
		const long off[2] = {row * lddu + col, row * lddv + col};
#pragma unroll
		for (int d = 0; d < 2; ++d) {
			float a_r[V], a_i[V];
			ldv<V, NT>(a_r, dst[d]->dz_re + off[d]);
			ldv<V, NT>(a_i, dst[d]->dz_im + off[d]);
#pragma unroll
			for (int k = 0; k < V; ++k) {
				a_r[k] = (a_r[k] + o_r[k]) + p_r[k];
				a_i[k] = (a_i[k] + o_i[k]) + p_i[k];
			}
			stv<V, NT>(dst[d]->dz_re + off[d], a_r);
			stv<V, NT>(dst[d]->dz_im + off[d], a_i);
			if (dst[d]->dzs_re) {
				float b_r[V], b_i[V];
				ldv<V, NT>(b_r, dst[d]->dzs_re + off[d]);
				ldv<V, NT>(b_i, dst[d]->dzs_im + off[d]);
#pragma unroll
				for (int k = 0; k < V; ++k) {
					b_r[k] = (b_r[k] + o_r[k]) + p_r[k];
					b_i[k] = (b_i[k] + (-o_i[k])) + (-p_i[k]);
				}
				stv<V, NT>(dst[d]->dzs_re + off[d], b_r);
				stv<V, NT>(dst[d]->dzs_im + off[d], b_i);
			}
		}
		return;
	}
#pragma unroll
	for (int k = 0; k < V; ++k) {
		o_r[k] += p_r[k];
		o_i[k] += p_i[k];
	}
	out_pair<V, NT>(du, row * lddu + col, o_r, o_i, 0);
	out_pair<V, NT>(dv, row * lddv + col, o_r, o_i, 0);
}

// A Residual one of whose operands is the result of a CGelu: the gradient of the Residual (g1, plus g2 when it feeds two
// consumers, added as residual_bwd_sym2_kernel adds them) goes to the other operand (du) and, optionally, to the CGelu's
// result (dv); its CGelu backward at h, the CGelu's operand, goes to dh with the arithmetic of gelu_bwd_sym_kernel.  The
// gradient of the CGelu's result is not read back: 40 bytes per complex element (32 with one consumer) against 32 + 24.
template <int V, int NT, bool TWO>
__global__ __launch_bounds__(TPB) void residual_gelu_bwd_sym_kernel(const float *__restrict__ g1_re, const float *__restrict__ g1_im,
		long ldg1, const float *__restrict__ g2_re, const float *__restrict__ g2_im, long ldg2, const float *__restrict__ hr,
		const float *__restrict__ hi, long ldh, Pair2 du, long lddu, Pair2 dv, long lddv, Pair2 dh, long lddh, int rows, int cols) {
	CNET_ELEM_INDEX();
	float o_r[V], o_i[V], a[V], b[V];
	ldv<V, NT>(o_r, g1_re + row * ldg1 + col);
	ldv<V, NT>(o_i, g1_im + row * ldg1 + col);
	if (TWO) {
		float p_r[V], p_i[V];
		ldv<V, NT>(p_r, g2_re + row * ldg2 + col);
		ldv<V, NT>(p_i, g2_im + row * ldg2 + col);
#pragma unroll
		for (int k = 0; k < V; ++k) {
			o_r[k] += p_r[k];
			o_i[k] += p_i[k];
		}
	}
	ldv<V, NT>(a, hr + row * ldh + col);
	ldv<V, NT>(b, hi + row * ldh + col);
	out_pair<V, NT>(du, row * lddu + col, o_r, o_i, 0);
	if (dv.dz_re) out_pair<V, NT>(dv, row * lddv + col, o_r, o_i, 0);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		const float px = 0.5f * gelu_slope(a[k]), py = 0.5f * gelu_slope(b[k]);
		const float sm = px + py, df = px - py;
		const float q_r = o_r[k] * sm + o_r[k] * df, q_i = o_i[k] * sm + (-o_i[k]) * df;
		o_r[k] = q_r;
		o_i[k] = q_i;
	}
	out_pair<V, NT>(dh, row * lddh + col, o_r, o_i, 0);
}

// The gradient that reaches a Hadamard through a CGelu on its result, formed in place: h = u .* v is recomputed (the bits
// of the forward pass), g becomes the CGelu backward of g at h (the arithmetic of gelu_bwd_sym_kernel), and is stored to
// dh, the gradient planes of the CGelu's operand, which stay readable (skipped when dh.dz_re is NULL).
template <int V, int NT>
__device__ __forceinline__ void through_gelu(const float (&a)[V], const float (&b)[V], const float (&c)[V], const float (&d)[V],
		float (&gr)[V], float (&gi)[V], const Pair2 &dh, long off) {
#pragma unroll
	for (int k = 0; k < V; ++k) {
		const float hr = a[k] * c[k] - b[k] * d[k], hi = a[k] * d[k] + b[k] * c[k];
		const float px = 0.5f * gelu_slope(hr), py = 0.5f * gelu_slope(hi);
		const float sm = px + py, df = px - py;
		const float o_r = gr[k] * sm + gr[k] * df, o_i = gi[k] * sm + (-gi[k]) * df;
		gr[k] = o_r;
		gi[k] = o_i;
	}
	if (dh.dz_re) out_pair<V, NT>(dh, off, gr, gi, 0);
}

// du = G v, dv = G u (per-row operands).  GELU: G is first taken through a CGelu that sits on the Hadamard's result.
template <int V, int NT, bool GELU>
__global__ __launch_bounds__(TPB) void hadamard_bwd_sym_kernel(const float *__restrict__ ur, const float *__restrict__ ui, long ldu,
		const float *__restrict__ vr, const float *__restrict__ vi, long ldv_, const float *__restrict__ g_re,
		const float *__restrict__ g_im, long ldg, Pair2 dh, long lddh, Pair2 du, long lddu, Pair2 dv, long lddv, int rows, int cols,
		int accumulate) {
	CNET_ELEM_INDEX();
	float a[V], b[V], c[V], d[V], gr[V], gi[V], o_r[V], o_i[V];
	ldv<V, NT>(a, ur + row * ldu + col);
	ldv<V, NT>(b, ui + row * ldu + col);
	ldv<V, NT>(c, vr + row * ldv_ + col);
	ldv<V, NT>(d, vi + row * ldv_ + col);
	ldv<V, NT>(gr, g_re + row * ldg + col);
	ldv<V, NT>(gi, g_im + row * ldg + col);
	if (GELU) through_gelu<V, NT>(a, b, c, d, gr, gi, dh, row * lddh + col);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		o_r[k] = gr[k] * c[k] - gi[k] * d[k];
		o_i[k] = gr[k] * d[k] + gi[k] * c[k];
	}
	out_pair<V, NT>(du, row * lddu + col, o_r, o_i, accumulate);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		o_r[k] = gr[k] * a[k] - gi[k] * b[k];
		o_i[k] = gr[k] * b[k] + gi[k] * a[k];
	}
	out_pair<V, NT>(dv, row * lddv + col, o_r, o_i, accumulate);
}

// v is one shared parameter row: as hadamard_bwd_shared_kernel, two partial planes per slab
template <int V, int NT, bool GELU>
__global__ __launch_bounds__(TPB) void hadamard_bwd_shared_sym_kernel(const float *__restrict__ ur, const float *__restrict__ ui,
		long ldu, const float *__restrict__ vr, const float *__restrict__ vi, const float *__restrict__ g_re,
		const float *__restrict__ g_im, long ldg, Pair2 dh, long lddh, Pair2 du, long lddu, float *__restrict__ partial, int rows,
		int cols, int rows_per_slab, int accumulate) {
	__shared__ float red[CS_Y][2][CS_X * V];
	const int tx = threadIdx.x % CS_X, ty = threadIdx.x / CS_X;
	// the groups of V columns are dealt evenly to the column blocks of the launch (n = 784: four blocks of 49 groups, not
	// three of 64 and one of 4, whose workgroups would sit idle beside full ones)
	const int per_block = ((cols + V - 1) / V + (int) gridDim.x - 1) / (int) gridDim.x;
	const long col = ((long) blockIdx.x * per_block + tx) * V;
	const bool live = tx < per_block && col < cols;
	const int slab = blockIdx.y;
	const int r0 = slab * rows_per_slab;
	const int r1 = min(rows, r0 + rows_per_slab);
	float acc[2][V];
#pragma unroll
	for (int p = 0; p < 2; ++p)
#pragma unroll
		for (int k = 0; k < V; ++k) acc[p][k] = 0.f;
	if (live) {
		float c[V], d[V];
		ldv<V, false>(c, vr + col);
		ldv<V, false>(d, vi + col);
		for (int row = r0 + ty; row < r1; row += CS_Y) {
			float a[V], b[V], gr[V], gi[V], o_r[V], o_i[V];
			ldv<V, NT>(a, ur + (long) row * ldu + col);
			ldv<V, NT>(b, ui + (long) row * ldu + col);
			ldv<V, NT>(gr, g_re + (long) row * ldg + col);
			ldv<V, NT>(gi, g_im + (long) row * ldg + col);
			if (GELU) through_gelu<V, NT>(a, b, c, d, gr, gi, dh, (long) row * lddh + col);
#pragma unroll
			for (int k = 0; k < V; ++k) {
				o_r[k] = gr[k] * c[k] - gi[k] * d[k];
				o_i[k] = gr[k] * d[k] + gi[k] * c[k];
			}
			out_pair<V, NT>(du, (long) row * lddu + col, o_r, o_i, accumulate);
#pragma unroll
			for (int k = 0; k < V; ++k) {
				acc[0][k] += gr[k] * a[k] - gi[k] * b[k];
				acc[1][k] += gr[k] * b[k] + gi[k] * a[k];
			}
		}
	}
#pragma unroll
	for (int p = 0; p < 2; ++p)
#pragma unroll
		for (int k = 0; k < V; ++k) red[ty][p][tx * V + k] = acc[p][k];
	__syncthreads();
	if (ty == 0 && live) {
#pragma unroll
		for (int p = 0; p < 2; ++p) {
			float t[V];
#pragma unroll
			for (int k = 0; k < V; ++k) t[k] = ((red[0][p][tx * V + k] + red[1][p][tx * V + k]) + red[2][p][tx * V + k]) + red[3][p][tx * V + k];
			stv<V, NT>(partial + ((long) slab * 2 + p) * cols + col, t);
		}
	}
}

// dst.dz (+)= sum over slabs of partial[slab][re, im][c], slabs added in index order; the conjugate goes to dst.dzs when
// those planes are given
template <int SLAB_LANES, int SLAB_COLS>
__global__ __launch_bounds__(SLAB_LANES * SLAB_COLS) void slab_sum_sym_kernel(const float *__restrict__ partial, int nslabs, int cols, Pair2 dst, int accumulate) {
	__shared__ float red[SLAB_LANES][SLAB_COLS];
	const int tx = threadIdx.x % SLAB_COLS, ty = threadIdx.x / SLAB_COLS;
	const long idx = (long) blockIdx.x * SLAB_COLS + tx;
	const bool live = idx < 2L * cols;
	const int p = live ? (int) (idx / cols) : 0;
	const int c = live ? (int) (idx - (long) p * cols) : 0;
	const int per = (nslabs + SLAB_LANES - 1) / SLAB_LANES, k0 = min(nslabs, ty * per), k1 = min(nslabs, k0 + per);
	red[ty][tx] = live ? cnet::ordered_sum(partial + ((long) k0 * 2 + p) * cols + c, 2L * cols, k1 - k0) : 0.f;
	__syncthreads();
	if (ty == 0 && live) {
		float s = red[0][tx];
#pragma unroll 8
		for (int l = 1; l < SLAB_LANES; ++l) s += red[l][tx];
		float *out = p == 0 ? dst.dz_re : dst.dz_im;
		out[c] = accumulate ? out[c] + s : s;
		if (dst.dzs_re) {
			float *m = p == 0 ? dst.dzs_re : dst.dzs_im;
			const float mv = p == 0 ? s : -s;
			m[c] = accumulate ? m[c] + mv : mv;
		}
	}
}

// L2Out: dz = conj z (and dz* = z)
template <int V, int NT>
__global__ __launch_bounds__(TPB) void l2out_bwd_sym_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		Pair2 dz, long lddz, int rows, int cols, int accumulate) {
	CNET_ELEM_INDEX();
	float a[V], b[V], nb[V];
	ldv<V, NT>(a, zr + row * ldz + col);
	ldv<V, NT>(b, zi + row * ldz + col);
#pragma unroll
	for (int k = 0; k < V; ++k) nb[k] = -b[k];
	out_pair<V, NT>(dz, row * lddz + col, a, nb, accumulate);
}

// CrossEntropy: dz* as in crossent_bwd_kernel, dz = conj(dz*); assigns
template <int V, int NT>
__global__ __launch_bounds__(TPB) void crossent_bwd_sym_kernel(const float *__restrict__ zr, const float *__restrict__ zi, long ldz,
		const float *__restrict__ s, const int *__restrict__ labels, Pair2 dz, long lddz, int rows, int cols) {
	CNET_ELEM_INDEX();
	float a[V], b[V], o_r[V], n_i[V];
	ldv<V, NT>(a, zr + row * ldz + col);
	ldv<V, NT>(b, zi + row * ldz + col);
	const float S = s[row];
	const int label = labels[row];
#pragma unroll
	for (int k = 0; k < V; ++k) {
		float o_i;
		if (col + k == label) {
			float m = (float) ((double) a[k] * (double) a[k] + (double) b[k] * (double) b[k]);
			m = (m < 1e-15f ? 1e-15f : m);
			o_r[k] = -a[k] * (S - m) / (m * S);
			o_i = -b[k] * (S - m) / (m * S);
		} else {
			o_r[k] = a[k] / S;
			o_i = b[k] / S;
		}
		n_i[k] = -o_i;
	}
	out_pair<V, NT>(dz, row * lddz + col, o_r, n_i, 0);
}

// ------------------------------------------------------------------------------------------------ plumbing
template <int V, int NT>
__global__ __launch_bounds__(TPB) void copy2d_kernel(const float *__restrict__ src, long lds, float *__restrict__ dst, long ldd,
		int rows, int cols, int add) {
	CNET_ELEM_INDEX();
	float t[V];
	ldv<V, NT>(t, src + row * lds + col);
	outv<V, NT>(dst + row * ldd + col, t, add);
}

// z -= lr * dzs ; dzs = 0   (impl/cfunc.h:147-152, impl/cnet.h:413-421 upstream)
template <int V, int NT>
__global__ __launch_bounds__(TPB) void sgd_kernel(float *__restrict__ zr, float *__restrict__ zi, float *__restrict__ dr,
		float *__restrict__ di, long n, float lr, int zero_grad) {
	const long i = ((long) blockIdx.x * TPB + threadIdx.x) * V;
	if (i >= n) return;
	float a[V], b[V], c[V], d[V], z[V];
	ldv<V, NT>(a, zr + i);
	ldv<V, NT>(b, zi + i);
	ldv<V, NT>(c, dr + i);
	ldv<V, NT>(d, di + i);
#pragma unroll
	for (int k = 0; k < V; ++k) {
		a[k] -= lr * c[k];
		b[k] -= lr * d[k];
		z[k] = 0.f;
	}
	stv<V, NT>(zr + i, a);
	stv<V, NT>(zi + i, b);
	if (zero_grad) {
		stv<V, NT>(dr + i, z);
		stv<V, NT>(di + i, z);
	}
}

// m = beta m + (1 - beta) dzs ; z -= lr m / denom ; dzs = 0   (impl/cfunc.h:273-287, gpu/kernels.cpp:494-514 upstream).
// denom = 1 - beta^(t+1) arrives as a double and the quotient is formed in double, as the CPU loop does
// (pow(float, int) promotes), so the parameter gets one rounding per step.
template <int V, int NT>
__global__ __launch_bounds__(TPB) void adam_kernel(float *__restrict__ zr, float *__restrict__ zi, float *__restrict__ mr,
		float *__restrict__ mi, float *__restrict__ dr, float *__restrict__ di, long n, float lr, float beta, double denom,
		int zero_grad) {
	const long i = ((long) blockIdx.x * TPB + threadIdx.x) * V;
	if (i >= n) return;
	float a[V], b[V], c[V], d[V], e[V], f[V], z[V];
	ldv<V, NT>(a, zr + i);
	ldv<V, NT>(b, zi + i);
	ldv<V, NT>(c, mr + i);
	ldv<V, NT>(d, mi + i);
	ldv<V, NT>(e, dr + i);
	ldv<V, NT>(f, di + i);
	const float one_minus_beta = 1 - beta;
#pragma unroll
	for (int k = 0; k < V; ++k) {
		c[k] = c[k] * beta + one_minus_beta * e[k];
		d[k] = d[k] * beta + one_minus_beta * f[k];
		a[k] = (float) ((double) a[k] - (double) (lr * c[k]) / denom);
		b[k] = (float) ((double) b[k] - (double) (lr * d[k]) / denom);
		z[k] = 0.f;
	}
	stv<V, NT>(zr + i, a);
	stv<V, NT>(zi + i, b);
	stv<V, NT>(mr + i, c);
	stv<V, NT>(mi + i, d);
	if (zero_grad) {
		stv<V, NT>(dr + i, z);
		stv<V, NT>(di + i, z);
	}
}

// Several parameter tensors in one launch (a net has many small ones; a launch per tensor costs more than the update).
// blockIdx.y selects the tensor, blocks past its end leave at once.  Same arithmetic as sgd_kernel.
constexpr int SGD_MULTI_MAX = 8;
struct SgdMulti {
	float *z_re[SGD_MULTI_MAX], *z_im[SGD_MULTI_MAX], *d_re[SGD_MULTI_MAX], *d_im[SGD_MULTI_MAX];
	long n[SGD_MULTI_MAX];
	int vec[SGD_MULTI_MAX];  // tensor can take the 128-bit path
};
__global__ __launch_bounds__(TPB) void sgd_multi_kernel(SgdMulti t, float lr, int zero_grad) {
	const int k = blockIdx.y;
	const long n = t.n[k];
	float *zr = t.z_re[k], *zi = t.z_im[k], *dr = t.d_re[k], *di = t.d_im[k];
	if (t.vec[k]) {
		const long i = ((long) blockIdx.x * TPB + threadIdx.x) * 4;
		if (i >= n) return;
		float a[4], b[4], c[4], d[4], z[4] = {0.f, 0.f, 0.f, 0.f};
		ldv<4, false>(a, zr + i);
		ldv<4, false>(b, zi + i);
		ldv<4, false>(c, dr + i);
		ldv<4, false>(d, di + i);
#pragma unroll
		for (int q = 0; q < 4; ++q) {
			a[q] -= lr * c[q];
			b[q] -= lr * d[q];
		}
		stv<4, false>(zr + i, a);
		stv<4, false>(zi + i, b);
		if (zero_grad) {
			stv<4, false>(dr + i, z);
			stv<4, false>(di + i, z);
		}
	} else {
		// scalar path: four consecutive elements per thread keep the grid shape of the vector path
		const long i0 = ((long) blockIdx.x * TPB + threadIdx.x) * 4;
		for (long i = i0; i < i0 + 4 && i < n; ++i) {
			zr[i] -= lr * dr[i];
			zi[i] -= lr * di[i];
			if (zero_grad) dr[i] = di[i] = 0.f;
		}
	}
}

// dst[k][i] += src[k][i] for up to SGD_MULTI_MAX dense arrays in one launch (blockIdx.y selects the array).
struct AddMulti {
	const float *src[SGD_MULTI_MAX];
	float *dst[SGD_MULTI_MAX];
	long n[SGD_MULTI_MAX];
	int vec[SGD_MULTI_MAX];
};
__global__ __launch_bounds__(TPB) void add_multi_kernel(AddMulti t) {
	const int k = blockIdx.y;
	const long n = t.n[k];
	const float *src = t.src[k];
	float *dst = t.dst[k];
	const long i0 = ((long) blockIdx.x * TPB + threadIdx.x) * 4;
	if (i0 >= n) return;
	if (t.vec[k]) {
		float a[4], b[4];
		ldv<4, false>(a, src + i0);
		ldv<4, false>(b, dst + i0);
#pragma unroll
		for (int q = 0; q < 4; ++q) b[q] += a[q];
		stv<4, false>(dst + i0, b);
	} else {
		for (long i = i0; i < i0 + 4 && i < n; ++i) dst[i] += src[i];
	}
}

__global__ __launch_bounds__(TPB) void zero_kernel(uint4 *__restrict__ p16, long n16, unsigned char *__restrict__ tail, int ntail) {
	const long i = (long) blockIdx.x * TPB + threadIdx.x;
	if (i < n16) p16[i] = make_uint4(0, 0, 0, 0);
	if (i < ntail) tail[i] = 0;
}

inline unsigned nblocks(long work) { return (unsigned) ((work + TPB - 1) / TPB); }

inline bool all_aligned(std::initializer_list<const void *> ptrs) {
	for (const void *p : ptrs)
		if (p && !cnet::aligned16(p)) return false;
	return true;
}
inline bool all_mult4(std::initializer_list<long> v) {
	for (long x : v)
		if (x % 4) return false;
	return true;
}

}  // namespace

using namespace cnet;

// the 128-bit variant of a kernel under cache policy `pol` (0..3)
#define CNET_LAUNCH_V4(kernel, pol, ...)                                    \
	do {                                                                    \
		switch (pol) {                                                      \
		case 1: hipLaunchKernelGGL((kernel<4, 1>), __VA_ARGS__); break;     \
		case 2: hipLaunchKernelGGL((kernel<4, 2>), __VA_ARGS__); break;     \
		case 3: hipLaunchKernelGGL((kernel<4, 3>), __VA_ARGS__); break;     \
		default: hipLaunchKernelGGL((kernel<4, 0>), __VA_ARGS__); break;    \
		}                                                                   \
	} while (0)

#define CNET_GRID_2D(V) dim3(nblocks((long) rows * (cols / (V)))), dim3(TPB), 0, rt().stream

extern "C" {

int cnet_memset_zero(void *dst, size_t bytes) {
	CNET_REQUIRE_INIT();
	if (!bytes) return CNET_OK;
	CNET_CHECK_ARG(dst != nullptr);
	// a fill kernel rather than hipMemsetAsync, so the call can be captured into a HIP graph
	unsigned char *p = (unsigned char *) dst;
	size_t head = (16 - ((uintptr_t) p & 15)) & 15;
	if (head > bytes) head = bytes;
	if (head) {
		hipLaunchKernelGGL(zero_kernel, dim3(1), dim3(TPB), 0, rt().stream, (uint4 *) nullptr, 0L, p, (int) head);
		CNET_LAUNCH_CHECK();
	}
	p += head;
	bytes -= head;
	long n16 = (long) (bytes / 16);
	int ntail = (int) (bytes % 16);
	if (n16 || ntail) {
		hipLaunchKernelGGL(zero_kernel, dim3(nblocks(n16 > ntail ? n16 : ntail)), dim3(TPB), 0, rt().stream, (uint4 *) p, n16,
				p + n16 * 16, ntail);
		CNET_LAUNCH_CHECK();
	}
	return CNET_OK;
}

int cnet_hadamard_fwd(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
		float *y_re, float *y_im, int64_t ldy, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(u_re && u_im && v_re && v_im && y_re && y_im);
	CNET_CHECK_ARG(ldu >= cols && ldy >= cols && (ldv == 0 || ldv >= cols));
	const int nt = stream_policy(ST_STORES, 4 + (ldv ? 2 : 0), (long) rows * cols);
	if (all_mult4({cols, ldu, ldv, ldy}) && all_aligned({u_re, u_im, v_re, v_im, y_re, y_im}))
		CNET_LAUNCH_V4(hadamard_fwd_kernel, nt, CNET_GRID_2D(4), u_re, u_im, ldu, v_re, v_im, ldv, y_re, y_im, ldy, rows, cols);
	else
		hipLaunchKernelGGL((hadamard_fwd_kernel<1, 0>), CNET_GRID_2D(1), u_re, u_im, ldu, v_re, v_im, ldv, y_re, y_im, ldy, rows, cols);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_hadamard_bwd(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
		const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
		float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu, float *dv_dz_re,
		float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(u_re && u_im && v_re && v_im && g_dz_re && g_dz_im && g_dzs_re && g_dzs_im);
	CNET_CHECK_ARG(du_dz_re && du_dz_im && du_dzs_re && du_dzs_im && dv_dz_re && dv_dz_im && dv_dzs_re && dv_dzs_im);
	CNET_CHECK_ARG(ldu >= cols && ldg >= cols && lddu >= cols && (ldv == 0 || (ldv >= cols && lddv >= cols)));
	CGrad4 g = {g_dz_re, g_dz_im, g_dzs_re, g_dzs_im};
	Grad4 du = {du_dz_re, du_dz_im, du_dzs_re, du_dzs_im};
	Grad4 dv = {dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im};
	bool vec = all_mult4({cols, ldu, ldv, ldg, lddu, ldv ? lddv : 0}) &&
			all_aligned({u_re, u_im, v_re, v_im, g_dz_re, g_dz_im, g_dzs_re, g_dzs_im, du_dz_re, du_dz_im, du_dzs_re,
					du_dzs_im, dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im});
	const int nt = stream_policy(ST_BOTH, 10 + (ldv ? 6 : 0), (long) rows * cols);
	if (ldv != 0) {
		if (vec)
			CNET_LAUNCH_V4(hadamard_bwd_kernel, nt, CNET_GRID_2D(4), u_re, u_im, ldu, v_re, v_im, ldv, g, ldg, du, lddu, dv, lddv,
					rows, cols, accumulate);
		else
			hipLaunchKernelGGL((hadamard_bwd_kernel<1, 0>), CNET_GRID_2D(1), u_re, u_im, ldu, v_re, v_im, ldv, g, ldg, du, lddu, dv, lddv,
					rows, cols, accumulate);
		CNET_LAUNCH_CHECK();
		return CNET_OK;
	}
	// shared parameter row: slabs of rows sized so that the grid covers the chip about four times
	const int V = vec ? 4 : 1;
	const long col_blocks = ((long) cols / V + CS_X - 1) / CS_X;
	int nslabs = (int) std::max(1L, std::min(256L, 2L * rt().prop.multiProcessorCount / col_blocks));  // as in the conjugate-pair variant: the same sums
	nslabs = std::min(nslabs, (rows + CS_Y - 1) / CS_Y);
	const int rows_per_slab = (rows + nslabs - 1) / nslabs;
	nslabs = (rows + rows_per_slab - 1) / rows_per_slab;
	float *partial = (float *) workspace((size_t) nslabs * 4 * cols * sizeof(float));
	if (!partial) return CNET_ERR_OUT_OF_MEMORY;
	dim3 grid((unsigned) col_blocks, (unsigned) nslabs);
	if (vec)
		CNET_LAUNCH_V4(hadamard_bwd_shared_kernel, nt, grid, dim3(TPB), 0, rt().stream, u_re, u_im, ldu, v_re, v_im, g, ldg, du,
				lddu, partial, rows, cols, rows_per_slab, accumulate);
	else
		hipLaunchKernelGGL((hadamard_bwd_shared_kernel<1, 0>), grid, dim3(TPB), 0, rt().stream, u_re, u_im, ldu, v_re, v_im, g, ldg, du,
				lddu, partial, rows, cols, rows_per_slab, accumulate);
	CNET_LAUNCH_CHECK();
	if (nslabs > 32)
		hipLaunchKernelGGL((slab_sum_kernel<64, 16>), dim3((unsigned) ((4L * cols + 15) / 16)), dim3(1024), 0, rt().stream, partial, nslabs, 4, cols, dv, accumulate);
	else
		hipLaunchKernelGGL((slab_sum_kernel<4, 64>), dim3((unsigned) ((4L * cols + 63) / 64)), dim3(256), 0, rt().stream, partial, nslabs, 4, cols, dv, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_cgelu_fwd(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && y_re && y_im && ldx >= cols && ldy >= cols);
	const int nt = stream_policy(ST_STORES, 4, (long) rows * cols);
	if (all_mult4({cols, ldx, ldy}) && all_aligned({x_re, x_im, y_re, y_im}))
		CNET_LAUNCH_V4(gelu_fwd_kernel, nt, CNET_GRID_2D(4), x_re, x_im, ldx, y_re, y_im, ldy, rows, cols);
	else
		hipLaunchKernelGGL((gelu_fwd_kernel<1, 0>), CNET_GRID_2D(1), x_re, x_im, ldx, y_re, y_im, ldy, rows, cols);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_cgelu_bwd(const float *x_re, const float *x_im, int64_t ldx, const float *g_dz_re, const float *g_dz_im,
		const float *g_dzs_re, const float *g_dzs_im, int64_t ldg, float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re,
		float *dx_dzs_im, int64_t lddx, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && g_dz_re && g_dz_im && g_dzs_re && g_dzs_im && dx_dz_re && dx_dz_im && dx_dzs_re && dx_dzs_im);
	CNET_CHECK_ARG(ldx >= cols && ldg >= cols && lddx >= cols);
	CGrad4 g = {g_dz_re, g_dz_im, g_dzs_re, g_dzs_im};
	Grad4 dx = {dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im};
	const int nt = stream_policy(ST_BOTH, 10, (long) rows * cols);
	if (all_mult4({cols, ldx, ldg, lddx}) &&
			all_aligned({x_re, x_im, g_dz_re, g_dz_im, g_dzs_re, g_dzs_im, dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im}))
		CNET_LAUNCH_V4(gelu_bwd_kernel, nt, CNET_GRID_2D(4), x_re, x_im, ldx, g, ldg, dx, lddx, rows, cols, accumulate);
	else
		hipLaunchKernelGGL((gelu_bwd_kernel<1, 0>), CNET_GRID_2D(1), x_re, x_im, ldx, g, ldg, dx, lddx, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_crelu_fwd(const float *x_re, const float *x_im, int64_t ldx, float *y_re, float *y_im, int64_t ldy, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && y_re && y_im && ldx >= cols && ldy >= cols);
	const int nt = stream_policy(ST_STORES, 4, (long) rows * cols);
	if (all_mult4({cols, ldx, ldy}) && all_aligned({x_re, x_im, y_re, y_im}))
		CNET_LAUNCH_V4(crelu_fwd_kernel, nt, CNET_GRID_2D(4), x_re, x_im, ldx, y_re, y_im, ldy, rows, cols);
	else
		hipLaunchKernelGGL((crelu_fwd_kernel<1, 0>), CNET_GRID_2D(1), x_re, x_im, ldx, y_re, y_im, ldy, rows, cols);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_crelu_bwd(const float *x_re, const float *x_im, int64_t ldx, const float *g_dz_re, const float *g_dz_im,
		const float *g_dzs_re, const float *g_dzs_im, int64_t ldg, float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re,
		float *dx_dzs_im, int64_t lddx, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && g_dz_re && g_dz_im && g_dzs_re && g_dzs_im && dx_dz_re && dx_dz_im && dx_dzs_re && dx_dzs_im);
	CNET_CHECK_ARG(ldx >= cols && ldg >= cols && lddx >= cols);
	CGrad4 g = {g_dz_re, g_dz_im, g_dzs_re, g_dzs_im};
	Grad4 dx = {dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im};
	const int nt = stream_policy(ST_BOTH, 10, (long) rows * cols);
	if (all_mult4({cols, ldx, ldg, lddx}) &&
			all_aligned({x_re, x_im, g_dz_re, g_dz_im, g_dzs_re, g_dzs_im, dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im}))
		CNET_LAUNCH_V4(crelu_bwd_kernel, nt, CNET_GRID_2D(4), x_re, x_im, ldx, g, ldg, dx, lddx, rows, cols, accumulate);
	else
		hipLaunchKernelGGL((crelu_bwd_kernel<1, 0>), CNET_GRID_2D(1), x_re, x_im, ldx, g, ldg, dx, lddx, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_residual_fwd(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
		float *y_re, float *y_im, int64_t ldy, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	// a leading dimension of 0 makes that operand one row shared by all rows (a parameter added to every sample)
	CNET_CHECK_ARG(u_re && u_im && v_re && v_im && y_re && y_im && (ldu >= cols || ldu == 0) && (ldv >= cols || ldv == 0) && ldy >= cols);
	const int nt = stream_policy(ST_BOTH, 2 + (ldu ? 2 : 0) + (ldv ? 2 : 0), (long) rows * cols);
	if (all_mult4({cols, ldu, ldv, ldy}) && all_aligned({u_re, u_im, v_re, v_im, y_re, y_im}))
		CNET_LAUNCH_V4(residual_fwd_kernel, nt, CNET_GRID_2D(4), u_re, u_im, ldu, v_re, v_im, ldv, y_re, y_im, ldy, rows, cols);
	else
		hipLaunchKernelGGL((residual_fwd_kernel<1, 0>), CNET_GRID_2D(1), u_re, u_im, ldu, v_re, v_im, ldv, y_re, y_im, ldy, rows, cols);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_residual_bwd(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg,
		float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu, float *dv_dz_re,
		float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && g_dzs_re && g_dzs_im);
	CNET_CHECK_ARG(du_dz_re && du_dz_im && du_dzs_re && du_dzs_im && dv_dz_re && dv_dz_im && dv_dzs_re && dv_dzs_im);
	CNET_CHECK_ARG(ldg >= cols && lddu >= cols && lddv >= cols);
	CGrad4 g = {g_dz_re, g_dz_im, g_dzs_re, g_dzs_im};
	Grad4 du = {du_dz_re, du_dz_im, du_dzs_re, du_dzs_im};
	Grad4 dv = {dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im};
	const int nt = stream_policy(ST_LOADS, 12, (long) rows * cols);
	if (all_mult4({cols, ldg, lddu, lddv}) &&
			all_aligned({g_dz_re, g_dz_im, g_dzs_re, g_dzs_im, du_dz_re, du_dz_im, du_dzs_re, du_dzs_im, dv_dz_re, dv_dz_im,
					dv_dzs_re, dv_dzs_im}))
		CNET_LAUNCH_V4(residual_bwd_kernel, nt, CNET_GRID_2D(4), g, ldg, du, lddu, dv, lddv, rows, cols, accumulate);
	else
		hipLaunchKernelGGL((residual_bwd_kernel<1, 0>), CNET_GRID_2D(1), g, ldg, du, lddu, dv, lddv, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_l2out_bwd(const float *z_re, const float *z_im, int64_t ldz, float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re,
		float *dz_dzs_im, int64_t lddz, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && dz_dz_re && dz_dz_im && dz_dzs_re && dz_dzs_im && ldz >= cols && lddz >= cols);
	Grad4 dz = {dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im};
	const int nt = stream_policy(ST_STORES, 6, (long) rows * cols);
	if (all_mult4({cols, ldz, lddz}) && all_aligned({z_re, z_im, dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im}))
		CNET_LAUNCH_V4(l2out_bwd_kernel, nt, CNET_GRID_2D(4), z_re, z_im, ldz, dz, lddz, rows, cols, accumulate);
	else
		hipLaunchKernelGGL((l2out_bwd_kernel<1, 0>), CNET_GRID_2D(1), z_re, z_im, ldz, dz, lddz, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_cross_entropy_bwd(const float *z_re, const float *z_im, int64_t ldz, const float *s, const int32_t *labels,
		float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && s && labels && dz_dz_re && dz_dz_im && dz_dzs_re && dz_dzs_im && ldz >= cols && lddz >= cols);
	Grad4 dz = {dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im};
	const int nt = stream_policy(ST_BOTH, 6, (long) rows * cols);
	if (all_mult4({cols, ldz, lddz}) && all_aligned({z_re, z_im, dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im}))
		CNET_LAUNCH_V4(crossent_bwd_kernel, nt, CNET_GRID_2D(4), z_re, z_im, ldz, s, labels, dz, lddz, rows, cols);
	else
		hipLaunchKernelGGL((crossent_bwd_kernel<1, 0>), CNET_GRID_2D(1), z_re, z_im, ldz, s, labels, dz, lddz, rows, cols);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

static int copy_or_add(const float *src, int64_t lds, float *dst, int64_t ldd, int rows, int cols, int add) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(src && dst && lds >= cols && ldd >= cols);
	const int nt = stream_policy(ST_LOADS, 2, (long) rows * cols);
	if (all_mult4({cols, lds, ldd}) && all_aligned({src, dst}))
		CNET_LAUNCH_V4(copy2d_kernel, nt, CNET_GRID_2D(4), src, lds, dst, ldd, rows, cols, add);
	else
		hipLaunchKernelGGL((copy2d_kernel<1, 0>), CNET_GRID_2D(1), src, lds, dst, ldd, rows, cols, add);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_copy2d(const float *src, int64_t lds, float *dst, int64_t ldd, int rows, int cols) {
	return copy_or_add(src, lds, dst, ldd, rows, cols, 0);
}

int cnet_add2d(const float *src, int64_t lds, float *dst, int64_t ldd, int rows, int cols) {
	return copy_or_add(src, lds, dst, ldd, rows, cols, 1);
}

int cnet_add_multi(int count, const float *const *src, float *const *dst, const int64_t *n) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(count >= 0);
	if (!count) return CNET_OK;
	CNET_CHECK_ARG(src && dst && n);
	for (int k = 0; k < count; ++k) CNET_CHECK_ARG(n[k] >= 0 && (n[k] == 0 || (src[k] && dst[k])));
	for (int first = 0; first < count; first += SGD_MULTI_MAX) {
		AddMulti t;
		int used = 0;
		long longest = 0;
		for (int k = first; k < count && k < first + SGD_MULTI_MAX; ++k) {
			if (!n[k]) continue;
			t.src[used] = src[k];
			t.dst[used] = dst[k];
			t.n[used] = (long) n[k];
			t.vec[used] = n[k] % 4 == 0 && all_aligned({src[k], dst[k]});
			longest = std::max(longest, (long) n[k]);
			++used;
		}
		if (!used) continue;
		hipLaunchKernelGGL(add_multi_kernel, dim3(nblocks((longest + 3) / 4), used), dim3(TPB), 0, rt().stream, t);
		CNET_LAUNCH_CHECK();
	}
	return CNET_OK;
}

int cnet_sgd_update(float *z_re, float *z_im, float *dzs_re, float *dzs_im, int64_t n, float lr, int zero_grad) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(n >= 0);
	if (!n) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && dzs_re && dzs_im);
	const int nt = stream_policy(ST_LOADS, 4, (long) n);
	if (n % 4 == 0 && all_aligned({z_re, z_im, dzs_re, dzs_im}))
		CNET_LAUNCH_V4(sgd_kernel, nt, dim3(nblocks(n / 4)), dim3(TPB), 0, rt().stream, z_re, z_im, dzs_re, dzs_im, (long) n, lr, zero_grad);
	else
		hipLaunchKernelGGL((sgd_kernel<1, 0>), dim3(nblocks(n)), dim3(TPB), 0, rt().stream, z_re, z_im, dzs_re, dzs_im, (long) n, lr, zero_grad);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_sgd_update_multi(int count, float *const *z_re, float *const *z_im, float *const *dzs_re, float *const *dzs_im,
		const int64_t *n, float lr, int zero_grad) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(count >= 0);
	if (!count) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && dzs_re && dzs_im && n);
	for (int k = 0; k < count; ++k) CNET_CHECK_ARG(n[k] >= 0 && (n[k] == 0 || (z_re[k] && z_im[k] && dzs_re[k] && dzs_im[k])));
	for (int first = 0; first < count; first += SGD_MULTI_MAX) {
		SgdMulti t;
		int used = 0;
		long longest = 0;
		for (int k = first; k < count && k < first + SGD_MULTI_MAX; ++k) {
			if (!n[k]) continue;
			t.z_re[used] = z_re[k];
			t.z_im[used] = z_im[k];
			t.d_re[used] = dzs_re[k];
			t.d_im[used] = dzs_im[k];
			t.n[used] = (long) n[k];
			t.vec[used] = n[k] % 4 == 0 && all_aligned({z_re[k], z_im[k], dzs_re[k], dzs_im[k]});
			longest = std::max(longest, (long) n[k]);
			++used;
		}
		if (!used) continue;
		hipLaunchKernelGGL(sgd_multi_kernel, dim3(nblocks((longest + 3) / 4), used), dim3(TPB), 0, rt().stream, t, lr, zero_grad);
		CNET_LAUNCH_CHECK();
	}
	return CNET_OK;
}

int cnet_adam_update(float *z_re, float *z_im, float *m_re, float *m_im, float *dzs_re, float *dzs_im, int64_t n, float lr,
		float beta, int t, int zero_grad) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(n >= 0 && t >= 0);
	if (!n) return CNET_OK;
	CNET_CHECK_ARG(z_re && z_im && m_re && m_im && dzs_re && dzs_im);
	const double denom = 1 - std::pow((double) beta, (double) (t + 1));
	CNET_CHECK_ARG(denom != 0.0);
	const int nt = stream_policy(ST_BOTH, 6, (long) n);
	if (n % 4 == 0 && all_aligned({z_re, z_im, m_re, m_im, dzs_re, dzs_im}))
		CNET_LAUNCH_V4(adam_kernel, nt, dim3(nblocks(n / 4)), dim3(TPB), 0, rt().stream, z_re, z_im, m_re, m_im, dzs_re, dzs_im,
				(long) n, lr, beta, denom, zero_grad);
	else
		hipLaunchKernelGGL((adam_kernel<1, 0>), dim3(nblocks(n)), dim3(TPB), 0, rt().stream, z_re, z_im, m_re, m_im, dzs_re, dzs_im,
				(long) n, lr, beta, denom, zero_grad);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

// ---- backward passes for a conjugate gradient pair (g.dzs == conj(g.dz)); the dz* planes of the results are optional
static inline Pair2 pair_of(float *dz_re, float *dz_im, float *dzs_re, float *dzs_im) { return Pair2{dz_re, dz_im, dzs_re, dzs_im}; }
#define CNET_CHECK_PAIR(p) CNET_CHECK_ARG((p).dz_re && (p).dz_im && (((p).dzs_re == nullptr) == ((p).dzs_im == nullptr)))
static inline int pair_planes(const Pair2 &p) { return p.dzs_re ? 4 : 2; }

int cnet_cgelu_bwd_sym(const float *x_re, const float *x_im, int64_t ldx, const float *g_dz_re, const float *g_dz_im, int64_t ldg,
		float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	const Pair2 dx = pair_of(dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im);
	CNET_CHECK_ARG(x_re && x_im && g_dz_re && g_dz_im);
	CNET_CHECK_PAIR(dx);
	CNET_CHECK_ARG(ldx >= cols && ldg >= cols && lddx >= cols);
	const int nt = stream_policy(ST_LOADS, 4 + pair_planes(dx), (long) rows * cols);
	if (all_mult4({cols, ldx, ldg, lddx}) && all_aligned({x_re, x_im, g_dz_re, g_dz_im, dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im}))
		CNET_LAUNCH_V4(gelu_bwd_sym_kernel, nt, CNET_GRID_2D(4), x_re, x_im, ldx, g_dz_re, g_dz_im, ldg, dx, lddx, rows, cols, accumulate);
	else
		hipLaunchKernelGGL((gelu_bwd_sym_kernel<1, 0>), CNET_GRID_2D(1), x_re, x_im, ldx, g_dz_re, g_dz_im, ldg, dx, lddx, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_crelu_bwd_sym(const float *x_re, const float *x_im, int64_t ldx, const float *g_dz_re, const float *g_dz_im, int64_t ldg,
		float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	const Pair2 dx = pair_of(dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im);
	CNET_CHECK_ARG(x_re && x_im && g_dz_re && g_dz_im);
	CNET_CHECK_PAIR(dx);
	CNET_CHECK_ARG(ldx >= cols && ldg >= cols && lddx >= cols);
	const int nt = stream_policy(ST_LOADS, 4 + pair_planes(dx), (long) rows * cols);
	if (all_mult4({cols, ldx, ldg, lddx}) && all_aligned({x_re, x_im, g_dz_re, g_dz_im, dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im}))
		CNET_LAUNCH_V4(crelu_bwd_sym_kernel, nt, CNET_GRID_2D(4), x_re, x_im, ldx, g_dz_re, g_dz_im, ldg, dx, lddx, rows, cols, accumulate);
	else
		hipLaunchKernelGGL((crelu_bwd_sym_kernel<1, 0>), CNET_GRID_2D(1), x_re, x_im, ldx, g_dz_re, g_dz_im, ldg, dx, lddx, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_residual_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, float *du_dz_re, float *du_dz_im, float *du_dzs_re,
		float *du_dzs_im, int64_t lddu, float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv, int rows,
		int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	const Pair2 du = pair_of(du_dz_re, du_dz_im, du_dzs_re, du_dzs_im), dv = pair_of(dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im);
	CNET_CHECK_ARG(g_dz_re && g_dz_im);
	CNET_CHECK_PAIR(du);
	CNET_CHECK_PAIR(dv);
	CNET_CHECK_ARG(ldg >= cols && lddu >= cols && lddv >= cols);
	const int nt = stream_policy(ST_STORES, 2 + pair_planes(du) + pair_planes(dv), (long) rows * cols);
	if (all_mult4({cols, ldg, lddu, lddv}) &&
			all_aligned({g_dz_re, g_dz_im, du_dz_re, du_dz_im, du_dzs_re, du_dzs_im, dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im}))
		CNET_LAUNCH_V4(residual_bwd_sym_kernel, nt, CNET_GRID_2D(4), g_dz_re, g_dz_im, ldg, du, lddu, dv, lddv, rows, cols, accumulate);
	else
		hipLaunchKernelGGL((residual_bwd_sym_kernel<1, 0>), CNET_GRID_2D(1), g_dz_re, g_dz_im, ldg, du, lddu, dv, lddv, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_residual_bwd_sym2(const float *g1_dz_re, const float *g1_dz_im, int64_t ldg1, const float *g2_dz_re, const float *g2_dz_im,
		int64_t ldg2, float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu, float *dv_dz_re, float *dv_dz_im,
		float *dv_dzs_re, float *dv_dzs_im, int64_t lddv, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	const Pair2 du = pair_of(du_dz_re, du_dz_im, du_dzs_re, du_dzs_im), dv = pair_of(dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im);
	CNET_CHECK_ARG(g1_dz_re && g1_dz_im && g2_dz_re && g2_dz_im);
	CNET_CHECK_PAIR(du);
	CNET_CHECK_PAIR(dv);
	CNET_CHECK_ARG(ldg1 >= cols && ldg2 >= cols && lddu >= cols && lddv >= cols);
	const int nt = stream_policy(ST_LOADS, 4 + pair_planes(du) + pair_planes(dv), (long) rows * cols);
	if (all_mult4({cols, ldg1, ldg2, lddu, lddv}) && all_aligned({g1_dz_re, g1_dz_im, g2_dz_re, g2_dz_im, du_dz_re, du_dz_im, du_dzs_re,
			du_dzs_im, dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im}))
		CNET_LAUNCH_V4(residual_bwd_sym2_kernel, nt, CNET_GRID_2D(4), g1_dz_re, g1_dz_im, ldg1, g2_dz_re, g2_dz_im, ldg2, du, lddu, dv, lddv,
				rows, cols, accumulate);
	else
		hipLaunchKernelGGL((residual_bwd_sym2_kernel<1, 0>), CNET_GRID_2D(1), g1_dz_re, g1_dz_im, ldg1, g2_dz_re, g2_dz_im, ldg2, du, lddu,
				dv, lddv, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

// the launch macro for kernels with a third template flag
#define CNET_LAUNCH_V4G_P(kernel, P, gelu, ...)                              \
	do {                                                                     \
		if (gelu) hipLaunchKernelGGL((kernel<4, P, true>), __VA_ARGS__);      \
		else hipLaunchKernelGGL((kernel<4, P, false>), __VA_ARGS__);         \
	} while (0)
#define CNET_LAUNCH_V4G(kernel, pol, gelu, ...)                              \
	do {                                                                     \
		switch (pol) {                                                       \
		case 1: CNET_LAUNCH_V4G_P(kernel, 1, gelu, __VA_ARGS__); break;      \
		case 2: CNET_LAUNCH_V4G_P(kernel, 2, gelu, __VA_ARGS__); break;      \
		case 3: CNET_LAUNCH_V4G_P(kernel, 3, gelu, __VA_ARGS__); break;      \
		default: CNET_LAUNCH_V4G_P(kernel, 0, gelu, __VA_ARGS__); break;     \
		}                                                                    \
	} while (0)
#define CNET_LAUNCH_V1G(kernel, gelu, ...)                                   \
	do {                                                                     \
		if (gelu) hipLaunchKernelGGL((kernel<1, 0, true>), __VA_ARGS__);  \
		else hipLaunchKernelGGL((kernel<1, 0, false>), __VA_ARGS__);     \
	} while (0)

int cnet_residual_cgelu_bwd_sym(const float *g1_dz_re, const float *g1_dz_im, int64_t ldg1, const float *g2_dz_re, const float *g2_dz_im,
		int64_t ldg2, const float *h_re, const float *h_im, int64_t ldh, float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im,
		int64_t lddu, float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv, float *dh_dz_re, float *dh_dz_im,
		float *dh_dzs_re, float *dh_dzs_im, int64_t lddh, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	const Pair2 du = pair_of(du_dz_re, du_dz_im, du_dzs_re, du_dzs_im), dv = pair_of(dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im),
			dh = pair_of(dh_dz_re, dh_dz_im, dh_dzs_re, dh_dzs_im);
	const bool two = g2_dz_re != nullptr, with_dv = dv_dz_re != nullptr;
	CNET_CHECK_ARG(g1_dz_re && g1_dz_im && h_re && h_im && (g2_dz_re == nullptr) == (g2_dz_im == nullptr));
	CNET_CHECK_PAIR(du);
	CNET_CHECK_PAIR(dh);
	if (with_dv) CNET_CHECK_PAIR(dv);
	else CNET_CHECK_ARG(!dv_dz_im && !dv_dzs_re && !dv_dzs_im);
	CNET_CHECK_ARG(ldg1 >= cols && (!two || ldg2 >= cols) && ldh >= cols && lddu >= cols && (!with_dv || lddv >= cols) && lddh >= cols);
	const int nt = stream_policy(ST_BOTH, 4 + (two ? 2 : 0) + pair_planes(du) + (with_dv ? pair_planes(dv) : 0) + pair_planes(dh), (long) rows * cols);
	if (all_mult4({cols, ldg1, two ? ldg2 : 0, ldh, lddu, with_dv ? lddv : 0, lddh}) &&
			all_aligned({g1_dz_re, g1_dz_im, g2_dz_re, g2_dz_im, h_re, h_im, du_dz_re, du_dz_im, du_dzs_re, du_dzs_im, dv_dz_re, dv_dz_im,
					dv_dzs_re, dv_dzs_im, dh_dz_re, dh_dz_im, dh_dzs_re, dh_dzs_im}))
		CNET_LAUNCH_V4G(residual_gelu_bwd_sym_kernel, nt, two, CNET_GRID_2D(4), g1_dz_re, g1_dz_im, ldg1, g2_dz_re, g2_dz_im, ldg2, h_re, h_im,
				ldh, du, lddu, dv, lddv, dh, lddh, rows, cols);
	else
		CNET_LAUNCH_V1G(residual_gelu_bwd_sym_kernel, two, CNET_GRID_2D(1), g1_dz_re, g1_dz_im, ldg1, g2_dz_re, g2_dz_im, ldg2, h_re, h_im, ldh,
				du, lddu, dv, lddv, dh, lddh, rows, cols);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

// whether the backward pass of a Hadamard for a conjugate pair runs on 128-bit accesses
static bool hadamard_sym_vec(bool gelu, const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
		const float *g_dz_re, const float *g_dz_im, int64_t ldg, const Pair2 &dh, int64_t lddh, const Pair2 &du, int64_t lddu, const Pair2 &dv,
		int64_t lddv, int cols) {
	return all_mult4({cols, ldu, ldv, ldg, lddu, ldv ? lddv : 0, gelu && dh.dz_re ? lddh : 0}) &&
			all_aligned({u_re, u_im, v_re, v_im, g_dz_re, g_dz_im, du.dz_re, du.dz_im, du.dzs_re, du.dzs_im, dv.dz_re, dv.dz_im, dv.dzs_re,
					dv.dzs_im, gelu ? dh.dz_re : nullptr, gelu ? dh.dz_im : nullptr, gelu ? dh.dzs_re : nullptr, gelu ? dh.dzs_im : nullptr});
}

// gelu: the incoming gradient belongs to a CGelu applied to the Hadamard's result; dh receives the gradient of that CGelu's
// operand
static int hadamard_bwd_sym_impl(const char *who, bool gelu, const float *u_re, const float *u_im, int64_t ldu, const float *v_re,
		const float *v_im, int64_t ldv, const float *g_dz_re, const float *g_dz_im, int64_t ldg, Pair2 dh, int64_t lddh, Pair2 du,
		int64_t lddu, Pair2 dv, int64_t lddv, int rows, int cols, int accumulate) {
	if (!rt().ready) return fail(CNET_ERR_NOT_INITIALIZED, "%s: cnet_init() has not been called", who);
	if (rows < 0 || cols < 0) return fail(CNET_ERR_INVALID_ARGUMENT, "%s: negative shape", who);
	if (!rows || !cols) return CNET_OK;
	auto pair_ok = [](const Pair2 &p) { return p.dz_re && p.dz_im && ((p.dzs_re == nullptr) == (p.dzs_im == nullptr)); };
	if (!(u_re && u_im && v_re && v_im && g_dz_re && g_dz_im && pair_ok(du) && pair_ok(dv) &&
			(!gelu || pair_ok(dh) || !(dh.dz_re || dh.dz_im || dh.dzs_re || dh.dzs_im))))
		return fail(CNET_ERR_INVALID_ARGUMENT, "%s: a required plane is NULL (the dz* planes of a result are optional, in pairs)", who);
	if (!(ldu >= cols && ldg >= cols && lddu >= cols && (ldv == 0 || (ldv >= cols && lddv >= cols)) && (!gelu || !dh.dz_re || lddh >= cols)))
		return fail(CNET_ERR_INVALID_ARGUMENT, "%s: a leading dimension is shorter than the row", who);
	const bool vec = hadamard_sym_vec(gelu, u_re, u_im, ldu, v_re, v_im, ldv, g_dz_re, g_dz_im, ldg, dh, lddh, du, lddu, dv, lddv, cols);
	const int nt = stream_policy(ST_LOADS, 4 + pair_planes(du) + (ldv ? 2 + pair_planes(dv) : 0) + (gelu && dh.dz_re ? pair_planes(dh) : 0), (long) rows * cols);
	if (ldv != 0) {
		if (vec)
			CNET_LAUNCH_V4G(hadamard_bwd_sym_kernel, nt, gelu, CNET_GRID_2D(4), u_re, u_im, ldu, v_re, v_im, ldv, g_dz_re, g_dz_im, ldg, dh, lddh,
					du, lddu, dv, lddv, rows, cols, accumulate);
		else
			CNET_LAUNCH_V1G(hadamard_bwd_sym_kernel, gelu, CNET_GRID_2D(1), u_re, u_im, ldu, v_re, v_im, ldv, g_dz_re, g_dz_im, ldg, dh, lddh, du,
					lddu, dv, lddv, rows, cols, accumulate);
		CNET_LAUNCH_CHECK();
		return CNET_OK;
	}
	const int V = vec ? 4 : 1;
	const long col_blocks = ((long) cols / V + CS_X - 1) / CS_X;
	int nslabs, rows_per_slab;
	cnet::gate_slabs(rows, cols, V, rt().prop.multiProcessorCount, &nslabs, &rows_per_slab);
	float *partial = (float *) workspace((size_t) nslabs * 2 * cols * sizeof(float));
	if (!partial) return CNET_ERR_OUT_OF_MEMORY;
	dim3 grid((unsigned) col_blocks, (unsigned) nslabs);
	if (vec)
		CNET_LAUNCH_V4G(hadamard_bwd_shared_sym_kernel, nt, gelu, grid, dim3(TPB), 0, rt().stream, u_re, u_im, ldu, v_re, v_im, g_dz_re, g_dz_im,
				ldg, dh, lddh, du, lddu, partial, rows, cols, rows_per_slab, accumulate);
	else
		CNET_LAUNCH_V1G(hadamard_bwd_shared_sym_kernel, gelu, grid, dim3(TPB), 0, rt().stream, u_re, u_im, ldu, v_re, v_im, g_dz_re, g_dz_im, ldg,
				dh, lddh, du, lddu, partial, rows, cols, rows_per_slab, accumulate);
	CNET_LAUNCH_CHECK();
	if (nslabs > 32)
		hipLaunchKernelGGL((slab_sum_sym_kernel<64, 16>), dim3((unsigned) ((2L * cols + 15) / 16)), dim3(1024), 0, rt().stream, partial, nslabs, cols, dv, accumulate);
	else
		hipLaunchKernelGGL((slab_sum_sym_kernel<4, 64>), dim3((unsigned) ((2L * cols + 63) / 64)), dim3(256), 0, rt().stream, partial, nslabs, cols, dv, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_hadamard_bwd_sym(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
		const float *g_dz_re, const float *g_dz_im, int64_t ldg, float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im,
		int64_t lddu, float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int64_t lddv, int rows, int cols,
		int accumulate) {
	return hadamard_bwd_sym_impl(__func__, false, u_re, u_im, ldu, v_re, v_im, ldv, g_dz_re, g_dz_im, ldg, Pair2{nullptr, nullptr, nullptr, nullptr}, 0,
			pair_of(du_dz_re, du_dz_im, du_dzs_re, du_dzs_im), lddu, pair_of(dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im), lddv, rows, cols,
			accumulate);
}

int cnet_hadamard_cgelu_bwd_sym(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
		const float *g_dz_re, const float *g_dz_im, int64_t ldg, float *dh_dz_re, float *dh_dz_im, float *dh_dzs_re, float *dh_dzs_im,
		int64_t lddh, float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu, float *dv_dz_re, float *dv_dz_im,
		float *dv_dzs_re, float *dv_dzs_im, int64_t lddv, int rows, int cols, int accumulate) {
	return hadamard_bwd_sym_impl(__func__, true, u_re, u_im, ldu, v_re, v_im, ldv, g_dz_re, g_dz_im, ldg,
			pair_of(dh_dz_re, dh_dz_im, dh_dzs_re, dh_dzs_im), lddh, pair_of(du_dz_re, du_dz_im, du_dzs_re, du_dzs_im), lddu,
			pair_of(dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im), lddv, rows, cols, accumulate);
}

int cnet_clinear_hadamard_cgelu_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, const float *x_re, const float *x_im,
		int64_t ldx, const float *w_re, const float *w_im, int64_t ldw, float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im,
		int64_t lddx, int accumulate_dx, float *dw_dz_re, float *dw_dz_im, float *dw_dzs_re, float *dw_dzs_im, int64_t lddw, int accumulate_dw,
		const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, float *dh_dz_re, float *dh_dz_im,
		float *dh_dzs_re, float *dh_dzs_im, int64_t lddh, float *du_dz_re, float *du_dz_im, float *du_dzs_re, float *du_dzs_im, int64_t lddu,
		float *dv_dz_re, float *dv_dz_im, float *dv_dzs_re, float *dv_dzs_im, int accumulate_gate, int B, int K, int N) {
	CNET_REQUIRE_INIT();
	const Pair2 dx = pair_of(dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im), dw = pair_of(dw_dz_re, dw_dz_im, dw_dzs_re, dw_dzs_im);
	const Pair2 dh = pair_of(dh_dz_re, dh_dz_im, dh_dzs_re, dh_dzs_im), du = pair_of(du_dz_re, du_dz_im, du_dzs_re, du_dzs_im);
	const Pair2 dv = pair_of(dv_dz_re, dv_dz_im, dv_dzs_re, dv_dzs_im);
	auto pair_ok = [](const Pair2 &p) { return p.dz_re && p.dz_im && ((p.dzs_re == nullptr) == (p.dzs_im == nullptr)); };
	// One launch when every argument is in order and both products are small (the workgroup that owns 16 columns of dx goes
	// on to the gate's backward pass of those columns); whatever is not goes to the two calls, which name what is wrong.
	const bool plain = B > 0 && K > 0 && N > 0 && g_dz_re && g_dz_im && x_re && x_im && w_re && w_im && u_re && u_im && v_re && v_im &&
			pair_ok(dx) && pair_ok(dw) && pair_ok(du) && pair_ok(dv) && (pair_ok(dh) || !(dh.dz_re || dh.dz_im || dh.dzs_re || dh.dzs_im)) &&
			ldg >= N && ldx >= K && ldw >= K && lddx >= K && lddw >= K && ldu >= K && lddu >= K && (!dh.dz_re || lddh >= K);
	if (plain) {
		cnet::GateBwd gate{u_re, u_im, ldu, v_re, v_im, dh, lddh, du, lddu, dv, accumulate_gate, 0, 0};
		const bool vec = hadamard_sym_vec(true, u_re, u_im, ldu, v_re, v_im, 0, dx_dz_re, dx_dz_im, lddx, dh, lddh, du, lddu, dv, K, K);
		cnet::gate_slabs(B, K, vec ? 4 : 1, rt().prop.multiProcessorCount, &gate.nslabs, &gate.rows_per_slab);
		int rc = CNET_OK;
		if (cnet::cgemm_linear_bwd_gate(g_dz_re, g_dz_im, ldg, x_re, x_im, ldx, w_re, w_im, ldw, dx, lddx, accumulate_dx, dw, lddw,
					accumulate_dw, B, K, N, gate, &rc))
			return rc;
	}
	const int rc = cnet_clinear_bwd_sym(g_dz_re, g_dz_im, ldg, x_re, x_im, ldx, w_re, w_im, ldw, dx_dz_re, dx_dz_im, dx_dzs_re, dx_dzs_im, lddx,
			accumulate_dx, dw_dz_re, dw_dz_im, dw_dzs_re, dw_dzs_im, lddw, accumulate_dw, B, K, N);
	if (rc != CNET_OK) return rc;
	return hadamard_bwd_sym_impl(__func__, true, u_re, u_im, ldu, v_re, v_im, 0, dx_dz_re, dx_dz_im, lddx, dh, lddh, du, lddu, dv, K, B, K,
			accumulate_gate);
}

int cnet_hadamard_cgelu_fwd(const float *u_re, const float *u_im, int64_t ldu, const float *v_re, const float *v_im, int64_t ldv,
		float *h_re, float *h_im, int64_t ldh, float *y_re, float *y_im, int64_t ldy, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	CNET_CHECK_ARG(u_re && u_im && v_re && v_im && h_re && h_im && y_re && y_im);
	CNET_CHECK_ARG(ldu >= cols && ldh >= cols && ldy >= cols && (ldv == 0 || ldv >= cols));
	const int nt = stream_policy(ST_STORES, 6 + (ldv ? 2 : 0), (long) rows * cols);
	if (all_mult4({cols, ldu, ldv, ldh, ldy}) && all_aligned({u_re, u_im, v_re, v_im, h_re, h_im, y_re, y_im}))
		CNET_LAUNCH_V4(hadamard_gelu_fwd_kernel, nt, CNET_GRID_2D(4), u_re, u_im, ldu, v_re, v_im, ldv, h_re, h_im, ldh, y_re, y_im, ldy, rows,
				cols);
	else
		hipLaunchKernelGGL((hadamard_gelu_fwd_kernel<1, 0>), CNET_GRID_2D(1), u_re, u_im, ldu, v_re, v_im, ldv, h_re, h_im, ldh, y_re, y_im,
				ldy, rows, cols);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_l2out_bwd_sym(const float *z_re, const float *z_im, int64_t ldz, float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re,
		float *dz_dzs_im, int64_t lddz, int rows, int cols, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	const Pair2 dz = pair_of(dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im);
	CNET_CHECK_ARG(z_re && z_im && ldz >= cols && lddz >= cols);
	CNET_CHECK_PAIR(dz);
	const int nt = stream_policy(ST_LOADS, 2 + pair_planes(dz), (long) rows * cols);
	if (all_mult4({cols, ldz, lddz}) && all_aligned({z_re, z_im, dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im}))
		CNET_LAUNCH_V4(l2out_bwd_sym_kernel, nt, CNET_GRID_2D(4), z_re, z_im, ldz, dz, lddz, rows, cols, accumulate);
	else
		hipLaunchKernelGGL((l2out_bwd_sym_kernel<1, 0>), CNET_GRID_2D(1), z_re, z_im, ldz, dz, lddz, rows, cols, accumulate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_cross_entropy_bwd_sym(const float *z_re, const float *z_im, int64_t ldz, const float *s, const int32_t *labels, float *dz_dz_re,
		float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && cols >= 0);
	if (!rows || !cols) return CNET_OK;
	const Pair2 dz = pair_of(dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im);
	CNET_CHECK_ARG(z_re && z_im && s && labels && ldz >= cols && lddz >= cols);
	CNET_CHECK_PAIR(dz);
	const int nt = stream_policy(ST_BOTH, 2 + pair_planes(dz), (long) rows * cols);
	if (all_mult4({cols, ldz, lddz}) && all_aligned({z_re, z_im, dz_dz_re, dz_dz_im, dz_dzs_re, dz_dzs_im}))
		CNET_LAUNCH_V4(crossent_bwd_sym_kernel, nt, CNET_GRID_2D(4), z_re, z_im, ldz, s, labels, dz, lddz, rows, cols);
	else
		hipLaunchKernelGGL((crossent_bwd_sym_kernel<1, 0>), CNET_GRID_2D(1), z_re, z_im, ldz, s, labels, dz, lddz, rows, cols);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

}  // extern "C"
