// Row primitives shared by the row kernels (reduce.hip) and by the matrix kernel that finishes a row of logits in its own
// store (cgemm.hip): the fixed-order lane and wavefront reductions, the cache-policy loads and stores, and the forward pass
// of CrossEntropy over one row.
#ifndef CNET_CSRC_ROWS_HPP_
#define CNET_CSRC_ROWS_HPP_

#include "common.hpp"

namespace cnet {
namespace rows {

// ---------------------------------------------------------------------------------------------- lane exchange
// value of the lane selected by a DPP control word, for 32-bit payloads
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
	return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
constexpr int DPP_QUAD_XOR1 = 0xB1;  // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_ROR4 = 0x124;
constexpr int DPP_ROW_ROR8 = 0x128;
constexpr int SWIZZLE_XOR16 = 0x401F;  // bit mode: and 0x1f, or 0, xor 0x10

template <class T, int STEP>
__device__ __forceinline__ T exchange(T v) {
	static_assert(sizeof(T) % 4 == 0, "32-bit words");
	constexpr int W = sizeof(T) / 4;
	union {
		T t;
		int w[W];
	} a, b;
	a.t = v;
#pragma unroll
	for (int k = 0; k < W; ++k) {
		if (STEP == 0) b.w[k] = dpp_i<DPP_QUAD_XOR1>(a.w[k]);
		if (STEP == 1) b.w[k] = dpp_i<DPP_QUAD_XOR2>(a.w[k]);
		if (STEP == 2) b.w[k] = dpp_i<DPP_ROW_ROR4>(a.w[k]);
		if (STEP == 3) b.w[k] = dpp_i<DPP_ROW_ROR8>(a.w[k]);
		if (STEP == 4) b.w[k] = __builtin_amdgcn_ds_swizzle(a.w[k], SWIZZLE_XOR16);
		if (STEP == 5) b.w[k] = __shfl_xor(a.w[k], 32, 64);
	}
	return b.t;
}

// After the six steps lane 0 (in fact every lane) holds op over all 64 lanes, combined in a fixed order.
template <class T, class Op>
__device__ __forceinline__ T wave_reduce(T v, Op op) {
	v = op(v, exchange<T, 0>(v));
	v = op(v, exchange<T, 1>(v));
	v = op(v, exchange<T, 2>(v));
	v = op(v, exchange<T, 3>(v));
	v = op(v, exchange<T, 4>(v));
	v = op(v, exchange<T, 5>(v));
	return v;
}

// G wavefronts of a workgroup share one row: combine their results in wavefront order through LDS.
// `slot` is this row's position within the workgroup.  Returns the total to every thread of the group.
template <class T, int G, class Op>
__device__ __forceinline__ T group_reduce(T v, Op op, T *lds, int slot, int wave_in_group, int lane) {
	v = wave_reduce(v, op);
	if (G == 1) return v;
	if (lane == 0) lds[slot * G + wave_in_group] = v;
	__syncthreads();
	T total = lds[slot * G];
#pragma unroll
	for (int k = 1; k < G; ++k) total = op(total, lds[slot * G + k]);
	__syncthreads();
	return total;
}

struct SumF {
	__device__ float operator()(float a, float b) const { return a + b; }
};
struct SumD {
	__device__ double operator()(double a, double b) const { return a + b; }
};
struct ArgMax {
	float v;
	int i;
};
// larger value wins; equal values keep the smaller index (the first maximum of a serial strict-> scan)
struct ArgMaxOp {
	__device__ ArgMax operator()(ArgMax a, ArgMax b) const {
		if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
		return a;
	}
};
// the largest |z|^2 of a row with its first index, and the runner-up value (to detect near ties); single precision is
// enough for both: they only decide whether the exact second pass is needed (a margin of 1e-5 against 1e-7 of rounding)
struct Top2 {
	float q1, q2;
	int i1, pad;
};
struct Top2Op {
	__device__ Top2 operator()(Top2 a, Top2 b) const {
		Top2 r;
		const bool b_wins = b.q1 > a.q1 || (b.q1 == a.q1 && b.i1 < a.i1);
		const Top2 &w = b_wins ? b : a, &l = b_wins ? a : b;
		r.q1 = w.q1;
		r.i1 = w.i1;
		r.q2 = fmaxf(w.q2, l.q1);
		r.pad = 0;
		return r;
	}
};
struct Cplx4 {
	float a, b, c, d;
};
struct SumC4 {
	__device__ Cplx4 operator()(Cplx4 x, Cplx4 y) const { return Cplx4{x.a + y.a, x.b + y.b, x.c + y.c, x.d + y.d}; }
};

// 128-bit accesses under a cache policy chosen at launch (cnet::stream_policy; uniform over the launch)
__device__ __forceinline__ float4 ld4(const float *p, int policy) {
	typedef float f32x4 __attribute__((ext_vector_type(4)));
	if (policy == cnet::ST_BOTH || policy == cnet::ST_LOADS) {
		const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
		return make_float4(t.x, t.y, t.z, t.w);
	}
	return *reinterpret_cast<const float4 *>(p);
}
__device__ __forceinline__ void st4(float *p, float4 v, int policy) {
	typedef float f32x4 __attribute__((ext_vector_type(4)));
	const f32x4 t = {v.x, v.y, v.z, v.w};
	// (written out: see stv in elementwise.hip)
	if (policy == cnet::ST_BOTH || policy == cnet::ST_STORES)
		asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" ::"v"(p), "v"(t) : "memory");
	else if (policy == cnet::ST_LOADS)
		asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(t) : "memory");
	else
		*reinterpret_cast<float4 *>(p) = v;
}

// ---------------------------------------------------------------------------------------------- CrossEntropy forward
// loss of one row: -log(max(|z_label / sqrt S|^2, 1e-15)) (impl/crossent.h:62-72 upstream).  A label outside the row, which
// upstream would read out of bounds, gives NaN here instead of a wild access.
__device__ __forceinline__ float label_loss(const float *__restrict__ pr, const float *__restrict__ pi, int label, int cols, double inv) {
	if ((unsigned) label >= (unsigned) cols) return __builtin_nanf("");
	const float o_r = (float) (pr[label] * inv), o_i = (float) (pi[label] * inv);
	float p = (float) ((double) o_r * o_r + (double) o_i * o_i);
	p = (p < 1e-15f ? 1e-15f : p);
	return -logf(p);
}

// impl/crossent.h:50-80, 117-130 upstream: S in double, clamped; out = z / sqrt(S); p_k = out_r^2 + out_i^2 evaluated
// in double and rounded to float; argmax = first strict maximum of p; loss = -log(max(p_label, 1e-15)).
// The four planes that receive the gradient of the row's loss in the same launch (all null: the forward pass alone).  The
// values are the ones of crossent_bwd_sym_kernel, formed by the same operations from the same S: dz* = z / S, at the label
// -z (S - m) / (m S) with m = max(|z_label|^2, 1e-15); dz = conj(dz*) (impl/crossent.h:82-104 upstream).
struct GradPlanes {
	float *dz_re, *dz_im, *dzs_re, *dzs_im;
	long ld;
};

__device__ __forceinline__ void crossent_grad(float a, float b, bool at_label, float S, float &g_re, float &g_im) {
	if (at_label) {
		float m = (float) ((double) a * (double) a + (double) b * (double) b);
		m = (m < 1e-15f ? 1e-15f : m);
		g_re = -a * (S - m) / (m * S);
		g_im = -b * (S - m) / (m * S);
	} else {
		g_re = a / S;
		g_im = b / S;
	}
}

// One row, owned by G wavefronts of a workgroup (thread t of the 64 G, lane `lane` of wavefront `wig`; `slot` is the row's
// place among the rows of the workgroup; lds_*: one entry per wavefront of the workgroup, not touched when G == 1).  pr, pi
// point at the row's logits, which may lie in LDS: the small-C matrix kernel runs this on a tile of logits it has just formed.
template <int V, int G, bool GRAD>
__device__ __forceinline__ void crossent_fwd_row_at(const float *__restrict__ pr, const float *__restrict__ pi, const int row, const bool live,
		const int t, const int lane, const int slot, const int wig, double *lds_d, ArgMax *lds_a, Top2 *lds_t,
		const int *__restrict__ labels, float *__restrict__ outr, float *__restrict__ outi, long ldo, float *__restrict__ s,
		float *__restrict__ loss, int *__restrict__ argmax, int cols, const GradPlanes &grad, int policy) {
	constexpr int STRIDE = 64 * G;
	// pass 1 (the only pass in the common case): sum |z|^2 in double (two fused multiply-adds per element: the squares of
	// floats are exact in double), and the two largest |z_k|^2 of the row in single precision
	double sum = 0.0;
	Top2 top = {-1.0f, -1.0f, 0x7fffffff, 0};
	auto visit = [&](float a, float b, int k) {
		sum = fma((double) b, (double) b, fma((double) a, (double) a, sum));
		const float q = fmaf(a, a, b * b);
		if (q > top.q1) {
			top.q2 = top.q1;
			top.q1 = q;
			top.i1 = k;
		} else if (q > top.q2) {
			top.q2 = q;
		}
	};
	if (V == 4) {
		for (int c = t * 4; c < cols; c += STRIDE * 4) {
			float4 a = ld4(pr + c, policy);
			float4 b = ld4(pi + c, policy);
			visit(a.x, b.x, c);
			visit(a.y, b.y, c + 1);
			visit(a.z, b.z, c + 2);
			visit(a.w, b.w, c + 3);
		}
	} else {
		for (int c = t; c < cols; c += STRIDE) visit(pr[c], pi[c], c);
	}
	sum = group_reduce<double, G>(sum, SumD(), lds_d, slot, wig, lane);
	top = group_reduce<Top2, G>(top, Top2Op(), lds_t, slot, wig, lane);
	float S = (float) sum;
	if (S <= 1.0e-15f) S = 1.0e-15f;
	double nrm = sqrt((double) S);
	if (nrm <= 1.0e-15) nrm = 1.0e-15;
	const double inv = 1.0 / nrm;
	const bool want_out = (outr != nullptr);
	// The reference argmax is taken over p_k = fl(|fl(z_k / sqrt S)|^2), which orders like |z_k|^2 except within a few
	// ulp.  When the runner-up is more than 1e-5 (relative) below the maximum the winner is already decided; otherwise,
	// or when the normalised planes are wanted, a second pass evaluates p_k exactly as the reference does.
	const bool clear_cut = top.q2 < top.q1 * (1.0f - 1.0e-5f);
	constexpr bool want_grad = GRAD;
	if (!want_out && !want_grad && clear_cut) {
		if (live && t == 0) {
			s[row] = S;
			loss[row] = label_loss(pr, pi, labels[row], cols, inv);
			argmax[row] = top.i1;
		}
		return;
	}

	ArgMax best = {-1.0f, 0x7fffffff};
	float *qr = want_out ? outr + (long) row * ldo : nullptr;
	float *qi = want_out ? outi + (long) row * ldo : nullptr;
	const int label = want_grad ? labels[row] : -1;
	const long goff = (long) row * grad.ld;
	if (V == 4) {
		for (int c = t * 4; c < cols; c += STRIDE * 4) {
			float4 a = *reinterpret_cast<const float4 *>(pr + c);
			float4 b = *reinterpret_cast<const float4 *>(pi + c);
			float o_r[4] = {(float) (a.x * inv), (float) (a.y * inv), (float) (a.z * inv), (float) (a.w * inv)};
			float o_i[4] = {(float) (b.x * inv), (float) (b.y * inv), (float) (b.z * inv), (float) (b.w * inv)};
#pragma unroll
			for (int k = 0; k < 4; ++k) {
				float p = (float) ((double) o_r[k] * o_r[k] + (double) o_i[k] * o_i[k]);
				if (p > best.v) best = ArgMax{p, c + k};
			}
			if (want_out && live) {
				*reinterpret_cast<float4 *>(qr + c) = make_float4(o_r[0], o_r[1], o_r[2], o_r[3]);
				*reinterpret_cast<float4 *>(qi + c) = make_float4(o_i[0], o_i[1], o_i[2], o_i[3]);
			}
			if (want_grad && live) {
				const float za[4] = {a.x, a.y, a.z, a.w}, zb[4] = {b.x, b.y, b.z, b.w};
				float g_r[4], g_i[4];
#pragma unroll
				for (int k = 0; k < 4; ++k) crossent_grad(za[k], zb[k], c + k == label, S, g_r[k], g_i[k]);
				*reinterpret_cast<float4 *>(grad.dz_re + goff + c) = make_float4(g_r[0], g_r[1], g_r[2], g_r[3]);
				*reinterpret_cast<float4 *>(grad.dz_im + goff + c) = make_float4(-g_i[0], -g_i[1], -g_i[2], -g_i[3]);
				if (grad.dzs_re) {
					*reinterpret_cast<float4 *>(grad.dzs_re + goff + c) = make_float4(g_r[0], g_r[1], g_r[2], g_r[3]);
					*reinterpret_cast<float4 *>(grad.dzs_im + goff + c) = make_float4(g_i[0], g_i[1], g_i[2], g_i[3]);
				}
			}
		}
	} else {
		for (int c = t; c < cols; c += STRIDE) {
			float o_r = (float) (pr[c] * inv), o_i = (float) (pi[c] * inv);
			float p = (float) ((double) o_r * o_r + (double) o_i * o_i);
			if (p > best.v) best = ArgMax{p, c};
			if (want_out && live) {
				qr[c] = o_r;
				qi[c] = o_i;
			}
			if (want_grad && live) {
				float g_r, g_i;
				crossent_grad(pr[c], pi[c], c == label, S, g_r, g_i);
				grad.dz_re[goff + c] = g_r;
				grad.dz_im[goff + c] = -g_i;
				if (grad.dzs_re) {
					grad.dzs_re[goff + c] = g_r;
					grad.dzs_im[goff + c] = g_i;
				}
			}
		}
	}
	best = group_reduce<ArgMax, G>(best, ArgMaxOp(), lds_a, slot, wig, lane);
	if (live && t == 0) {
		s[row] = S;
		loss[row] = label_loss(pr, pi, labels[row], cols, inv);
		argmax[row] = best.i;
	}
}

}  // namespace rows
}  // namespace cnet

#endif
