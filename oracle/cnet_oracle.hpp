// CPU restatement of CNet's per-sample complex-valued layer arithmetic.
//
// TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP path and the
// timed CPU baseline of the benchmark.  Nothing in the product (the HIP library, its
// C-ABI, the C++ host facade) may include, link or call it.
//
// Every function names the reference lines it follows (paths under the upstream CNet
// tree).  Arithmetic type choices (float vs double intermediates, accumulation order,
// complex product form (ac-bd, ad+bc)) follow the reference CPU path so results can be
// compared bit for bit with a build of the upstream sources (oracle/ref_shim.cpp).
//
// Planes: a complex vector of length n is two float arrays re[n], im[n]; a gradient
// carrier is four more: dz_re, dz_im, dzs_re, dzs_im  (dz = dL/dz, dzs = dL/d conj z).
#ifndef CNET_ORACLE_HPP_
#define CNET_ORACLE_HPP_

#include <algorithm>
#include <cassert>
#include <cmath>
#include <complex>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace orc {

typedef std::complex<float> cf;

// ------------------------------------------------------------------------------------
// Six-plane storage block (impl/vars.h:16-54): one allocation, planes back to back.
// ------------------------------------------------------------------------------------
struct Planes {
	int n;
	std::vector<float> store;
	float *re, *im, *dz_re, *dz_im, *dzs_re, *dzs_im;

	explicit Planes(int len = 0) : n(0), re(0), im(0), dz_re(0), dz_im(0), dzs_re(0), dzs_im(0) {
		if (len > 0) resize(len);
	}
	void resize(int len) {
		n = len;
		store.assign((size_t) 6 * len, 0.0f);
		re = store.data();
		im = re + len;
		dz_re = im + len;
		dz_im = dz_re + len;
		dzs_re = dz_im + len;
		dzs_im = dzs_re + len;
	}
	Planes(const Planes &o) : n(0) { *this = o; }
	Planes &operator=(const Planes &o) {
		if (this != &o) {
			resize(o.n > 0 ? o.n : 0);
			if (o.n > 0) store = o.store, rebind();
		}
		return *this;
	}
	void rebind() {
		re = store.data();
		im = re + n;
		dz_re = im + n;
		dz_im = dz_re + n;
		dzs_re = dz_im + n;
		dzs_im = dzs_re + n;
	}
	// impl/vars.h:49-54
	void zero_gradients() { std::fill(dz_re, dz_re + (size_t) 4 * n, 0.0f); }
	cf z(int i) const { return cf(re[i], im[i]); }
	cf dz(int i) const { return cf(dz_re[i], dz_im[i]); }
	cf dzs(int i) const { return cf(dzs_re[i], dzs_im[i]); }
};

// A read-only view of the upstream gradient of a consumer slot: the four gradient planes
// of the consumer's input block, already advanced to the producer's offset.
struct GradIn {
	const float *dz_re, *dz_im, *dzs_re, *dzs_im;
	cf dz(int i) const { return cf(dz_re[i], dz_im[i]); }
	cf dzs(int i) const { return cf(dzs_re[i], dzs_im[i]); }
};

// Accumulating view of the four gradient planes of a layer's own input block.
struct GradOut {
	float *dz_re, *dz_im, *dzs_re, *dzs_im;
};

// ------------------------------------------------------------------------------------
// xorshift64* generator and polar normal (utils/myrand.h:16-28, 63-65, 90-106).
// Used by tests and the bench to produce identical seeded inputs for every backend.
// ------------------------------------------------------------------------------------
struct Rng {
	uint64_t s;
	double spare;
	explicit Rng(uint64_t seed) : s(0x2545F4914F6CDD1DULL ^ seed), spare(0.0) {}
	uint64_t next() {
		uint64_t x = s;
		x ^= x >> 12;
		x ^= x << 25;
		x ^= x >> 27;
		s = x;
		return x * 0x2545F4914F6CDD1DULL;
	}
	double uniform() { return 5.42101086242752217E-20 * next(); }
	double normal(double mu, double sig) {
		if (spare == 0.) {
			double a, b, r;
			do {
				a = 2.0 * uniform() - 1.0;
				b = 2.0 * uniform() - 1.0;
				r = a * a + b * b;
			} while (r >= 1.0 || r == 0.0);
			double f = sqrt(-2.0 * log(r) / r);
			spare = a * f;
			return mu + sig * b * f;
		}
		double f = spare;
		spare = 0.;
		return mu + sig * f;
	}
};

// ------------------------------------------------------------------------------------
// Linear  (impl/linear.h:51-110).  Input block = [x (K) | W (N rows of K)], y_o = sum_i x_i W[o][i].
// ------------------------------------------------------------------------------------
inline void linear_forward(int K, int N, const float *xr, const float *xi, const float *wr,
		const float *wi, float *yr, float *yi) {
#pragma omp parallel for
	for (int o = 0; o < N; ++o) {
		cf acc = 0;
		const float *wro = wr + (size_t) o * K, *wio = wi + (size_t) o * K;
		for (int i = 0; i < K; ++i) acc += cf(xr[i], xi[i]) * cf(wro[i], wio[i]);
		yr[o] = acc.real();
		yi[o] = acc.imag();
	}
}

// impl/linear.h:73-110: outer loop over the input index, inner over outputs; the x
// gradients accumulate straight into the float planes in output order; each W entry is
// touched exactly once per call.
inline void linear_backward(int K, int N, const float *xr, const float *xi, const float *wr,
		const float *wi, GradIn g, GradOut dx, GradOut dw) {
#pragma omp parallel for
	for (int i = 0; i < K; ++i) {
		for (int o = 0; o < N; ++o) {
			cf G = g.dz(o), Gs = g.dzs(o);
			size_t wi_idx = (size_t) o * K + i;
			cf w(wr[wi_idx], wi[wi_idx]);
			cf a = G * w;
			cf b = Gs * std::conj(w);
			dx.dz_re[i] += a.real();
			dx.dz_im[i] += a.imag();
			dx.dzs_re[i] += b.real();
			dx.dzs_im[i] += b.imag();
			cf x(xr[i], xi[i]);
			a = G * x;
			b = Gs * std::conj(x);
			dw.dz_re[wi_idx] += a.real();
			dw.dz_im[wi_idx] += a.imag();
			dw.dzs_re[wi_idx] += b.real();
			dw.dzs_im[wi_idx] += b.imag();
		}
	}
}

// ------------------------------------------------------------------------------------
// Fourier transform (impl/utils.h:83-297, impl/ft.h:37-80).
// The forward path is a float FFT whose twiddles come from a float rotation recurrence;
// that recurrence is what makes the CPU forward differ from the exact DFT by ~1e-4 at
// n=4096, so it is restated step for step.
// ------------------------------------------------------------------------------------
inline unsigned bit_reverse32(unsigned v) {
	unsigned r = 0;
	for (int b = 0; b < 32; ++b)
		if (v & (0x80000000u >> b)) r |= (1u << b);
	return r;
}

// impl/utils.h:178-230  (radix-2, decimation in time, sign -).
inline void fft_pow2(int n, float *re, float *im) {
	if (n <= 1) return;
	int levels = -1;
	for (int b = 0; b < 32; ++b)
		if ((1 << b) == n) levels = b;
	assert(levels >= 0);
	for (int a = 0; a < n; ++a) {
		int b = (int) (bit_reverse32((unsigned) a) >> (32 - levels));
		if (b > a) {
			std::swap(re[a], re[b]);
			std::swap(im[a], im[b]);
		}
	}
	std::vector<float> ct(n / 2), st(n / 2);
	ct[0] = 1;
	st[0] = 0;
	float qc = std::cos(2 * M_PI / n);
	float qs = std::sin(2 * M_PI / n);
	for (int t = 1; t < n / 2; ++t) {
		ct[t] = ct[t - 1] * qc - st[t - 1] * qs;
		st[t] = st[t - 1] * qc + ct[t - 1] * qs;
	}
	for (int size = 2; size <= n; size *= 2) {
		int half = size / 2, step = n / size;
		for (int base = 0; base < n; base += size) {
			for (int j = base, t = 0; j < base + half; ++j, t += step) {
				float pr = re[j + half] * ct[t] + im[j + half] * st[t];
				float pi = -re[j + half] * st[t] + im[j + half] * ct[t];
				re[j + half] = re[j] - pr;
				im[j + half] = im[j] - pi;
				re[j] += pr;
				im[j] += pi;
			}
		}
	}
}

// impl/utils.h:163-176: circular convolution of two power-of-two vectors, result in y.
inline void fft_convolve_pow2(int n, float *xr, float *xi, float *yr, float *yi) {
	fft_pow2(n, xr, xi);
	fft_pow2(n, yr, yi);
	for (int t = 0; t < n; ++t) {
		float tmp = xr[t] * yr[t] - xi[t] * yi[t];
		xi[t] = xi[t] * yr[t] + xr[t] * yi[t];
		xr[t] = tmp;
	}
	fft_pow2(n, xi, xr);  // inverse = forward with planes swapped
	for (int t = 0; t < n; ++t) {
		yr[t] = xr[t] / n;
		yi[t] = xi[t] / n;
	}
}

// impl/utils.h:232-297: chirp-z for arbitrary length.
inline void fft_bluestein(int n, float *re, float *im) {
	int m = 1;
	while (m < n * 2 - 1) m *= 2;
	std::vector<float> tc(2 * n), ts(2 * n);
	tc[0] = 1;
	ts[0] = 0;
	float qc = std::cos(M_PI / n);
	float qs = std::sin(M_PI / n);
	for (int t = 1; t < 2 * n; ++t) {
		tc[t] = tc[t - 1] * qc - ts[t - 1] * qs;
		ts[t] = ts[t - 1] * qc + tc[t - 1] * qs;
	}
	std::vector<float> ct(n), st(n);
	for (int t = 0; t < n; ++t) {
		int j = (int) (((long) t * t) % (n * 2));
		ct[t] = tc[j];
		st[t] = ts[j];
	}
	std::vector<float> ar(m, 0.0f), ai(m, 0.0f), br(m, 0.0f), bi(m, 0.0f);
	for (int t = 0; t < n; ++t) {
		ar[t] = re[t] * ct[t] + im[t] * st[t];
		ai[t] = -re[t] * st[t] + im[t] * ct[t];
	}
	br[0] = ct[0];
	bi[0] = st[0];
	for (int t = 1; t < n; ++t) {
		br[t] = br[m - t] = ct[t];
		bi[t] = bi[m - t] = st[t];
	}
	fft_convolve_pow2(m, ar.data(), ai.data(), br.data(), bi.data());
	for (int t = 0; t < n; ++t) {
		re[t] = br[t] * ct[t] + bi[t] * st[t];
		im[t] = -br[t] * st[t] + bi[t] * ct[t];
	}
}

// impl/utils.h:89-99
inline void fft_any(int n, float *re, float *im) {
	if (n == 0) return;
	if ((n & (n - 1)) == 0)
		fft_pow2(n, re, im);
	else
		fft_bluestein(n, re, im);
}

// impl/utils.h:300-320: root[k] = exp(-2 pi i k / n) evaluated in double, stored in float.
inline std::vector<cf> unity_roots(int n) {
	std::vector<cf> r;
	r.reserve(n);
	for (int k = 0; k <= n - 1; ++k) r.push_back(cf(std::cos(-2 * k * M_PI / n), std::sin(-2 * k * M_PI / n)));
	return r;
}

// impl/ft.h:37-55: y = FFT(x) / sqrt(n); the divisor is a double sqrt of the int length.
inline void dft_forward(int n, const float *xr, const float *xi, float *yr, float *yi) {
	std::vector<float> br(xr, xr + n), bi(xi, xi + n);
	fft_any(n, br.data(), bi.data());
	for (int t = 0; t < n; ++t) {
		br[t] /= sqrt(n);
		bi[t] /= sqrt(n);
	}
	std::copy(br.begin(), br.end(), yr);
	std::copy(bi.begin(), bi.end(), yi);
}

// impl/ft.h:57-80: O(n^2) sums against the root table, float scaling.
inline void dft_backward(int n, const std::vector<cf> &root, GradIn g, GradOut dx) {
	float scaling = sqrt(n);
#pragma omp parallel for
	for (int q = 0; q < n; ++q) {
		cf a = 0, b = 0;
		for (int p = 0; p < n; ++p) {
			int e = q * p;
			cf w = root[e % n];
			a += g.dz(p) * w;
			b += g.dzs(p) * std::conj(w);
		}
		dx.dz_re[q] += a.real() / scaling;
		dx.dz_im[q] += a.imag() / scaling;
		dx.dzs_re[q] += b.real() / scaling;
		dx.dzs_im[q] += b.imag() / scaling;
	}
}

// ------------------------------------------------------------------------------------
// TriangFourier  (impl/ft.h:139-189): the O(n^2) DFT sums restricted to in <= out,
// y[o] = (1/sqrt n) sum_{i <= o} x[i] root(i o), float accumulation in index order.
// ------------------------------------------------------------------------------------
inline void triang_forward(int n, const std::vector<cf> &root, const float *xr, const float *xi, float *yr, float *yi) {
	float scaling = sqrt(n);
	for (int o = 0; o < n; ++o) {
		cf sum = 0;
		for (int i = 0; i < n; ++i) {
			if (o < i) continue;
			int e = i * o;
			sum += cf(xr[i], xi[i]) * root[e % n];
		}
		sum /= scaling;
		yr[o] = sum.real();
		yi[o] = sum.imag();
	}
}

inline void triang_backward(int n, const std::vector<cf> &root, GradIn g, GradOut dx) {
	float scaling = sqrt(n);
	for (int i = 0; i < n; ++i) {
		cf a = 0, b = 0;
		for (int o = 0; o < n; ++o) {
			if (o < i) continue;
			int e = i * o;
			cf w = root[e % n];
			a += g.dz(o) * w;
			b += g.dzs(o) * std::conj(w);
		}
		dx.dz_re[i] += a.real() / scaling;
		dx.dz_im[i] += a.imag() / scaling;
		dx.dzs_re[i] += b.real() / scaling;
		dx.dzs_im[i] += b.imag() / scaling;
	}
}

// ------------------------------------------------------------------------------------
// Hadamard  (impl/hadamard.h:34-68).  Input block = [u (n) | v (n)], y = u .* v.
// ------------------------------------------------------------------------------------
inline void hadamard_forward(int n, const float *ur, const float *ui, const float *vr, const float *vi,
		float *yr, float *yi) {
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		cf p = cf(ur[k], ui[k]) * cf(vr[k], vi[k]);
		yr[k] = p.real();
		yi[k] = p.imag();
	}
}

inline void hadamard_backward(int n, const float *ur, const float *ui, const float *vr, const float *vi,
		GradIn g, GradOut du, GradOut dv) {
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		cf G = g.dz(k), Gs = g.dzs(k);
		cf u(ur[k], ui[k]), v(vr[k], vi[k]);
		cf a = G * v, b = Gs * std::conj(v);
		du.dz_re[k] += a.real();
		du.dz_im[k] += a.imag();
		du.dzs_re[k] += b.real();
		du.dzs_im[k] += b.imag();
		a = G * u;
		b = Gs * std::conj(u);
		dv.dz_re[k] += a.real();
		dv.dz_im[k] += a.imag();
		dv.dzs_re[k] += b.real();
		dv.dzs_im[k] += b.imag();
	}
}

// ------------------------------------------------------------------------------------
// CGelu  (impl/relu.h:10, 119-168): tanh-GELU applied to the real and imaginary parts.
// ------------------------------------------------------------------------------------
inline float gelu_scale() { return sqrtf(2.0f / M_PI); }

inline float gelu_value(float t) {
	float cube = 0.044715f * t * t * t;
	return 0.5f * t * (1.0f + tanhf(gelu_scale() * (t + cube)));
}

inline float gelu_slope(float t) {
	float cube = 0.044715f * t * t * t;
	float arg = gelu_scale() * (t + cube);
	float th = tanhf(arg);
	float ch = coshf(arg);
	float sech2 = 1.0f / (ch * ch);
	return 0.5f * (1.0f + th) + t * 0.5f * sech2 * gelu_scale() * (1.0f + 3.0f * 0.044715f * t * t);
}

inline void gelu_forward(int n, const float *xr, const float *xi, float *yr, float *yi) {
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		yr[k] = gelu_value(xr[k]);
		yi[k] = gelu_value(xi[k]);
	}
}

inline void gelu_backward(int n, const float *xr, const float *xi, GradIn g, GradOut dx) {
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		float px = 0.5 * gelu_slope(xr[k]);  // double product, rounded to float
		float py = 0.5 * gelu_slope(xi[k]);
		float s = px + py, d = px - py;
		cf a = 0, b = 0;
		a += g.dz(k) * s + g.dzs(k) * d;
		b += g.dz(k) * d + g.dzs(k) * s;
		dx.dz_re[k] += a.real();
		dx.dz_im[k] += a.imag();
		dx.dzs_re[k] += b.real();
		dx.dzs_im[k] += b.imag();
	}
}

// ------------------------------------------------------------------------------------
// CRelu  (impl/relu.h:32-63): passes z where both Re z > 0 and Im z > 0, else 0; the
// backward pass hands both gradients through under the same test.
// ------------------------------------------------------------------------------------
inline void crelu_forward(int n, const float *xr, const float *xi, float *yr, float *yi) {
	for (int k = 0; k < n; ++k) {
		bool on = xr[k] > 0 && xi[k] > 0;
		yr[k] = on ? xr[k] : 0;
		yi[k] = on ? xi[k] : 0;
	}
}

inline void crelu_backward(int n, const float *xr, const float *xi, GradIn g, GradOut dx) {
	for (int k = 0; k < n; ++k) {
		if (xr[k] > 0 && xi[k] > 0) {
			dx.dz_re[k] += g.dz_re[k];
			dx.dz_im[k] += g.dz_im[k];
			dx.dzs_re[k] += g.dzs_re[k];
			dx.dzs_im[k] += g.dzs_im[k];
		}
	}
}

// ------------------------------------------------------------------------------------
// Residual  (impl/residual.h:40-77).  Input block = [u | v], y = u + v.
// ------------------------------------------------------------------------------------
inline void residual_forward(int n, const float *ur, const float *ui, const float *vr, const float *vi,
		float *yr, float *yi) {
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		cf s = cf(ur[k], ui[k]) + cf(vr[k], vi[k]);
		yr[k] = s.real();
		yi[k] = s.imag();
	}
}

inline void residual_backward(int n, GradIn g, GradOut du, GradOut dv) {
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		cf G = g.dz(k), Gs = g.dzs(k);
		du.dz_re[k] += G.real();
		du.dz_im[k] += G.imag();
		du.dzs_re[k] += Gs.real();
		du.dzs_im[k] += Gs.imag();
		dv.dz_re[k] += G.real();
		dv.dz_im[k] += G.imag();
		dv.dzs_re[k] += Gs.real();
		dv.dzs_im[k] += Gs.imag();
	}
}

// ------------------------------------------------------------------------------------
// SoftMax = L2 normalisation  (impl/softmax.h:33-73) with the generic Wirtinger chain rule
// (impl/cfunc.h:290-325).  State kept between forward and backward: S and S^(3/2).
// ------------------------------------------------------------------------------------
struct SoftMaxState {
	float square_norm;
	float norm_cubed;
};

inline SoftMaxState softmax_forward(int n, const float *zr, const float *zi, float *yr, float *yi) {
	double sum = 0.0;
	for (int k = 0; k < n; ++k) sum = sum + (std::pow(zr[k], 2) + std::pow(zi[k], 2));
	SoftMaxState st;
	st.square_norm = sum;
	sum = sqrt(sum);
	if (sum <= 1.0e-15) sum = 1.0e-15;
	st.norm_cubed = pow(sum, 3);
	if (st.norm_cubed < 1.0e-15) sum = 1.0e-15;
	if (yr) {
#pragma omp parallel for
		for (int k = 0; k < n; ++k) {
			yr[k] = (float) zr[k] / sum;
			yi[k] = (float) zi[k] / sum;
		}
	}
	return st;
}

inline cf softmax_dz(const SoftMaxState &st, const float *zr, const float *zi, int out, int in) {
	cf zi_(zr[in], zi[in]);
	if (in == out) return 0.5f * (cf(2.0f * st.square_norm, 0) - zi_ * std::conj(zi_)) / st.norm_cubed;
	return -0.5f * cf(zr[out], zi[out]) * std::conj(zi_) / st.norm_cubed;
}

inline cf softmax_dzs(const SoftMaxState &st, const float *zr, const float *zi, int out, int in) {
	cf zi_(zr[in], zi[in]);
	if (in == out) return -0.5f * zi_ * zi_ / st.norm_cubed;
	return -0.5f * cf(zr[out], zi[out]) * zi_ / st.norm_cubed;
}

inline void softmax_backward(int n, const SoftMaxState &st, const float *zr, const float *zi, GradIn g, GradOut dx) {
#pragma omp parallel for
	for (int i = 0; i < n; ++i) {
		cf a = 0, b = 0;
		for (int o = 0; o < n; ++o) {
			cf G = g.dz(o), Gs = g.dzs(o);
			cf d1 = softmax_dz(st, zr, zi, o, i);
			cf d2 = softmax_dzs(st, zr, zi, o, i);
			a += G * d1;
			a += Gs * std::conj(d2);
			b += G * d2;
			b += Gs * std::conj(d1);
		}
		dx.dz_re[i] += a.real();
		dx.dz_im[i] += a.imag();
		dx.dzs_re[i] += b.real();
		dx.dzs_im[i] += b.imag();
	}
}

// ------------------------------------------------------------------------------------
// CrossEntropy  (impl/crossent.h:44-130).
// ------------------------------------------------------------------------------------
// forward: returns the clamped S = sum |z|^2; out = z / sqrt(S)   (impl/crossent.h:61-80)
inline float crossent_forward(int n, const float *zr, const float *zi, float *outr, float *outi) {
	double sum = 0.0;
	for (int k = 0; k < n; ++k) sum += (std::pow(zr[k], 2) + std::pow(zi[k], 2));
	float S = sum;
	if (S <= 1.0e-15) S = 1.0e-15;
	sum = sqrt(S);
	if (sum <= 1.0e-15) sum = 1.0e-15;
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		outr[k] = zr[k] / sum;
		outi[k] = zi[k] / sum;
	}
	return S;
}

// impl/crossent.h:38-59
inline float crossent_probability(const float *outr, const float *outi, int k) {
	return std::pow(outr[k], 2) + std::pow(outi[k], 2);
}

inline float crossent_loss(const float *outr, const float *outi, int label) {
	float p = crossent_probability(outr, outi, label);
	p = (p < 1e-15 ? 1e-15 : p);
	return -std::log(p);
}

// impl/crossent.h:82-104: assigns (does not accumulate) both gradient planes.
inline void crossent_backward(int n, const float *zr, const float *zi, float S, int label, GradOut dx) {
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		if (k == label) {
			float m = std::pow(zr[k], 2) + std::pow(zi[k], 2);
			m = (m < 1e-15 ? 1e-15 : m);
			dx.dzs_re[k] = -zr[k] * (S - m) / (m * S);
			dx.dzs_im[k] = -zi[k] * (S - m) / (m * S);
		} else {
			dx.dzs_re[k] = zr[k] / S;
			dx.dzs_im[k] = zi[k] / S;
		}
		dx.dz_re[k] = dx.dzs_re[k];
		dx.dz_im[k] = -dx.dzs_im[k];
	}
}

// impl/crossent.h:117-130: first index of the strict maximum of |out_k|^2.
inline int crossent_prediction(int n, const float *outr, const float *outi) {
	float best = std::pow(outr[0], 2) + std::pow(outi[0], 2);
	int arg = 0;
	for (int k = 1; k < n; ++k) {
		float v = std::pow(outr[k], 2) + std::pow(outi[k], 2);
		if (v > best) {
			arg = k;
			best = v;
		}
	}
	return arg;
}

// ------------------------------------------------------------------------------------
// L2Out  (impl/l2out.h:33-58, impl/cfunc.h:327-339): loss = sum |z|^2 in float.
// ------------------------------------------------------------------------------------
inline float l2out_forward(int n, const float *zr, const float *zi) {
	float acc = 0;
	for (int k = 0; k < n; ++k) acc += (float) pow(zr[k], 2) + (float) pow(zi[k], 2);
	return acc;
}

inline void l2out_backward(int n, const float *zr, const float *zi, GradOut dx) {
#pragma omp parallel for
	for (int k = 0; k < n; ++k) {
		dx.dz_re[k] += zr[k];
		dx.dz_im[k] += -zi[k];
		dx.dzs_re[k] += zr[k];
		dx.dzs_im[k] += zi[k];
	}
}

// ------------------------------------------------------------------------------------
// CEmbedding  (impl/embed.h:109-148): row gather with zero padding; dzs scatter-add.
// tokens holds `count` valid ids (count <= slots).
// ------------------------------------------------------------------------------------
inline void embedding_forward(int dim, int slots, const float *tr, const float *ti, const int *tokens, int count,
		float *yr, float *yi) {
	for (int p = 0; p < count; ++p) {
		size_t src = (size_t) tokens[p] * dim;
		std::copy(tr + src, tr + src + dim, yr + (size_t) dim * p);
		std::copy(ti + src, ti + src + dim, yi + (size_t) dim * p);
	}
	if (count < slots) {
		memset(yr + (size_t) dim * count, 0, sizeof(float) * dim * (slots - count));
		memset(yi + (size_t) dim * count, 0, sizeof(float) * dim * (slots - count));
	}
}

inline void embedding_backward(int dim, const int *tokens, int count, const float *gsr, const float *gsi,
		float *dsr, float *dsi) {
	for (int p = 0; p < count; ++p) {
		size_t dst = (size_t) tokens[p] * dim;
		for (int k = 0; k < dim; ++k) {
			dsr[dst + k] += gsr[(size_t) dim * p + k];
			dsi[dst + k] += gsi[(size_t) dim * p + k];
		}
	}
}

// ------------------------------------------------------------------------------------
// SGD step  (impl/cfunc.h:147-152).  The caller zeroes the gradients afterwards.
// ------------------------------------------------------------------------------------
inline void sgd_update(int n, float *zr, float *zi, const float *dsr, const float *dsi, float lr) {
	for (int k = 0; k < n; ++k) {
		zr[k] -= lr * (dsr[k]);
		zi[k] -= lr * dsi[k];
	}
}

// ------------------------------------------------------------------------------------
// Adam-style step  (impl/cfunc.h:273-287; device twin gpu/kernels.cpp:494-514).  The first
// moment lives in the node's own dz planes (impl/cfunc.h:341-349); there is no second
// moment.  pow(float, int) promotes to double, so the step is evaluated in double and
// rounded once when it is subtracted from the float parameter.
// ------------------------------------------------------------------------------------
inline void adam_update(int n, float *zr, float *zi, float *mr, float *mi, const float *dsr, const float *dsi,
		float lr, float beta1, int t) {
	for (int k = 0; k < n; ++k) {
		mr[k] = mr[k] * beta1 + (1 - beta1) * dsr[k];
		mi[k] = mi[k] * beta1 + (1 - beta1) * dsi[k];
		zr[k] -= lr * mr[k] / (1 - pow(beta1, t + 1));
		zi[k] -= lr * mi[k] / (1 - pow(beta1, t + 1));
	}
}

// ====================================================================================
// Graph runtime: the per-sample semantics of ComplexNet (impl/cnet.h:228-289, 366-421)
// and of the producer-writes-into-consumer wiring of CFunc (impl/cfunc.h:211-224).
// ====================================================================================
enum Kind {  // numeric values as impl/cnet.h:31-42
	kHadamard = 1, kEmbedding = 2, kLinear = 3, kFourier = 4, kCrossEntropy = 5, kResidual = 6,
	kSoftMax = 7, kInput = 8, kCrelu = 9, kGelu = 10, kL2Out = 11, kTriangFourier = 12
};

struct Node {
	int kind;
	int uid;
	int out_size;
	int p0, p1, p2;  // kind-specific sizes
	Planes in;      // the node's own input block
	Planes out;     // CrossEntropy: normalised output (n); L2Out: loss (1)
	std::vector<Node *> next;
	std::vector<int> offset;
	std::vector<Node *> prev;
	bool is_input, is_output;
	std::vector<int> tokens;     // embedding
	std::vector<cf> roots;       // fourier
	SoftMaxState sm;
	float S;                     // cross entropy square norm
	Node() : kind(0), uid(0), out_size(0), p0(0), p1(0), p2(0), is_input(false), is_output(false), S(0) {
		sm.square_norm = 0;
		sm.norm_cubed = 0;
	}
	GradIn upstream(int c) const {
		GradIn g;
		const Planes &o = next[c]->in;
		int off = offset[c];
		g.dz_re = o.dz_re + off;
		g.dz_im = o.dz_im + off;
		g.dzs_re = o.dzs_re + off;
		g.dzs_im = o.dzs_im + off;
		return g;
	}
	GradOut own(int off) {
		GradOut d;
		d.dz_re = in.dz_re + off;
		d.dz_im = in.dz_im + off;
		d.dzs_re = in.dzs_re + off;
		d.dzs_im = in.dzs_im + off;
		return d;
	}
};

class Net {
	std::vector<Node *> list_;
	std::map<int, Node *> by_uid_;
	std::vector<Node *> inputs_;
	int next_uid_;

public:
	Net() : next_uid_(0) {}
	~Net() {
		for (size_t k = 0; k < list_.size(); ++k) delete list_[k];
	}
	Node *at(int uid) { return by_uid_.count(uid) ? by_uid_[uid] : NULL; }
	const std::vector<Node *> &nodes() const { return list_; }

	// Sizes follow the constructors: CInput(out) impl/cinput.h:15-18; Linear(in1,in2)
	// impl/linear.h:17-22; FourierTrans(n) impl/ft.h:19-21; Hadamard(n,n) impl/hadamard.h:14-17;
	// CGelu(n) impl/relu.h:102; Residual(n) impl/residual.h:15; SoftMax(n) impl/softmax.h:14-16;
	// CrossEntropy(n) impl/crossent.h:14-17; L2Out(n) impl/l2out.h:14-16;
	// CEmbedding(dim, slots, vocab) impl/embed.h:41-45.
	int add(int kind, int p0, int p1, int p2, const int *in_uids, int n_in, int uid = 0) {
		Node *nd = new Node();
		nd->kind = kind;
		nd->p0 = p0;
		nd->p1 = p1;
		nd->p2 = p2;
		int in_len = 0;
		switch (kind) {
		case kInput: in_len = p0; nd->out_size = p0; nd->is_input = true; break;
		case kLinear: assert(p1 % p0 == 0); in_len = p0 + p1; nd->out_size = p1 / p0; break;
		case kFourier: in_len = p0; nd->out_size = p0; nd->roots = unity_roots(p0); break;
		case kHadamard: in_len = 2 * p0; nd->out_size = p0; break;
		case kGelu: in_len = p0; nd->out_size = p0; break;
		case kCrelu: in_len = p0; nd->out_size = p0; break;
		case kTriangFourier: in_len = p0; nd->out_size = p0; nd->roots = unity_roots(p0); break;
		case kResidual: in_len = 2 * p0; nd->out_size = p0; break;
		case kSoftMax: in_len = p0; nd->out_size = p0; break;
		case kCrossEntropy: in_len = p0; nd->out_size = 1; nd->is_output = true; nd->out.resize(p0); break;
		case kL2Out: in_len = p0; nd->out_size = 1; nd->is_output = true; nd->out.resize(1); break;
		case kEmbedding: in_len = p2 * p0; nd->out_size = p1 * p0; nd->is_input = true; break;
		default: delete nd; return -1;
		}
		nd->in.resize(in_len);
		if (uid > 0) {  // impl/cnet.h:228-246: an explicit uid is kept and moves the counter past it
			assert(!by_uid_.count(uid));
			nd->uid = uid;
			next_uid_ = std::max(next_uid_, uid);
		} else {
			nd->uid = ++next_uid_;
		}
		list_.push_back(nd);
		by_uid_[nd->uid] = nd;
		if (nd->is_input) inputs_.push_back(nd);
		int off = 0;  // impl/cnet.h:259-268: running sum of the producers' output sizes
		for (int k = 0; k < n_in; ++k) {
			Node *src = by_uid_[in_uids[k]];
			assert(src);
			assert(nd->in.n >= off + src->out_size);
			src->next.push_back(nd);
			src->offset.push_back(off);
			nd->prev.push_back(src);
			off += src->out_size;
		}
		return nd->uid;
	}

	// Run one node's forward, writing into every consumer at its offset.
	void node_forward(Node *nd) {
		int nc = (int) nd->next.size();
		std::vector<float> yr, yi;
		if (!nd->is_output) {
			assert(nc);
			yr.resize(nd->out_size);
			yi.resize(nd->out_size);
		}
		const Planes &x = nd->in;
		switch (nd->kind) {
		case kInput:
			std::copy(x.re, x.re + x.n, yr.begin());
			std::copy(x.im, x.im + x.n, yi.begin());
			break;
		case kLinear:
			linear_forward(nd->p0, nd->out_size, x.re, x.im, x.re + nd->p0, x.im + nd->p0, yr.data(), yi.data());
			break;
		case kFourier: dft_forward(nd->p0, x.re, x.im, yr.data(), yi.data()); break;
		case kHadamard:
			hadamard_forward(nd->p0, x.re, x.im, x.re + nd->p0, x.im + nd->p0, yr.data(), yi.data());
			break;
		case kGelu: gelu_forward(nd->p0, x.re, x.im, yr.data(), yi.data()); break;
		case kCrelu: crelu_forward(nd->p0, x.re, x.im, yr.data(), yi.data()); break;
		case kTriangFourier: triang_forward(nd->p0, nd->roots, x.re, x.im, yr.data(), yi.data()); break;
		case kResidual:
			residual_forward(nd->p0, x.re, x.im, x.re + nd->p0, x.im + nd->p0, yr.data(), yi.data());
			break;
		case kSoftMax: nd->sm = softmax_forward(nd->p0, x.re, x.im, yr.data(), yi.data()); break;
		case kCrossEntropy: nd->S = crossent_forward(nd->p0, x.re, x.im, nd->out.re, nd->out.im); break;
		case kL2Out: nd->out.re[0] = l2out_forward(nd->p0, x.re, x.im); break;
		case kEmbedding:
			embedding_forward(nd->p0, nd->p1, x.re, x.im, nd->tokens.data(), (int) nd->tokens.size(), yr.data(),
					yi.data());
			break;
		}
		for (int c = 0; c < nc; ++c) {
			std::copy(yr.begin(), yr.end(), nd->next[c]->in.re + nd->offset[c]);
			std::copy(yi.begin(), yi.end(), nd->next[c]->in.im + nd->offset[c]);
		}
	}

	// Every layer adds the contribution of each consumer in turn (the per-consumer outer
	// loops of impl/linear.h:74, impl/ft.h:59, impl/hadamard.h:47, ...).
	void node_backward(Node *nd, int label) {
		int nc = (int) nd->next.size();
		Planes &x = nd->in;
		switch (nd->kind) {
		case kInput:  // impl/cinput.h:54-65: only dzs is gathered
			for (int k = 0; k < x.n; ++k)
				for (int c = 0; c < nc; ++c) {
					x.dzs_re[k] += nd->next[c]->in.dzs_re[nd->offset[c] + k];
					x.dzs_im[k] += nd->next[c]->in.dzs_im[nd->offset[c] + k];
				}
			break;
		case kEmbedding:
			for (size_t p = 0; p < nd->tokens.size(); ++p)
				for (int k = 0; k < nd->p0; ++k)
					for (int c = 0; c < nc; ++c) {
						size_t dst = (size_t) nd->tokens[p] * nd->p0 + k;
						x.dzs_re[dst] += nd->next[c]->in.dzs_re[nd->offset[c] + nd->p0 * p + k];
						x.dzs_im[dst] += nd->next[c]->in.dzs_im[nd->offset[c] + nd->p0 * p + k];
					}
			break;
		case kLinear:
			for (int c = 0; c < nc; ++c)
				linear_backward(nd->p0, nd->out_size, x.re, x.im, x.re + nd->p0, x.im + nd->p0, nd->upstream(c),
						nd->own(0), nd->own(nd->p0));
			break;
		case kFourier:
			for (int c = 0; c < nc; ++c) dft_backward(nd->p0, nd->roots, nd->upstream(c), nd->own(0));
			break;
		case kHadamard:
			for (int c = 0; c < nc; ++c)
				hadamard_backward(nd->p0, x.re, x.im, x.re + nd->p0, x.im + nd->p0, nd->upstream(c), nd->own(0),
						nd->own(nd->p0));
			break;
		case kGelu:
			for (int c = 0; c < nc; ++c) gelu_backward(nd->p0, x.re, x.im, nd->upstream(c), nd->own(0));
			break;
		case kCrelu:
			for (int c = 0; c < nc; ++c) crelu_backward(nd->p0, x.re, x.im, nd->upstream(c), nd->own(0));
			break;
		case kTriangFourier:
			for (int c = 0; c < nc; ++c) triang_backward(nd->p0, nd->roots, nd->upstream(c), nd->own(0));
			break;
		case kResidual:
			for (int c = 0; c < nc; ++c) residual_backward(nd->p0, nd->upstream(c), nd->own(0), nd->own(nd->p0));
			break;
		case kSoftMax:
			for (int c = 0; c < nc; ++c) softmax_backward(nd->p0, nd->sm, x.re, x.im, nd->upstream(c), nd->own(0));
			break;
		case kCrossEntropy:
			// impl/cnet.h:400-411: only backward(label) does work; plain backward() is empty.
			if (label >= 0) crossent_backward(nd->p0, x.re, x.im, nd->S, label, nd->own(0));
			break;
		case kL2Out: l2out_backward(nd->p0, x.re, x.im, nd->own(0)); break;
		}
	}

	// impl/cnet.h:366-377
	void forward() {
		for (size_t k = 0; k < list_.size(); ++k) {
			if (!list_[k]->is_input) list_[k]->in.zero_gradients();
			node_forward(list_[k]);
		}
	}
	// impl/cnet.h:389-411 (label < 0 selects the label-free variant)
	void backward(int label) {
		for (int k = (int) list_.size() - 1; k >= 0; --k) node_backward(list_[k], label);
	}
	// impl/cnet.h:413-421: every input node (data inputs too) steps, then clears all four
	// gradient planes.
	void update(float lr, int batch) {
		for (size_t k = 0; k < inputs_.size(); ++k) {
			Planes &x = inputs_[k]->in;
			sgd_update(x.n, x.re, x.im, x.dzs_re, x.dzs_im, lr / batch);
			x.zero_gradients();
		}
	}
	// impl/cnet.h:423-431: every input node takes the Adam-style step, then only dz* is cleared
	// (dz keeps the first moment).
	void adam_update_inputs(float lr, int batch, float beta, int t) {
		for (size_t k = 0; k < inputs_.size(); ++k) {
			Planes &x = inputs_[k]->in;
			adam_update(x.n, x.re, x.im, x.dz_re, x.dz_im, x.dzs_re, x.dzs_im, lr / batch, beta, t);
			std::fill(x.dzs_re, x.dzs_re + x.n, 0.0f);
			std::fill(x.dzs_im, x.dzs_im + x.n, 0.0f);
		}
	}
	// ---- the .mod record stream of impl/model_saver.h:483-967: big-endian int32 / float32 throughout.
	//   magic 0xABCDE0EE, then per function in insertion order:
	//   type id, uid, input length, output size, number of producers, producer uids,
	//   then CInput: re[len], im[len]; CEmbedding: dim, slots, vocab, re[len], im[len]; Linear: in1, in2.
	static void put32(std::string &o, uint32_t v) {
		for (int k = 3; k >= 0; --k) o.push_back((char) ((v >> (8 * k)) & 0xff));
	}
	static void putf(std::string &o, const float *p, int n) {
		for (int k = 0; k < n; ++k) {
			uint32_t u;
			memcpy(&u, p + k, 4);
			put32(o, u);
		}
	}
	std::string save() const {
		std::string o;
		put32(o, 0xABCDE0EEu);
		for (size_t k = 0; k < list_.size(); ++k) {
			const Node *nd = list_[k];
			put32(o, (uint32_t) nd->kind);
			put32(o, (uint32_t) nd->uid);
			put32(o, (uint32_t) nd->in.n);
			put32(o, (uint32_t) nd->out_size);
			put32(o, (uint32_t) nd->prev.size());
			for (size_t q = 0; q < nd->prev.size(); ++q) put32(o, (uint32_t) nd->prev[q]->uid);
			if (nd->kind == kEmbedding) {
				put32(o, (uint32_t) nd->p0);
				put32(o, (uint32_t) nd->p1);
				put32(o, (uint32_t) nd->p2);
			}
			if (nd->kind == kInput || nd->kind == kEmbedding) {
				putf(o, nd->in.re, nd->in.n);
				putf(o, nd->in.im, nd->in.n);
			}
			if (nd->kind == kLinear) {
				put32(o, (uint32_t) nd->p0);
				put32(o, (uint32_t) nd->p1);
			}
		}
		return o;
	}
	// Appends the stored functions to this net (upstream restores into an empty net); false on a bad magic number,
	// an unknown type id or a truncated record.
	bool restore(const std::string &blob) {
		size_t pos = 0;
		auto get32 = [&](int *v) {
			if (pos + 4 > blob.size()) return false;
			uint32_t u = 0;
			for (int k = 0; k < 4; ++k) u = (u << 8) | (unsigned char) blob[pos + k];
			pos += 4;
			*v = (int) u;
			return true;
		};
		auto getf = [&](float *p, int n) {
			for (int k = 0; k < n; ++k) {
				int v;
				if (!get32(&v)) return false;
				memcpy(p + k, &v, 4);
			}
			return true;
		};
		int magic;
		if (!get32(&magic) || (uint32_t) magic != 0xABCDE0EEu) return false;
		int kind;
		while (get32(&kind)) {
			int uid, in_len, out_size, nprev;
			if (!get32(&uid) || !get32(&in_len) || !get32(&out_size) || !get32(&nprev)) return false;
			std::vector<int> prev(nprev);
			for (int q = 0; q < nprev; ++q)
				if (!get32(&prev[q])) return false;
			int p0 = 0, p1 = 0, p2 = 0;
			switch (kind) {  // constructor arguments as the Restore* members choose them (impl/model_saver.h:557-800)
			case kInput: case kFourier: case kTriangFourier: case kCrossEntropy: case kL2Out: case kSoftMax: p0 = in_len; break;
			case kCrelu: case kGelu: case kHadamard: case kResidual: p0 = out_size; break;
			case kEmbedding:
				if (!get32(&p0) || !get32(&p1) || !get32(&p2)) return false;
				break;
			case kLinear: break;
			default: return false;
			}
			if (kind == kLinear && (!get32(&p0) || !get32(&p1))) return false;
			if (kind == kInput || kind == kEmbedding) {
				int got = add(kind, p0, p1, p2, prev.data(), nprev, uid);
				if (got != uid) return false;
				Node *nd = at(uid);
				if (!getf(nd->in.re, nd->in.n) || !getf(nd->in.im, nd->in.n)) return false;
			} else if (add(kind, p0, p1, p2, prev.data(), nprev, uid) != uid) {
				return false;
			}
		}
		return true;
	}
	float loss(int uid, int label) {
		Node *nd = at(uid);
		if (nd->kind == kCrossEntropy) return crossent_loss(nd->out.re, nd->out.im, label);
		return nd->out.re[0];
	}
	int prediction(int uid) {
		Node *nd = at(uid);
		return crossent_prediction(nd->p0, nd->out.re, nd->out.im);
	}
};

}  // namespace orc

#endif  // CNET_ORACLE_HPP_
