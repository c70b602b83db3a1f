// C entry points of the CPU oracle (test infrastructure; see cnet_oracle.hpp).
// Two groups:
//   cno_net_*  : a per-sample graph with the step semantics of the upstream ComplexNet.
//                oracle/ref_shim.cpp exports the same group on top of the upstream classes,
//                so one Python binding drives both and compares them.
//   cno_<layer>_{fwd,bwd} : batch loops over independent samples (one upstream "clone"
//                per row), used for GPU parity at medium sizes and as the timed CPU port.
#include "cnet_oracle.hpp"

#ifdef _OPENMP
#include <omp.h>
#endif

using namespace orc;

namespace {
inline GradIn gin(const float *const *g, size_t off) {
	GradIn r;
	r.dz_re = g[0] + off;
	r.dz_im = g[1] + off;
	r.dzs_re = g[2] + off;
	r.dzs_im = g[3] + off;
	return r;
}
inline GradOut gout(float *const *g, size_t off) {
	GradOut r;
	r.dz_re = g[0] + off;
	r.dz_im = g[1] + off;
	r.dzs_re = g[2] + off;
	r.dzs_im = g[3] + off;
	return r;
}
inline void zero4(float *const *g, size_t n) {
	for (int p = 0; p < 4; ++p) std::fill(g[p], g[p] + n, 0.0f);
}
}  // namespace

extern "C" {

const char *cno_backend() { return "port"; }

int cno_threads() {
#ifdef _OPENMP
	return omp_get_max_threads();
#else
	return 1;
#endif
}

// ---------------------------------------------------------------- graph API
void *cno_net_new() { return new Net(); }
void cno_net_free(void *h) { delete (Net *) h; }

int cno_net_add(void *h, int kind, int p0, int p1, int p2, const int *in_uids, int n_in) {
	return ((Net *) h)->add(kind, p0, p1, p2, in_uids, n_in);
}

int cno_net_len(void *h, int uid) {
	Node *nd = ((Net *) h)->at(uid);
	return nd ? nd->in.n : -1;
}

// plane 0..5: re, im, dz_re, dz_im, dzs_re, dzs_im of the node's input block;
// plane 6, 7: re, im of the output block of CrossEntropy (normalised z) / L2Out (loss).
float *cno_net_plane(void *h, int uid, int plane) {
	Node *nd = ((Net *) h)->at(uid);
	if (!nd) return NULL;
	if (plane >= 0 && plane < 6) return nd->in.re + (size_t) plane * nd->in.n;
	if (plane == 6) return nd->out.re;
	if (plane == 7) return nd->out.im;
	return NULL;
}

void cno_net_set_tokens(void *h, int uid, const int *tok, int count) {
	Node *nd = ((Net *) h)->at(uid);
	nd->tokens.assign(tok, tok + count);
}

void cno_net_forward(void *h) { ((Net *) h)->forward(); }
void cno_net_backward(void *h, int label) { ((Net *) h)->backward(label); }
void cno_net_update(void *h, float lr, int batch) { ((Net *) h)->update(lr, batch); }
// .mod stream: returns the stream length; copies it when it fits into cap bytes
long cno_net_save(void *h, char *buf, long cap) {
	std::string blob = ((Net *) h)->save();
	if ((long) blob.size() <= cap) memcpy(buf, blob.data(), blob.size());
	return (long) blob.size();
}
int cno_net_restore(void *h, const char *buf, long len) { return ((Net *) h)->restore(std::string(buf, (size_t) len)) ? 1 : 0; }
int cno_net_count(void *h) { return (int) ((Net *) h)->nodes().size(); }
int cno_net_uid_at(void *h, int index) { return ((Net *) h)->nodes()[index]->uid; }
int cno_net_kind(void *h, int uid) { return ((Net *) h)->at(uid)->kind; }
void cno_net_adam_update(void *h, float lr, int batch, float beta, int t) { ((Net *) h)->adam_update_inputs(lr, batch, beta, t); }
float cno_net_loss(void *h, int uid, int label) { return ((Net *) h)->loss(uid, label); }
int cno_net_prediction(void *h, int uid) { return ((Net *) h)->prediction(uid); }
void cno_node_forward(void *h, int uid) { ((Net *) h)->node_forward(((Net *) h)->at(uid)); }
void cno_node_backward(void *h, int uid, int label) { ((Net *) h)->node_backward(((Net *) h)->at(uid), label); }
void cno_node_zero_gradients(void *h, int uid) { ((Net *) h)->at(uid)->in.zero_gradients(); }

// ---------------------------------------------------------------- generators
void cno_fill_normal(uint64_t seed, long n, double mu, double sig, float *out) {
	Rng r(seed);
	for (long k = 0; k < n; ++k) out[k] = (float) r.normal(mu, sig);
}
void cno_fill_uniform(uint64_t seed, long n, double lo, double hi, float *out) {
	Rng r(seed);
	for (long k = 0; k < n; ++k) out[k] = (float) (lo + (hi - lo) * r.uniform());
}
void cno_fill_int(uint64_t seed, long n, int range, int *out) {
	Rng r(seed);
	for (long k = 0; k < n; ++k) out[k] = (int) (r.next() % (uint64_t) range);
}

// ---------------------------------------------------------------- batch layer loops
// x[B][K], w[N][K] (shared), y[B][N]
void cno_linear_fwd(int B, int K, int N, const float *xr, const float *xi, const float *wr, const float *wi,
		float *yr, float *yi) {
	for (int b = 0; b < B; ++b)
		linear_forward(K, N, xr + (size_t) b * K, xi + (size_t) b * K, wr, wi, yr + (size_t) b * N, yi + (size_t) b * N);
}

// g: 4 planes [B][N]; dx: 4 planes [B][K] (overwritten); dw: 4 planes [N][K] = per-sample
// gradients summed in row order b = 0..B-1 (the order in which the upstream parameter
// node accumulates samples between two updates, impl/cinput.h:54-65).
void cno_linear_bwd(int B, int K, int N, const float *xr, const float *xi, const float *wr, const float *wi,
		const float *const *g, float *const *dx, float *const *dw) {
	zero4(dx, (size_t) B * K);
	zero4(dw, (size_t) N * K);
	std::vector<float> tmp((size_t) 4 * N * K);
	float *t4[4] = {tmp.data(), tmp.data() + (size_t) N * K, tmp.data() + (size_t) 2 * N * K,
			tmp.data() + (size_t) 3 * N * K};
	for (int b = 0; b < B; ++b) {
		std::fill(tmp.begin(), tmp.end(), 0.0f);
		linear_backward(K, N, xr + (size_t) b * K, xi + (size_t) b * K, wr, wi, gin(g, (size_t) b * N),
				gout(dx, (size_t) b * K), gout(t4, 0));
		for (int p = 0; p < 4; ++p) {
			float *dst = dw[p];
			const float *src = t4[p];
#pragma omp parallel for
			for (long k = 0; k < (long) N * K; ++k) dst[k] += src[k];
		}
	}
}

void cno_dft_fwd(int B, int n, const float *xr, const float *xi, float *yr, float *yi) {
#pragma omp parallel for
	for (int b = 0; b < B; ++b)
		dft_forward(n, xr + (size_t) b * n, xi + (size_t) b * n, yr + (size_t) b * n, yi + (size_t) b * n);
}

void cno_dft_bwd(int B, int n, const float *const *g, float *const *dx) {
	zero4(dx, (size_t) B * n);
	std::vector<cf> roots = unity_roots(n);
	for (int b = 0; b < B; ++b) dft_backward(n, roots, gin(g, (size_t) b * n), gout(dx, (size_t) b * n));
}

// v_shared != 0: v is one parameter vector [n] used by every row and dv is the row-ordered
// sum of per-row gradients; otherwise v and dv are [B][n].
void cno_hadamard_fwd(int B, int n, const float *ur, const float *ui, const float *vr, const float *vi,
		int v_shared, float *yr, float *yi) {
	for (int b = 0; b < B; ++b) {
		size_t o = (size_t) b * n, ov = v_shared ? 0 : o;
		hadamard_forward(n, ur + o, ui + o, vr + ov, vi + ov, yr + o, yi + o);
	}
}

void cno_hadamard_bwd(int B, int n, const float *ur, const float *ui, const float *vr, const float *vi,
		int v_shared, const float *const *g, float *const *du, float *const *dv) {
	zero4(du, (size_t) B * n);
	zero4(dv, v_shared ? (size_t) n : (size_t) B * n);
	std::vector<float> tmp((size_t) 4 * n);
	float *t4[4] = {tmp.data(), tmp.data() + n, tmp.data() + 2 * n, tmp.data() + 3 * n};
	for (int b = 0; b < B; ++b) {
		size_t o = (size_t) b * n, ov = v_shared ? 0 : o;
		if (v_shared) {
			std::fill(tmp.begin(), tmp.end(), 0.0f);
			hadamard_backward(n, ur + o, ui + o, vr, vi, gin(g, o), gout(du, o), gout(t4, 0));
			for (int p = 0; p < 4; ++p)
				for (int k = 0; k < n; ++k) dv[p][k] += t4[p][k];
		} else {
			hadamard_backward(n, ur + o, ui + o, vr + ov, vi + ov, gin(g, o), gout(du, o), gout(dv, o));
		}
	}
}

void cno_gelu_fwd(long total, const float *xr, const float *xi, float *yr, float *yi) {
	gelu_forward((int) total, xr, xi, yr, yi);
}

void cno_gelu_bwd(long total, const float *xr, const float *xi, const float *const *g, float *const *dx) {
	zero4(dx, (size_t) total);
	gelu_backward((int) total, xr, xi, gin(g, 0), gout(dx, 0));
}

void cno_crelu_fwd(long total, const float *xr, const float *xi, float *yr, float *yi) {
	crelu_forward((int) total, xr, xi, yr, yi);
}

void cno_crelu_bwd(long total, const float *xr, const float *xi, const float *const *g, float *const *dx) {
	zero4(dx, (size_t) total);
	crelu_backward((int) total, xr, xi, gin(g, 0), gout(dx, 0));
}

void cno_triang_fwd(int B, int n, const float *xr, const float *xi, float *yr, float *yi) {
	std::vector<cf> roots = unity_roots(n);
#pragma omp parallel for
	for (int b = 0; b < B; ++b)
		triang_forward(n, roots, xr + (size_t) b * n, xi + (size_t) b * n, yr + (size_t) b * n, yi + (size_t) b * n);
}

void cno_triang_bwd(int B, int n, const float *const *g, float *const *dx) {
	zero4(dx, (size_t) B * n);
	std::vector<cf> roots = unity_roots(n);
#pragma omp parallel for
	for (int b = 0; b < B; ++b) triang_backward(n, roots, gin(g, (size_t) b * n), gout(dx, (size_t) b * n));
}

void cno_residual_fwd(long total, const float *ur, const float *ui, const float *vr, const float *vi, float *yr,
		float *yi) {
	residual_forward((int) total, ur, ui, vr, vi, yr, yi);
}

void cno_residual_bwd(long total, const float *const *g, float *const *du, float *const *dv) {
	zero4(du, (size_t) total);
	zero4(dv, (size_t) total);
	residual_backward((int) total, gin(g, 0), gout(du, 0), gout(dv, 0));
}

void cno_softmax_fwd(int B, int n, const float *zr, const float *zi, float *yr, float *yi, float *S) {
	for (int b = 0; b < B; ++b) {
		size_t o = (size_t) b * n;
		SoftMaxState st = softmax_forward(n, zr + o, zi + o, yr + o, yi + o);
		if (S) S[b] = st.square_norm;
	}
}

void cno_softmax_bwd(int B, int n, const float *zr, const float *zi, const float *const *g, float *const *dz) {
	zero4(dz, (size_t) B * n);
	for (int b = 0; b < B; ++b) {
		size_t o = (size_t) b * n;
		SoftMaxState st = softmax_forward(n, zr + o, zi + o, NULL, NULL);
		softmax_backward(n, st, zr + o, zi + o, gin(g, o), gout(dz, o));
	}
}

void cno_crossent_fwd(int B, int n, const float *zr, const float *zi, const int *labels, float *outr, float *outi,
		float *S, float *loss, int *pred) {
	for (int b = 0; b < B; ++b) {
		size_t o = (size_t) b * n;
		S[b] = crossent_forward(n, zr + o, zi + o, outr + o, outi + o);
		loss[b] = crossent_loss(outr + o, outi + o, labels[b]);
		pred[b] = crossent_prediction(n, outr + o, outi + o);
	}
}

void cno_crossent_bwd(int B, int n, const float *zr, const float *zi, const int *labels, float *const *dz) {
	std::vector<float> tr(n), ti(n);
	for (int b = 0; b < B; ++b) {
		size_t o = (size_t) b * n;
		float S = crossent_forward(n, zr + o, zi + o, tr.data(), ti.data());
		crossent_backward(n, zr + o, zi + o, S, labels[b], gout(dz, o));
	}
}

void cno_l2out_fwd(int B, int n, const float *zr, const float *zi, float *loss) {
	for (int b = 0; b < B; ++b) loss[b] = l2out_forward(n, zr + (size_t) b * n, zi + (size_t) b * n);
}

void cno_l2out_bwd(int B, int n, const float *zr, const float *zi, float *const *dz) {
	zero4(dz, (size_t) B * n);
	l2out_backward((int) ((long) B * n), zr, zi, gout(dz, 0));
}

// tokens[B][T] with -1 padding at the tail of a row (impl/batch.h:82-86)
void cno_embedding_fwd(int B, int T, int D, const float *tr, const float *ti, const int *tokens, float *yr,
		float *yi) {
	for (int b = 0; b < B; ++b) {
		const int *row = tokens + (size_t) b * T;
		int count = 0;
		while (count < T && row[count] >= 0) ++count;
		embedding_forward(D, T, tr, ti, row, count, yr + (size_t) b * T * D, yi + (size_t) b * T * D);
	}
}

void cno_embedding_bwd(int B, int T, int D, int V, const int *tokens, const float *gsr, const float *gsi,
		float *dsr, float *dsi) {
	std::fill(dsr, dsr + (size_t) V * D, 0.0f);
	std::fill(dsi, dsi + (size_t) V * D, 0.0f);
	for (int b = 0; b < B; ++b) {
		const int *row = tokens + (size_t) b * T;
		int count = 0;
		while (count < T && row[count] >= 0) ++count;
		embedding_backward(D, row, count, gsr + (size_t) b * T * D, gsi + (size_t) b * T * D, dsr, dsi);
	}
}

void cno_sgd_update(long n, float *zr, float *zi, const float *dsr, const float *dsi, float lr) {
	sgd_update((int) n, zr, zi, dsr, dsi, lr);
}

void cno_adam_update(long n, float *zr, float *zi, float *mr, float *mi, const float *dsr, const float *dsi, float lr,
		float beta, int t) {
	adam_update((int) n, zr, zi, mr, mi, dsr, dsi, lr, beta, t);
}

// Dense matrix of the CPU forward transform: column q = forward(unit vector e_q).
// F[p][q], row-major, so that y = F x reproduces dft_forward on any x up to summation order.
void cno_dft_matrix(int n, float *fr, float *fi) {
	std::vector<float> er(n), ei(n), yr(n), yi(n);
	for (int q = 0; q < n; ++q) {
		std::fill(er.begin(), er.end(), 0.0f);
		std::fill(ei.begin(), ei.end(), 0.0f);
		er[q] = 1.0f;
		dft_forward(n, er.data(), ei.data(), yr.data(), yi.data());
		for (int p = 0; p < n; ++p) {
			fr[(size_t) p * n + q] = yr[p];
			fi[(size_t) p * n + q] = yi[p];
		}
	}
}

}  // extern "C"
