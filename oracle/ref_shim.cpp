// Thin C wrapper that drives the UPSTREAM CNet CPU classes, compiled from the upstream
// sources where they lie (include path given by the Makefile; nothing is copied into this
// repository).  It exports the same cno_net_* entry points as oracle_capi.cpp so the
// restatement can be compared with the real thing, call by call.
//
// TEST INFRASTRUCTURE ONLY: built into oracle/_ref/, never linked by the product.
#include <cstring>
#include <climits>
#include <cassert>

#include "impl/cnet.h"
#include "impl/batch.h"
#include "impl/model_saver.h"

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

struct RefNet {
	ComplexNet net;
	std::map<int, int> kind_of;
};

Vars *out_block(CFunc *f) {
	if (OutputFunc *o = dynamic_cast<OutputFunc *>(f)) return o->mutableOutput();
	return NULL;
}

}  // namespace

extern "C" {

const char *cno_backend() { return "reference"; }

int cno_threads() {
#ifdef _OPENMP
	return omp_get_max_threads();
#else
	return 1;
#endif
}

void *cno_net_new() { return new RefNet(); }
void cno_net_free(void *h) { delete (RefNet *) h; }

int cno_net_add(void *h, int kind, int p0, int p1, int p2, const int *in_uids, int n_in) {
	RefNet *r = (RefNet *) h;
	CFunc *f = NULL;
	switch (kind) {
	case isInput: f = new CInput(OutSize(p0)); break;
	case isLinear: f = new Linear(InSize(p0), InSize(p1)); break;
	case isFourier: f = new FourierTrans(InSize(p0)); break;
	case isHadamard: f = new Hadamard(InSize(p0), InSize(p0)); break;
	case isGelu: f = new CGelu(InSize(p0)); break;
	case isCrelu: f = new CRelu(InSize(p0)); break;
	case isTrianFourier: f = new TriangFourier(InSize(p0)); break;
	case isResidual: f = new Residual(InSize(p0)); break;
	case isSoftMax: f = new SoftMax(InSize(p0)); break;
	case isCrossEntropy: f = new CrossEntropy(InSize(p0)); break;
	case isL2Out: f = new L2Out(InSize(p0)); break;
	case isEmbedding: f = new CEmbedding(p0, p1, p2); break;
	default: return -1;
	}
	std::vector<int> ins(in_uids, in_uids + n_in);
	int uid = r->net.add(f, ins);
	r->kind_of[uid] = kind;
	return uid;
}

int cno_net_len(void *h, int uid) {
	CFunc *f = ((RefNet *) h)->net[uid];
	return f ? f->input().length_ : -1;
}

float *cno_net_plane(void *h, int uid, int plane) {
	CFunc *f = ((RefNet *) h)->net[uid];
	if (!f) return NULL;
	if (plane >= 0 && plane < 6) return f->mutable_input()->real_ + (size_t) plane * f->input().length_;
	Vars *o = out_block(f);
	if (!o) return NULL;
	return plane == 6 ? o->real_ : (plane == 7 ? o->imag_ : NULL);
}

void cno_net_set_tokens(void *h, int uid, const int *tok, int count) {
	CEmbedding *e = dynamic_cast<CEmbedding *>(((RefNet *) h)->net[uid]);
	assert(e);
	e->setInput(std::vector<int>(tok, tok + count));
}

void cno_net_forward(void *h) { ((RefNet *) h)->net.forward(); }

void cno_net_backward(void *h, int label) {
	if (label >= 0)
		((RefNet *) h)->net.backward(label);
	else
		((RefNet *) h)->net.backward();
}

void cno_net_update(void *h, float lr, int batch) { ((RefNet *) h)->net.update(lr, batch); }

long cno_net_save(void *h, char *buf, long cap) {
	ModelSaver saver;
	std::string blob = saver.SaveToString(((RefNet *) h)->net);
	if ((long) blob.size() <= cap) memcpy(buf, blob.data(), blob.size());
	return (long) blob.size();
}
int cno_net_restore(void *h, const char *buf, long len) {
	ModelSaver saver;
	RefNet *r = (RefNet *) h;
	if (!saver.RestoreFromString(r->net, std::string(buf, (size_t) len))) return 0;
	for (auto f : r->net.functionList()) r->kind_of[f->uid()] = f->getType();
	return 1;
}
int cno_net_count(void *h) { return (int) ((RefNet *) h)->net.functionList().size(); }
int cno_net_uid_at(void *h, int index) { return ((RefNet *) h)->net.functionList()[index]->uid(); }
int cno_net_kind(void *h, int uid) { return ((RefNet *) h)->net[uid]->getType(); }
void cno_net_adam_update(void *h, float lr, int batch, float beta, int t) { ((RefNet *) h)->net.adamUpdate(lr, batch, beta, t); }

float cno_net_loss(void *h, int uid, int label) {
	OutputFunc *o = dynamic_cast<OutputFunc *>(((RefNet *) h)->net[uid]);
	assert(o);
	return o->loss(label);
}

int cno_net_prediction(void *h, int uid) {
	CrossEntropy *c = dynamic_cast<CrossEntropy *>(((RefNet *) h)->net[uid]);
	assert(c);
	return c->get_prediction();
}

void cno_node_forward(void *h, int uid) { ((RefNet *) h)->net[uid]->forward(); }

void cno_node_backward(void *h, int uid, int label) {
	CFunc *f = ((RefNet *) h)->net[uid];
	if (label >= 0 && dynamic_cast<CrossEntropy *>(f))
		f->backward(label);
	else
		f->backward();
}

void cno_node_zero_gradients(void *h, int uid) { ((RefNet *) h)->net[uid]->mutable_input()->zero_gradients(); }

// Generators from the upstream SimpleRand, for checking the restated xorshift/polar pair.
void cno_fill_normal(uint64_t seed, long n, double mu, double sig, float *out) {
	SimpleRand r(seed);
	for (long k = 0; k < n; ++k) out[k] = (float) r.normal(mu, sig);
}
void cno_fill_uniform(uint64_t seed, long n, double lo, double hi, float *out) {
	SimpleRand r(seed);
	for (long k = 0; k < n; ++k) out[k] = (float) (lo + (hi - lo) * r.randDouble());
}

}  // extern "C"
