// Timing driver for training loops through the C++ host facade (cnet_amd/host/cnet.hpp) on the device library: what
// bench.py runs for the "train samples/sec" half of the metric.  Synthetic, seeded data from its own generator; no
// comparison with anything (the parity tests do that), one JSON line per run on stdout.
//
//   train_bench readme B steps [graphs] [both_halves] [frozen_input] [complex_samples] [on_device]
//       FourierTrans(784) -> Hadamard -> CGelu -> Linear 784 -> 10 -> CrossEntropy, SGD, batches from a
//       BatchedDataReader; the loop of upstream cnet.cpp:119-150 in several input / read-back modes.
//   train_bench stack n blocks B steps lr [both_halves]
//       blocks x (Linear n -> n, CGelu, Residual), L2Out against targets, SGD (the residual stack workload).
//   train_bench token batch seq dim hidden vocab steps lr [both_halves]
//       the complex token model, one token per sample: CEmbedding -> SeqFourierTrans -> Hadamard gate -> Linear, CGelu,
//       Linear -> Linear to the vocabulary -> CrossEntropy on the next token, SGD.
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "cnet_amd/host/cnet.hpp"
#include "cnet_amd/host/data.hpp"

namespace {

// xorshift64* with Box-Muller normals: the same values on every host
struct Gen {
	uint64_t s;
	explicit Gen(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 0x1234567ull) {
		for (int k = 0; k < 4; ++k) next();
	}
	uint64_t next() {
		s ^= s >> 12;
		s ^= s << 25;
		s ^= s >> 27;
		return s * 0x2545F4914F6CDD1Dull;
	}
	double uniform() { return (double) (next() >> 11) * (1.0 / 9007199254740992.0); }
	double normal() {
		const double u = std::max(uniform(), 1e-300), v = uniform();
		return std::sqrt(-2.0 * std::log(u)) * std::cos(6.283185307179586 * v);
	}
	void fill_normal(float *p, size_t n, double sig) {
		for (size_t k = 0; k < n; ++k) p[k] = (float) (sig * normal());
	}
};

void build_readme(CNet &net, int n, int classes, int *inp, int *outp) {
	*inp = net.add(new CInput(OutSize(n)));
	auto fft = net.add(new FourierTrans(InSize(n)), {*inp});
	auto h_data = net.add(new CInput(OutSize(n)));
	auto hdm = net.add(new Hadamard(InSize(n), InSize(n)), {fft, h_data});
	auto gelu = net.add(new CGelu(InSize(n)), {hdm});
	auto l_data = net.add(new CInput(OutSize(n * classes)));
	auto lin = net.add(new Linear(InSize(n), InSize(n * classes)), {gelu, l_data});
	*outp = net.add(new CrossEntropy(InSize(classes)), {lin});
	net.init_inputs(11);
}

struct SyntheticReader : public BatchedDataReader {
	SyntheticReader(int dim, int count, int classes, bool complex_samples) : BatchedDataReader(dim) {
		Gen rng(123);
		std::vector<float> re(dim), im(dim);
		reserve(count);
		for (int s = 0; s < count; ++s) {
			for (int k = 0; k < dim; ++k) {
				re[k] = (float) rng.uniform();  // real parts uniform in [0, 1], imaginary parts 0: image-like samples
				im[k] = complex_samples ? (float) rng.uniform() : 0.f;
			}
			addPlanes(re.data(), im.data(), (int) (rng.next() % classes));
		}
	}
	bool readData() override { return true; }
};

// A device that has just been handed over, or has sat idle while the host built a net, runs its first ~30 ms of work at
// lower clocks.  Before a timed loop the forward pass is queued over and over for 40 ms (it changes nothing that the loop
// reads: activations and the loss of a batch that is fed again or replaced), so the loop measures the sustained rate.
template <class Forward>
void wake_device(CNet &net, Forward forward) {
	const auto t0 = std::chrono::steady_clock::now();
	while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < 0.04) {
		for (int k = 0; k < 4; ++k) forward();
		net.sync();
	}
}

bool has(int argc, char **argv, int from, const char *word) {
	for (int k = from; k < argc; ++k)
		if (std::string(argv[k]) == word) return true;
	return false;
}

// Modes of the README-net loop:
//   0 the batch is copied inside gpuForward            1 batches staged ahead with gpuPrefetch, loss read every step
//   2 as 1, phases replayed from recorded graphs       3 as 0 with recorded graphs
//   4 as 1 with gpuTrainStep (one recorded graph)      5 as 1 with both halves of every gradient pair computed
//   6 as 1, the loss of a step read one step later     7 as 6 with gpuTrainStep
//   8 as 6 with the data input marked not trainable     9 as 6 with the reader's samples stored on the device
int run_readme(int B, int steps, bool with_graphs, bool both_halves, bool frozen_input, bool complex_samples, bool on_device) {
	const int n = 784, classes = 10;
	const float lr = 0.01f;
	if (cnet_init(0) != CNET_OK) {
		fprintf(stderr, "train_bench: cnet_init failed: %s\n", cnet_last_error());
		return 2;
	}
	SyntheticReader data(n, 3 * B + 7, classes, complex_samples);
	constexpr int MODES = 10;
	double ms[MODES] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
	float last_loss[MODES] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
	for (int mode = 0; mode < MODES; ++mode) {
		if (!with_graphs && ((mode >= 2 && mode <= 4) || mode == 7)) continue;
		if (mode == 5 && !both_halves) continue;
		if (mode == 8 && !frozen_input) continue;
		if (mode == 9 && !on_device) continue;
		const bool prefetch = mode == 1 || mode == 2 || mode >= 4, graphs = mode == 2 || mode == 3, one_graph = mode == 4 || mode == 7;
		const bool late_loss = mode == 6 || mode == 7 || mode == 8 || mode == 9;
		CNet::PendingLoss pending;
		CNet net;
		int inp, outp;
		build_readme(net, n, classes, &inp, &outp);
		net.allocateOnGpu(B);
		CInput *cin = (CInput *) net[inp];
		CrossEntropy *cen = (CrossEntropy *) net[outp];
		SyntheticReader reader = data;
		if (mode == 9) reader.storeOnDevice();  // before the clock starts: the samples are in device memory when the loop begins
		InputBatch ring[3] = {InputBatch(B, n), InputBatch(B, n), InputBatch(B, n)};
		if (graphs) net.useGraphs(true);
		if (mode == 5) net.conjugateGradients(false);
		if (mode == 8) net.setInputTrainable(cin, false);
		{
			SyntheticReader other = data;  // a batch of its own: the timed loop reads the same samples with or without this
			InputBatch wb(B, n);
			other.nextBatch(wb);
			wake_device(net, [&] { net.gpuForward(cin, cen, wb); });
		}
		net.sync();
		auto t0 = std::chrono::steady_clock::now();
		if (prefetch) {
			reader.nextBatch(ring[0]);
			net.gpuPrefetch(cin, ring[0]);
			if (steps > 1) reader.nextBatch(ring[1]);
		}
		float loss = 0.f;
		for (int s = 0; s < steps; ++s) {
			InputBatch &cur = ring[s % 3];
			if (!prefetch) reader.nextBatch(cur);
			const float rate = (s < steps / 2 ? lr : 0.5f * lr) / B;
			// The next batch is sent off as soon as the forward pass of this one is queued (which is what frees the other
			// buffer of the data input): its copy then has the whole step to arrive in.  Queued after the update instead,
			// the copy's own latency shows whenever the host is barely ahead of the device (batch 64: 75 against 60 us per step).
			const bool more = prefetch && s + 1 < steps;
			if (one_graph) {
				net.gpuTrainStep(cin, cen, cur, rate);
				if (more) net.gpuPrefetch(cin, ring[(s + 1) % 3]);
			} else {
				net.gpuForward(cin, cen, cur);
				if (more) net.gpuPrefetch(cin, ring[(s + 1) % 3]);
				net.gpuBackward();
				net.gpuUpdateInputs(rate);
			}
			if (late_loss) {
				CNet::PendingLoss now = net.gpuQueueLoss(cen);
				if (s > 0) loss = net.getLoss(pending, &ring[(s + 2) % 3]);
				if (s + 2 < steps) reader.nextBatch(ring[(s + 2) % 3]);
				pending = now;
				continue;
			}
			if (prefetch && s + 2 < steps) reader.nextBatch(ring[(s + 2) % 3]);
			loss = net.getLoss(cen, &cur);
		}
		if (late_loss) loss = net.getLoss(pending, NULL);
		net.sync();
		ms[mode] = 1e3 * std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / steps;
		last_loss[mode] = loss;
	}
	auto rate = [&](int m) { return ms[m] > 0 ? B / ms[m] * 1e3 : 0.0; };
	printf("{\"workload\": \"README net 784 -> 10, SGD, batches from a BatchedDataReader\", \"batch\": %d, \"steps\": %d, "
		   "\"ms_per_step_copy_in_forward\": %.3f, \"ms_per_step_prefetch\": %.3f, \"ms_per_step_prefetch_graphs\": %.3f, "
		   "\"ms_per_step_graphs\": %.3f, \"samples_per_sec_copy_in_forward\": %.1f, \"samples_per_sec_prefetch\": %.1f, "
		   "\"samples_per_sec_prefetch_graphs\": %.1f, \"ms_per_step_train_step_graph\": %.3f, \"samples_per_sec_train_step_graph\": %.1f, "
		   "\"ms_per_step_prefetch_two_products_per_gradient_pair\": %.3f, \"ms_per_step_prefetch_loss_read_one_step_late\": %.3f, "
		   "\"samples_per_sec_prefetch_loss_read_one_step_late\": %.1f, \"ms_per_step_train_step_graph_loss_read_one_step_late\": %.3f, "
		   "\"ms_per_step_data_input_not_trainable\": %.3f, \"samples_per_sec_data_input_not_trainable\": %.1f, "
		   "\"ms_per_step_samples_stored_on_device\": %.3f, \"samples_per_sec_samples_stored_on_device\": %.1f, "
		   "\"last_loss\": %.5f, \"last_loss_samples_stored_on_device\": %.5f, \"samples\": \"%s\", \"upload_bytes_per_step\": %zu}\n",
			B, steps, ms[0], ms[1], ms[2], ms[3], rate(0), rate(1), rate(2), ms[4], rate(4), ms[5], ms[6], rate(6), ms[7], ms[8], rate(8),
			ms[9], rate(9), last_loss[6], last_loss[9], complex_samples ? "complex: real and imaginary parts uniform in [0, 1]" : "real parts uniform in [0, 1], imaginary parts 0 (the imaginary plane is cleared on the device, not sent)",
			(size_t) (complex_samples ? 2 : 1) * B * n * sizeof(float));
	return std::isfinite(last_loss[6]) ? 0 : 1;
}

int run_stack(int n, int blocks, int B, int steps, float lr, bool both_halves) {
	Gen rng(4);
	CNet net;
	std::vector<int> w;
	int x = net.add(new CInput(OutSize(n))), cur = x;
	for (int b = 0; b < blocks; ++b) {
		int wb = net.add(new CInput(OutSize(n * n)));
		w.push_back(wb);
		int lin = net.add(new Linear(InSize(n), InSize(n * n)), {cur, wb});
		int ge = net.add(new CGelu(InSize(n)), {lin});
		cur = net.add(new Residual(InSize(n)), {cur, ge});
	}
	CInput *tin = new CInput(OutSize(n));
	tin->setIsBatched(true);  // the (negated) L2 target: a second per-sample data input
	int t = net.add(tin);
	int diff = net.add(new Residual(InSize(n)), {cur, t});
	int l2i = net.add(new L2Out(InSize(n)), {diff});
	if (both_halves) net.conjugateGradients(false);  // dz* products computed as upstream does, not written as conjugates
	for (int b = 0; b < blocks; ++b) rng.fill_normal(net[w[b]]->mutable_input()->real_, (size_t) 2 * n * n, 1.0 / std::sqrt((double) n));
	net.allocateOnGpu(B);
	std::vector<float> xs((size_t) 2 * B * n), ts((size_t) 2 * B * n);
	rng.fill_normal(xs.data(), xs.size(), 1.0);
	rng.fill_normal(ts.data(), ts.size(), 1.0);
	InputBatch bx(B, n), bt(B, n);
	for (int b = 0; b < B; ++b) {
		bx.add(xs.data() + (size_t) b * n, xs.data() + (size_t) (B + b) * n, n, 0);
		bt.add(ts.data() + (size_t) b * n, ts.data() + (size_t) (B + b) * n, n, 0);
	}
	CInput *cx = (CInput *) net[x], *ct = (CInput *) net[t];
	L2Out *l2 = (L2Out *) net[l2i];
	std::vector<float> losses;
	// Both data inputs are sent again every step: the update also steps them (impl/cnet.h:413-421 upstream).  The batch of
	// the main input travels on the upload stream under the previous step; the targets are queued on the compute stream.
	// The host queues the whole step and reads the loss last.
	auto one = [&]() {
		net.gpuSetInput(ct, bt);
		net.gpuForward(cx, l2, bx);
		net.gpuBackward();
		net.gpuUpdateInputs(lr / B);  // upstream GPU loop: l_rate / batch.size() (cnet.cpp:147 upstream)
		net.gpuPrefetch(cx, bx);
		losses.push_back(net.getLoss(l2, NULL));
	};
	// timed region = the `steps` training steps from the initial weights (the first call also pays the one-off
	// workspace growth of the backward pass; it is part of the job)
	net.gpuSetInput(ct, bt);
	// (the warm-up sends its batch ahead as the loop does, so that every device buffer of the data input has been the target
	// of a copy before the clock starts: the first copy into a buffer while kernels run stalls host and device for 7 ms, once
	// per buffer, which a loop of 10 steps would carry as 6 % of its time)
	wake_device(net, [&] {
		net.gpuPrefetch(cx, bx);
		net.gpuForward(cx, l2, bx);
	});
	net.sync();
	auto t0 = std::chrono::steady_clock::now();
	net.gpuPrefetch(cx, bx);
	auto t1 = t0;
	std::string each;  // every step ends with its loss on the host, so the host's clock sees the steps one by one
	auto last = t0;
	for (int s = 0; s < steps; ++s) {
		one();
		const auto now = std::chrono::steady_clock::now();
		if (s == 0) t1 = now;  // getLoss has waited for step 0
		char buf[32];
		snprintf(buf, sizeof(buf), "%s%.2f", s ? ", " : "", 1e3 * std::chrono::duration<double>(now - last).count());
		each += buf;
		last = now;
	}
	net.sync();
	const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
	const double sec_later = std::chrono::duration<double>(std::chrono::steady_clock::now() - t1).count();
	std::string all;
	for (float l : losses) {
		char buf[64];
		snprintf(buf, sizeof(buf), "%s%.6g", all.empty() ? "" : ", ", l);
		all += std::isfinite(l) ? buf : (all.empty() ? "null" : ", null");
	}
	// matrix products executed per Linear and step: forward, and per gradient pair one product (the other half written as
	// its conjugate) or two (both computed), for the input and for the weight
	const int products = both_halves ? 5 : 3;
	const double flops = 8.0 * products * B * (double) n * n * blocks;
	printf("{\"workload\": \"residual stack: %d x (Linear %d->%d, CGelu, Residual), L2Out, SGD\", \"batch\": %d, \"steps\": %d, "
		   "\"lr\": %g, \"ms_per_step\": %.3f, \"ms_per_step_after_the_first\": %.3f, \"samples_per_sec\": %.1f, "
		   "\"complex_products_per_linear\": %d, \"gemm_tflops_executed\": %.2f, \"ms_of_each_step\": [%s], \"mean_loss_per_step\": [%s]}\n",
			blocks, n, n, B, steps, (double) lr, 1e3 * sec / steps, steps > 1 ? 1e3 * sec_later / (steps - 1) : 0.0, B * steps / sec, products,
			flops * steps / sec / 1e12, each.c_str(), all.c_str());
	return 0;
}

// The complex token model with one token per sample: an EmbeddingBatch of batch x seq one-token samples, CEmbedding, the
// transform along the sequence (SeqFourierTrans), a Hadamard gate with shared weights, Linear dim -> hidden, CGelu, Linear
// hidden -> dim, Linear dim -> vocab, CrossEntropy on the next token (the last position of a sequence is labelled with its
// first token).  One step = upload of the tokens and labels, forward, backward, SGD on the table and every weight, and the
// read-back of the mean loss.
int run_token(int Bq, int S, int D, int H, int V, int steps, float lr, bool both_halves) {
	Gen rng(7);
	const int R = Bq * S;
	CNet net;
	int emb = net.add(new CEmbedding(D, 1, V));
	int mix = net.add(new SeqFourierTrans(InSize(D), S), {emb});
	int gd = net.add(new CInput(OutSize(D)));
	int had = net.add(new Hadamard(InSize(D), InSize(D)), {mix, gd});
	int w1 = net.add(new CInput(OutSize(H * D)));
	int l1 = net.add(new Linear(InSize(D), InSize(H * D)), {had, w1});
	int ge = net.add(new CGelu(InSize(H)), {l1});
	int w2 = net.add(new CInput(OutSize(D * H)));
	int l2 = net.add(new Linear(InSize(H), InSize(D * H)), {ge, w2});
	int w3 = net.add(new CInput(OutSize(V * D)));
	int l3 = net.add(new Linear(InSize(D), InSize(V * D)), {l2, w3});
	int ce = net.add(new CrossEntropy(InSize(V)), {l3});
	if (both_halves) net.conjugateGradients(false);
	rng.fill_normal(net[emb]->mutable_input()->real_, (size_t) 2 * V * D, 1.0);
	rng.fill_normal(net[gd]->mutable_input()->real_, (size_t) 2 * D, 0.05);
	rng.fill_normal(net[w1]->mutable_input()->real_, (size_t) 2 * H * D, 1.0 / std::sqrt((double) D));
	rng.fill_normal(net[w2]->mutable_input()->real_, (size_t) 2 * D * H, 1.0 / std::sqrt((double) H));
	rng.fill_normal(net[w3]->mutable_input()->real_, (size_t) 2 * V * D, 1.0 / std::sqrt((double) D));
	((CEmbedding *) net[emb])->setInput({0});
	net.allocateOnGpu(R);
	std::vector<int> ids(R);
	for (auto &t : ids) t = (int) (rng.next() % (uint64_t) V);
	EmbeddingBatch batch(R, 1);
	for (int r = 0; r < R; ++r) batch.add(std::vector<int>(1, ids[r]), ids[r / S * S + (r % S + 1) % S]);
	CEmbedding *e = (CEmbedding *) net[emb];
	CrossEntropy *c = (CrossEntropy *) net[ce];
	std::vector<float> losses;
	auto one = [&]() {
		net.gpuForward(e, c, batch);
		net.gpuBackward();
		net.gpuUpdateInputs(lr / R);
		losses.push_back(net.getLoss(c, NULL));
	};
	one();  // the first step pays the one-off growth of the library workspace and the twiddle planes
	net.sync();
	auto t0 = std::chrono::steady_clock::now();
	for (int s = 0; s < steps; ++s) one();
	net.sync();
	const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
	std::string all;
	for (float l : losses) {
		char buf[64];
		snprintf(buf, sizeof(buf), "%s%.6g", all.empty() ? "" : ", ", l);
		all += buf;
	}
	// complex products executed per step: each Linear forward + one (conjugate pairs) or two per gradient; the transform
	// forward + two backward
	const double lin = 8.0 * R * ((double) D * H + (double) H * D + (double) D * V), dft = 8.0 * Bq * (double) S * S * D;
	const double flops = (both_halves ? 5 : 3) * lin + 3 * dft;
	printf("{\"workload\": \"configs[4] through the C++ facade: complex token model, one token per sample, fwd + bwd + SGD\", "
		   "\"batch\": %d, \"seq\": %d, \"dim\": %d, \"hidden\": %d, \"vocab\": %d, \"steps\": %d, \"lr\": %g, "
		   "\"gradient_pairs\": \"%s\", \"ms_per_step\": %.3f, \"tokens_per_sec\": %.1f, \"gemm_tflops_executed\": %.2f, "
		   "\"mean_loss_per_step\": [%s], \"loss_of_uniform_guess\": %.4f}\n",
			Bq, S, D, H, V, steps, (double) lr, both_halves ? "both halves computed" : "dz* written as conj(dz)", 1e3 * sec / steps,
			R * steps / sec, flops * steps / sec / 1e12, all.c_str(), std::log((double) V));
	return std::isfinite(losses.back()) ? 0 : 1;
}

}  // namespace

int main(int argc, char **argv) {
	const std::string what = argc > 1 ? argv[1] : "";
	setvbuf(stdout, NULL, _IOLBF, 0);
	try {
		if (what == "readme")
			return run_readme(argc > 2 ? atoi(argv[2]) : 4096, argc > 3 ? atoi(argv[3]) : 30, has(argc, argv, 4, "graphs"),
					has(argc, argv, 4, "both_halves"), has(argc, argv, 4, "frozen_input"), has(argc, argv, 4, "complex_samples"), has(argc, argv, 4, "on_device"));
		if (what == "stack")
			return run_stack(argc > 2 ? atoi(argv[2]) : 2048, argc > 3 ? atoi(argv[3]) : 8, argc > 4 ? atoi(argv[4]) : 2048,
					argc > 5 ? atoi(argv[5]) : 10, argc > 6 ? (float) atof(argv[6]) : 0.01f, has(argc, argv, 7, "both_halves"));
		if (what == "token")
			return run_token(argc > 2 ? atoi(argv[2]) : 16, argc > 3 ? atoi(argv[3]) : 512, argc > 4 ? atoi(argv[4]) : 1024,
					argc > 5 ? atoi(argv[5]) : 4096, argc > 6 ? atoi(argv[6]) : 32768, argc > 7 ? atoi(argv[7]) : 5,
					argc > 8 ? (float) atof(argv[8]) : 0.05f, has(argc, argv, 9, "both_halves"));
	} catch (const std::exception &e) {
		fprintf(stderr, "train_bench: %s\n", e.what());
		return 2;
	}
	fprintf(stderr, "usage: train_bench readme B steps [graphs] [both_halves] [frozen_input] [complex_samples] [on_device] | stack n blocks B steps lr [both_halves] | token batch seq dim hidden vocab steps lr [both_halves]\n");
	return 64;
}
