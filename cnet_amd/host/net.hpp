// cnet_amd/host/net.hpp
// CNet (upstream gpu/gpu_func.h): owns the nodes, plans their device planes and the fused launches, and runs forward pass,
// backward pass and update as calls into the device library.  Included by cnet.hpp (after functions.hpp).
#ifndef CNET_AMD_HOST_NET_HPP_
#define CNET_AMD_HOST_NET_HPP_

// ---------------------------------------------------------------------------------------------------------------
// gpu/gpu_func.h: CNet
// ---------------------------------------------------------------------------------------------------------------
class CNet {
	std::vector<CFunc *> func_list_;  // owned
	std::map<int, CFunc *> map_;
	std::vector<CFunc *> inputs_, outputs_;
	int next_uid_ = 0;
	bool graph_ready_ = false;
	std::vector<std::vector<CFunc *>> func_at_depth_;  // filled by init_exec_graph()

	// device plan
	int batch_ = 0;                   // 0: nothing allocated
	std::vector<void *> allocations_;
	CFunc *main_input_ = NULL;
	int32_t *d_labels_ = NULL;
	std::vector<int> labels_;
	bool batch_labels_ = false;       // labels_ came with a batch (they then win over a label argument, as upstream)
	// Device buffers of the data input, used in turn: stage_[active_] is what the kernels read, the next one can be filled by
	// gpuPrefetch() meanwhile.  Three rather than two: the buffer about to be refilled was then last read two steps ago, and
	// the point of the compute stream at which it was retired has been reached by the time the upload stream is told to wait
	// for it (with two buffers that point is the end of the step that is still running when the next batch is sent off).
	static constexpr int kStages = 3;
	struct Stage {
		float *z = NULL;            // 2 planes [batch][len]
		int32_t *labels = NULL;     // [batch]
		int32_t *host_labels = NULL;  // page-locked staging of the labels
		int64_t labels_ticket = -1;   // the last copy out of host_labels
		const InputBatch *holds = NULL;
		bool imag_zero = false;       // the staged batch held real samples: its imaginary plane on the device is all +0
		// Every element of the imaginary plane of this buffer on the device is +0 (it was cleared and nothing has written to it
		// since): the next batch of real samples that lands here need not clear it again.
		bool imag_dev_zero = false;
		int64_t upload_ticket = -1;   // the point of the upload stream at which the staged batch and its labels have landed
		// The staged batch names samples on the device and is small: nothing was queued for it; its rows are copied on the
		// compute stream when it is fed (see gatherOnCompute).
		bool deferred = false;
	};
	// A batch whose samples are on the device and whose copy is a few microseconds of kernel (up to 1 MiB) skips the upload
	// stream: the hand-over between the streams (two waits and two recorded points per step) costs the host more than the
	// copy costs the device in front of the forward pass.
	bool gatherOnCompute(const InputBatch &batch, size_t plane_bytes) const { return batch.resident_ && 2 * plane_bytes <= ((size_t) 1 << 20); }
	Stage stage_[kStages];
	int active_ = 0;
	int nextStage() const { return (active_ + 1) % kStages; }
	// recorded phases of a step, one set per buffer of the data input (device pointers are frozen into a recording)
	struct StepGraphs {
		void *fwd = NULL, *bwd = NULL, *upd = NULL;
		float upd_lr = 0.f;
		bool fwd_real = false, step_real = false;  // the forward pass in the recording took the transform of real samples
		void *step = NULL;      // forward + backward + update in one recording (gpuTrainStep)
		float step_lr = 0.f;
		bool step_warm = false;  // the three phases have run once with this buffer since the last change of the plan
	};
	StepGraphs graphs_[kStages];
	bool use_graphs_ = false;
	bool conjugate_gradients_ = true;
	bool fuse_layers_ = true;
	bool send_zero_planes_ = false;
	bool real_transforms_ = true;
	bool lazy_loss_rows_ = true;
	float *loss_scratch_ = NULL;  // device [rows]: where materializeLossRows sends the losses it has no use for
	int loss_scratch_rows_ = 0;
	float *loss_ring_ = NULL;  // page-locked [kLossSlots][batch]: losses on their way to the host (gpuQueueLoss)
	int64_t loss_queued_ = 0;
	std::vector<const float *> gather_src_;  // pending dz* gathers of the input functions (see nodeBackward)
	std::vector<float *> gather_dst_;
	std::vector<int64_t> gather_len_;
	void flushGathers() {
		if (gather_src_.empty()) return;
		const int rc = cnet_add_multi((int) gather_src_.size(), gather_src_.data(), gather_dst_.data(), gather_len_.data());
		gather_src_.clear();
		gather_dst_.clear();
		gather_len_.clear();
		ck(rc, "cnet_add_multi");
	}
	// ---- deferred gathers of the input functions (see CFunc::pending_) ----
	bool defer_gathers_ = true;
	static bool deferrable(CFunc *f) { return f->typeId() == isInput && f->trainable_ && f->no_outputs() == 1; }
	// adds every gradient that is still with a consumer to its input function's own planes, as the backward pass would have
	void flushPending() {
		std::vector<const float *> src;
		std::vector<float *> dst;
		std::vector<int64_t> len;
		for (auto f : inputs_) {
			if (!f->pending_) continue;
			CFunc::Slot &own = f->slots_[0];
			src.push_back(f->pending_->g(2));
			dst.push_back(own.g(2));
			len.push_back(2 * (int64_t) own.rows * own.len);
			f->pending_ = NULL;
			f->grad_clean_ = false;
		}
		if (!src.empty()) ck(cnet_add_multi((int) src.size(), src.data(), dst.data(), len.data()), "cnet_add_multi");
	}
	// a kernel or a copy other than a batch upload has written (or is about to write) the value planes of `f`
	void dataValuesWritten(CFunc *f) {
		if (f == main_input_) stage_[active_].imag_dev_zero = false;
	}
	// ---- lazy data inputs (see CFunc::lazy_bwd_) ----
	bool lazy_inputs_ = true;
	// what of the backward pass of consumer c only serves the data input d: 0 nothing, 1 all of it (a transform of d),
	// 2 its input-gradient product (a Linear with d as its data operand).  The second kind needs a copy of the weights when
	// an update comes first, which a recording would have to hold: launch-by-launch passes only.
	int lazyKind(CFunc *d, CFunc *c) const {
		if (c->rows_ != d->rows_ || c->no_outputs() == 0) return 0;
		const int t = c->typeId();
		if ((t == isFourier || t == isTrianFourier) && c->slots_.size() == 1 && c->slots_[0].producer == d) return 1;
		if (t == isLinear && !use_graphs_ && !in_train_step_ && c->slots_.size() == 2 && c->slots_[0].producer == d &&
				c->slots_[1].producer != d)
			return 2;
		return 0;
	}
	// a data input some of whose consumers have work that can wait
	bool lazyEligible(CFunc *d) const {
		if (!lazy_inputs_ || d->typeId() != isInput || !d->trainable_ || isParameter(d)) return false;
		for (auto c : d->next_func_)
			if (lazyKind(d, c)) return true;
		return false;
	}
	// does now what was left out: the consumers' skipped shares from the gradients their own consumers left (they stay where
	// they are until the next backward pass), then the gather or, when an update was asked for in the meantime, that update
	void materializeLazy() {
		for (auto d : inputs_) {
			if (!d->lazy_bwd_) {
				d->lazy_upd_ = false;
				continue;
			}
			for (auto f : d->next_func_) {
				if (!f->lazy_owed_) continue;
				f->lazy_owed_ = f->lazy_skip_now_ = false;
				if (f->typeId() != isLinear) {
					nodeBackward(f, true);
					continue;
				}
				// dx = g w with the weights the skipped pass would have read
				const float *w_re = f->w_saved_valid_ ? f->w_saved_ : zre(f, 1);
				const float *w_im = f->w_saved_valid_ ? f->w_saved_ + f->slots_[1].len : zim(f, 1);
				CFunc::Slot &a = f->slots_[0];
				const int K = a.len, N = f->out_size_;
				for (int c = 0; c < f->no_outputs(); ++c) {
					CFunc::Slot &u = upstream(f, c);
					if (conjugate_gradients_)
						ck(cnet_clinear_bwd_input_sym(u.g(0), u.g(1), u.len, w_re, w_im, K, a.g(0), a.g(1), a.gs(2), a.gs(3), K, f->rows_, K, N,
								c > 0), "cnet_clinear_bwd_input_sym");
					else
						ck(cnet_clinear_bwd_input(u.g(0), u.g(1), u.g(2), u.g(3), u.len, w_re, w_im, K, a.g(0), a.g(1), a.g(2), a.g(3), K,
								f->rows_, K, N, c > 0), "cnet_clinear_bwd_input");
				}
				f->w_saved_valid_ = false;
			}
			d->lazy_bwd_ = false;
			CFunc::Slot &own = d->slots_[0];
			const int64_t n = (int64_t) own.rows * own.len;
			if (d->no_outputs() == 1) {
				CFunc::Slot &u = upstream(d, 0);
				if (d->lazy_upd_) {  // the node's own planes are clear: the step reads the gradient where it is, nothing to clear
					ck(cnet_sgd_update(own.z, own.z + n, u.g(2), u.g(3), n, d->lazy_lr_, 0), "cnet_sgd_update");
					dataValuesWritten(d);
					d->lazy_upd_ = false;
				} else if (defer_gathers_ && d->grad_clean_ && !d->pending_) {
					d->pending_ = &u;
				} else {
					const float *src = u.g(2);
					float *dst = own.g(2);
					const int64_t len = 2 * n;
					ck(cnet_add_multi(1, &src, &dst, &len), "cnet_add_multi");
					d->grad_clean_ = false;
				}
				continue;
			}
			// several consumers: their contributions are added to the node's own planes as the backward pass would have done
			for (int c = 0; c < d->no_outputs(); ++c) {
				const float *src = upstream(d, c).g(2);
				float *dst = own.g(2);
				const int64_t len = 2 * n;
				ck(cnet_add_multi(1, &src, &dst, &len), "cnet_add_multi");
			}
			if (d->lazy_upd_) {
				ck(cnet_sgd_update(own.z, own.z + n, own.g(2), own.g(3), n, d->lazy_lr_, 1), "cnet_sgd_update");
				dataValuesWritten(d);
				d->lazy_upd_ = false;
			} else {
				d->grad_clean_ = false;
			}
		}
	}
	// a new batch is about to overwrite the values of `d`: work that was left out for it and whose result would be
	// overwritten is dropped; a backward pass without an update still owes its gradient
	void beforeFeed(CFunc *d) {
		if (d->lazy_bwd_ && d->lazy_upd_) {
			d->lazy_bwd_ = d->lazy_upd_ = false;
			for (auto f : d->next_func_) f->lazy_owed_ = f->w_saved_valid_ = false;
		} else if (d->lazy_bwd_) {
			materializeLazy();
		}
	}
	// an update is about to change the weights: a Linear that still owes the input gradient of a data input keeps the
	// values that product has to read
	void saveWeightsOwed() {
		for (auto d : inputs_) {
			if (!d->lazy_bwd_ || d->lazy_upd_) continue;
			for (auto f : d->next_func_) {
				if (!f->lazy_owed_ || f->typeId() != isLinear || !f->slots_[1].producer->trainable_) continue;
				const size_t count = 2 * (size_t) f->slots_[1].len;
				if (!f->w_saved_) f->w_saved_ = dalloc<float>(count);
				ck(cnet_memcpy_d2d(f->w_saved_, zre(f, 1), count * sizeof(float)), "cnet_memcpy_d2d");
				f->w_saved_valid_ = true;
			}
		}
	}
	// decides, for the backward pass about to be queued, which input functions leave their gradient with the consumer and
	// which data inputs are left out altogether; true when every candidate does (the state a recorded backward pass stands
	// for)
	bool planDeferral(bool allow) {
		bool all = true;
		for (auto f : inputs_) {
			const bool eligible = lazyEligible(f);
			f->lazy_now_ = allow && eligible && f->grad_clean_ && !f->pending_ && !f->lazy_bwd_ && !f->lazy_upd_;
			if (eligible)
				for (auto c : f->next_func_)
					if (lazyKind(f, c)) c->lazy_skip_now_ = f->lazy_now_;
			f->defer_now_ = !f->lazy_now_ && allow && defer_gathers_ && deferrable(f) && f->grad_clean_ && !f->pending_;
			if (eligible ? !f->lazy_now_ : (deferrable(f) && !f->defer_now_)) all = false;
		}
		return all;
	}
	// after the pass has been queued (or replayed): note where the gradients are
	void noteDeferred() {
		for (auto f : inputs_) {
			if (f->lazy_now_) {
				f->lazy_bwd_ = true;
				for (auto c : f->next_func_) {
					if (c->lazy_skip_now_) c->lazy_owed_ = true;
					c->lazy_skip_now_ = false;
				}
			} else if (f->defer_now_) {
				f->pending_ = &upstream(f, 0);
			} else if (f->trainable_ && f->no_outputs() > 0) {
				f->grad_clean_ = false;
			}
			f->defer_now_ = f->lazy_now_ = false;
		}
	}
	// the state a recorded update stands for: every gradient that can be is still with its consumer, every data input that
	// can be is waiting for its backward pass
	bool allPending() const {
		for (auto f : inputs_) {
			if (lazyEligible(f)) {
				if (!f->lazy_bwd_ || f->lazy_upd_) return false;
			} else if (deferrable(f) && !f->pending_) {
				return false;
			}
		}
		return true;
	}
	bool allCleanNonePending() const {
		for (auto f : inputs_) {
			if (f->lazy_bwd_ || f->lazy_upd_) return false;
			if (deferrable(f) && (!f->grad_clean_ || f->pending_)) return false;
		}
		return true;
	}
	SimpleRand rand_{(uint64_t) clock()};  // upstream ComplexNet::rand_ (impl/cnet.h:56): the coin of sample()
	bool input_dz_dirty_ = false;  // the dz planes of the input functions hold a first moment
	// data inputs whose batch is still travelling on the upload stream (gpuSetInput): the compute stream waits for the
	// upload stream before the first kernel that touches one of them
	std::vector<CFunc *> in_flight_;
	void settleUploads() {
		if (in_flight_.empty()) return;
		in_flight_.clear();
		ck(cnet_compute_wait_upload(), "cnet_compute_wait_upload");
	}
	bool readsInFlight(CFunc *f) const {
		if (in_flight_.empty()) return false;
		for (auto &sl : f->slots_)
			for (auto g : in_flight_)
				if (sl.producer == g || f == g) return true;
		return false;
	}
	bool warmed_[3] = {false, false, false};  // phase has run once since useGraphs(true)

	void dropGraphs() {
		for (auto &g : graphs_) {
			for (void *e : {g.fwd, g.bwd, g.upd, g.step})
				if (e) cnet_graph_destroy(e);
			g = StepGraphs();
		}
		warmed_[0] = warmed_[1] = warmed_[2] = false;
	}
	template <class Body>
	void runPhase(int phase, void *&exec, Body body) {
		if (!use_graphs_) {
			body();
			return;
		}
		if (!exec) {
			if (!warmed_[phase]) {  // first time: run as usual, so that every buffer the library needs exists
				body();
				warmed_[phase] = true;
				return;
			}
			ck(cnet_graph_begin(), "cnet_graph_begin");
			try {
				body();
			} catch (...) {
				cnet_graph_end(NULL);
				throw;
			}
			ck(cnet_graph_end(&exec), "cnet_graph_end");
		}
		ck(cnet_graph_launch(exec), "cnet_graph_launch");
	}

	static void ck(int rc, const char *what) {
		if (rc != CNET_OK)
			throw std::runtime_error(std::string(what) + " failed (" + std::to_string(rc) + "): " + cnet_last_error());
	}
	template <class T>
	T *dalloc(size_t count) {
		void *p = NULL;
		ck(cnet_alloc(count * sizeof(T), &p), "cnet_alloc");
		allocations_.push_back(p);
		return (T *) p;
	}
	bool per_sample_call_ = false;  // forward() / backward() of the per-sample API are running
	// the labels, the gradient planes or the kind of gradient pair changed: what a forward pass wrote ahead no longer stands
	void lossGradientsStale() {
		for (auto f : outputs_)
			if (f->typeId() == isCrossEntropy) ((CrossEntropy *) f)->grad_from_forward_ = false;
	}
	// ---- per-row losses of the output functions (see OutLoss) ----
	bool host_losses_ = true;
	bool in_train_step_ = false;  // gpuTrainStep is queueing or recording: its forward pass writes to the device buffer
	std::vector<void *> host_allocations_;
	void planLoss(OutLoss &l, int rows) {
		l = OutLoss();
		l.rows = rows;
		l.dev = dalloc<float>(rows);
		ck(cnet_memset_zero(l.dev, rows * sizeof(float)), "zero");
		void *h = NULL;
		if (cnet_host_alloc((size_t) OutLoss::kSlots * rows * sizeof(float), &h) == CNET_OK && h) {
			host_allocations_.push_back(h);
			l.host = (float *) h;
			std::fill(l.host, l.host + (size_t) OutLoss::kSlots * rows, 0.f);
		}
		l.cur = l.dev;
	}
	static OutLoss *lossOf(CFunc *f) {
		if (!f) return NULL;
		if (f->typeId() == isCrossEntropy) return &((CrossEntropy *) f)->loss_;
		if (f->typeId() == isL2Out) return &((L2Out *) f)->loss_;
		return NULL;
	}
	// where the forward pass that is being queued writes its losses
	float *lossTarget(OutLoss &l) {
		if (host_losses_ && !use_graphs_ && !in_train_step_ && l.host) {
			l.serial++;
			l.cur = l.host + (size_t) (l.serial % OutLoss::kSlots) * l.rows;
			l.cur_on_host = true;
		} else {
			l.cur = l.dev;
			l.cur_on_host = false;
		}
		return const_cast<float *>(l.cur);
	}
	// `count` losses of the last forward pass from row `first` on, for the host (waits for the device)
	void readLoss(OutLoss &l, float *dst, int first, int count) {
		if (l.cur_on_host) {
			ck(cnet_sync(), "cnet_sync");
			std::copy(l.cur + first, l.cur + first + count, dst);
		} else {
			ck(cnet_memcpy_d2h(dst, l.dev + first, (size_t) count * sizeof(float)), "cnet_memcpy_d2h");
		}
	}
	static bool isParameter(CFunc *f) {  // stored once: every CInput that carries no per-sample data
		if (f->typeId() != isInput) return false;
		CInput *c = (CInput *) f;
		return !c->isMainInput() && !c->isBatched();
	}
	CFunc::Slot *slotOf(CFunc *consumer, CFunc *producer, int offset) {
		for (auto &s : consumer->slots_)
			if (s.producer == producer && s.offset == offset) return &s;
		return NULL;
	}

public:
	CNet() {}
	~CNet() {
		try {
			releaseGpu();
		} catch (...) {
		}
		for (auto f : func_list_) delete f;
	}
	CNet(const CNet &) = delete;
	CNet &operator=(const CNet &) = delete;

	bool hasGPU() { return cnet_init(0) == CNET_OK; }

	std::string PrintInfo(bool &was_failure) {
		cnet_device_info info;
		if (cnet_init(0) != CNET_OK || cnet_get_device_info(&info) != CNET_OK) {
			was_failure = true;
			return std::string("PrintInfo: ") + cnet_last_error();
		}
		was_failure = false;
		std::ostringstream oss;
		oss << "Device Number: 0\n  Device name: " << info.name << " (" << info.arch << ")\n  TotalGlobalMem: "
			<< info.hbm_bytes / (1024 * 1024) << "\n  WarpSize: " << info.wavefront_size << "\n  MultiProcessorCount: "
			<< info.compute_units << "\n  Clock (KHz): " << info.clock_khz << "\n  fp32 matrix peak (TFLOP/s): "
			<< info.fp32_matrix_peak_tflops << "\n";
		return oss.str();
	}

	// ---- graph construction (impl/cnet.h:228-289) ----
	int add(CFunc *func) {
		assert(func);
		if (batch_) {
			delete func;  // the net owns what it is given, also when it refuses it
			throw std::logic_error("add: the net is already allocated on the GPU");
		}
		if (func->uid_ == 0) func->uid_ = ++next_uid_;
		else next_uid_ = std::max(next_uid_, func->uid_);
		func->type_ = func->typeId();
		if (map_.find(func->uid_) != map_.end()) {
			const std::string msg = "add: duplicate uid " + std::to_string(func->uid_);
			delete func;  // the net owns what it is given, also when it refuses it
			throw std::invalid_argument(msg);
		}
		func_list_.push_back(func);
		map_[func->uid_] = func;
		if (func->is_input_) inputs_.push_back(func);
		if (func->is_output_) outputs_.push_back(func);
		return func->uid_;
	}
	int add(CFunc *func, const std::vector<int> &in_uids) {
		int uid = add(func);
		int offset = 0;
		for (auto in_uid : in_uids) {
			auto it = map_.find(in_uid);
			if (it == map_.end()) throw std::invalid_argument("add: unknown input uid " + std::to_string(in_uid));
			it->second->addOutput(func, offset);
			offset += it->second->out_size_;
			func->prev_func_.push_back(it->second);
		}
		if (offset > func->input().length_) throw std::invalid_argument("add: inputs longer than " + func->getName());
		return uid;
	}
	int add(CFunc *func, std::initializer_list<int> in_uids) { return add(func, std::vector<int>(in_uids)); }
	CFunc *&operator[](int uid) { return map_[uid]; }
	std::vector<CFunc *> &functionList() { return func_list_; }
	const std::vector<CFunc *> &inputs() const { return inputs_; }

	void init_inputs() { init_inputs((uint64_t) clock()); }
	void init_inputs(uint64_t seed) {  // impl/cnet.h:301-311
		int indx = 1;
		for (auto f : inputs_) {
			f->setRandSeed(seed + indx++);
			f->init_inputs();
		}
	}
	// impl/cnet.h:156-198: the functions of every depth, within a depth by type (descending) and size (ascending); the
	// executor here walks func_list_ (insertion order is a topological order), the lists serve callers that ask by depth
	void init_exec_graph(bool print_status = false) {
		graph_ready_ = true;
		int deepest = 0;
		for (auto f : func_list_) deepest = std::max(deepest, f->depth());
		func_at_depth_.assign(func_list_.empty() ? 0 : deepest + 1, std::vector<CFunc *>());
		for (auto f : func_list_) {
			if (!(f->isOutput() || f->no_outputs())) throw std::logic_error("init_exec_graph: " + f->getName() + " feeds nothing and is no output");
			func_at_depth_[f->depth()].push_back(f);
		}
		for (auto &level : func_at_depth_)
			std::stable_sort(level.begin(), level.end(), [](const CFunc *a, const CFunc *b) {
				return a->typeId() == b->typeId() ? a->sizeInBytes() < b->sizeInBytes() : a->typeId() > b->typeId();
			});
		if (print_status)
			for (size_t d = 0; d < func_at_depth_.size(); ++d) {
				std::cout << "Depth " << d << ": ";
				for (auto f : func_at_depth_[d]) std::cout << f->getName() << " " << f->sizeInBytes() << ", ";
				std::cout << std::endl;
			}
	}
	// ---- the small accessors of upstream's ComplexNet (impl/cnet.h:77-83, 201-226, 252-254, 312-357), which CNet::cpuNet()
	//      hands out there; here the net and its device plan are one object ----
	CNet &cpuNet() { return *this; }
	int noClones() { return 0; }  // the batch is rows of one graph, not copies of it
	int maxDepth() { return (int) func_at_depth_.size(); }  // 0 before init_exec_graph()
	std::vector<CFunc *> &getFuncAtDepth(int depth) {
		if (depth < 0 || depth >= maxDepth()) throw std::out_of_range("getFuncAtDepth: depth " + std::to_string(depth) + " of " + std::to_string(maxDepth()));
		return func_at_depth_[depth];
	}
	void print_func_at_depth(int depth) {
		if (maxDepth() == 0) {
			std::cout << "init_exec_graph() not called yet." << std::endl;
			return;
		}
		if (depth < 0 || depth >= maxDepth()) {
			std::cout << "print_func_at_depth called with wrong depth: " << depth << std::endl;
			return;
		}
		std::cout << func_at_depth_[depth].size() << " functions: ";
		for (auto f : func_at_depth_[depth]) std::cout << f->getName() << ", ";
		std::cout << std::endl;
	}
	unsigned long long getTotalSizeBytes() {  // six planes per function input, as one sample takes them
		unsigned long long sum = 0;
		for (auto f : func_list_) sum += f->sizeInBytes();
		return sum;
	}
	int getNoVars() {
		int sum = 0;
		for (auto f : inputs_) sum += f->input().length_;
		return sum;
	}
	void print_inputs() {
		for (auto f : inputs_) {
			std::cout << f->getName();
			for (int i = 0; i < f->input().length_; ++i) std::cout << " " << f->input().z(i) << ",";
			std::cout << std::endl;
		}
	}
	CFunc *layer_at(int indx) {
		if (indx < 0 || indx >= (int) func_list_.size()) throw std::out_of_range("layer_at: index " + std::to_string(indx));
		return func_list_[indx];
	}
	CFunc *front() {
		if (func_list_.empty()) throw std::logic_error("front: empty net");
		return func_list_.front();
	}
	CFunc *back() {
		if (func_list_.empty()) throw std::logic_error("back: empty net");
		return func_list_.back();
	}
	// impl/cnet.h:437-484 (upstream asserts; here the first function that differs is named): same functions in the same
	// order, each with the same uid, sizes and consumers, input functions with the same values
	bool testEqual(CNet &other, std::string *why = NULL) {
		auto differs = [&](const std::string &what) {
			if (why) *why = what;
			return false;
		};
		if (func_list_.size() != other.func_list_.size()) return differs("number of functions");
		for (size_t k = 0; k < func_list_.size(); ++k)
			if (*func_list_[k] != *other.func_list_[k]) return differs(func_list_[k]->getName());
		return true;
	}
	std::string toString() {
		std::ostringstream oss;
		oss << func_list_.size() << " functions: " << " vars: " << getNoVars() << std::endl;
		for (auto f : func_list_) {
			oss << "depth: " << f->depth() << ": " << f->getName() << ": from C^" << f->input().length_ << " to C^" << f->out_size_;
			for (int i = 0; i < f->no_outputs(); ++i) oss << " into " << f->next(i)->getName() << " at offset " << f->offset(i);
			oss << "\n";
		}
		return oss.str();
	}
	CFunc *findFirstInput() {
		for (auto f : func_list_)
			if (dynamic_cast<InputFunc *>(f)) return f;
		return NULL;
	}
	CFunc *findFirstOutput() {
		for (auto f : func_list_)
			if (dynamic_cast<OutputFunc *>(f)) return f;
		return NULL;
	}

	// ---- device plan (upstream allocateOnGpu / AllocateNet, gpu/gpu_func.h:576-643, 1071-1086) ----
	bool allocateOnGpu(int batch_size) {
		if (batch_size < 1) throw std::invalid_argument("allocateOnGpu: batch size must be positive");
		if (batch_) throw std::logic_error("Net already initialised on GPU.");
		if (func_list_.empty()) throw std::logic_error("AllocateNet error: 0 depth net.");
		ck(cnet_init(0), "cnet_init");
		CFunc *inp = findFirstInput(), *outp = findFirstOutput();
		if (!inp || !outp) throw std::logic_error("allocateOnGpu: the net needs an input and an output function");
		dynamic_cast<InputFunc *>(inp)->setIsMainInput(true);
		dynamic_cast<OutputFunc *>(outp)->setIsMainOutput(true);
		main_input_ = inp;
		batch_ = batch_size;
		try {
			plan();
		} catch (...) {
			releaseGpu();
			throw;
		}
		return true;
	}

	void releaseGpu() {
		if (!batch_ && allocations_.empty()) return;
		for (void *p : allocations_) cnet_free(p);
		allocations_.clear();
		loss_scratch_ = NULL;
		loss_scratch_rows_ = 0;
		for (auto f : func_list_)
			if (f->typeId() == isCrossEntropy) {
				((CrossEntropy *) f)->d_norm_ = NULL;
				((CrossEntropy *) f)->norm_current_ = false;
			}
		for (void *p : host_allocations_) cnet_host_free(p);
		host_allocations_.clear();
		for (auto f : outputs_)
			if (OutLoss *l = lossOf(f)) *l = OutLoss();
		lossGradientsStale();
		for (auto f : func_list_) {
			f->slots_.clear();
			f->out_ = NULL;
			f->rows_ = 0;
			f->pending_ = NULL;
			f->grad_clean_ = false;
			f->lazy_bwd_ = f->lazy_upd_ = f->lazy_now_ = f->lazy_skip_now_ = f->lazy_owed_ = f->w_saved_valid_ = false;
			f->w_saved_ = NULL;
		}
		batch_ = 0;
		d_labels_ = NULL;
		in_flight_.clear();
		dropGraphs();
		use_graphs_ = false;
		input_dz_dirty_ = false;
		for (auto &st : stage_) {
			if (st.host_labels) cnet_host_free(st.host_labels);
			st = Stage();
		}
		active_ = 0;
		if (loss_ring_) cnet_host_free(loss_ring_);
		loss_ring_ = NULL;
		loss_queued_ = 0;
	}

	int batchSize() const { return batch_; }

private:
	void plan() {
		// rows: data inputs and everything downstream of them are batched; parameter nodes have one row
		for (auto f : func_list_) {
			if (f->typeId() == isInput) {
				f->rows_ = isParameter(f) ? 1 : batch_;
			} else if (f->typeId() == isEmbedding) {
				f->rows_ = batch_;
			} else {
				f->rows_ = 1;
				for (auto p : f->prev_func_) f->rows_ = std::max(f->rows_, p->rows_);
			}
		}
		for (auto f : func_list_) {
			const int t = f->typeId();
			const size_t rows = f->rows_;
			if (t == isInput) {
				// the node's own six planes are the parameter / the data; consumers read its z planes in place
				float *six = dalloc<float>(6 * rows * f->input().length_);
				f->out_ = six;
				CFunc::Slot s;
				s.producer = NULL;
				s.len = f->input().length_;
				s.rows = (int) rows;
				s.grad = six + 2 * rows * s.len;
				s.z = six;
				f->slots_.push_back(s);
				ck(cnet_memset_zero(six, 6 * rows * s.len * sizeof(float)), "zero");
			} else if (t == isEmbedding) {
				CEmbedding *e = (CEmbedding *) f;
				float *six = dalloc<float>(6 * (size_t) f->input().length_);  // the table, stored once
				CFunc::Slot s;
				s.len = f->input().length_;
				s.rows = 1;
				s.grad = six + 2 * (size_t) s.len;
				s.z = six;
				f->slots_.push_back(s);
				ck(cnet_memset_zero(six, 6 * (size_t) s.len * sizeof(float)), "zero");
				e->d_tokens_ = dalloc<int32_t>(rows * e->no_out_tokens_);
				f->out_ = dalloc<float>(2 * rows * f->out_size_);
			} else {
				int k = 0;
				for (auto p : f->prev_func_) {
					CFunc::Slot s;
					s.producer = p;
					// offset of this producer inside the concatenated per-sample input block (impl/cnet.h:259-268)
					s.offset = 0;
					for (int j = 0; j < k; ++j) s.offset += f->prev_func_[j]->out_size_;
					s.len = p->out_size_;
					s.rows = p->rows_;
					s.grad = dalloc<float>(4 * (size_t) s.rows * s.len);
					ck(cnet_memset_zero(s.grad, 4 * (size_t) s.rows * s.len * sizeof(float)), "zero");
					f->slots_.push_back(s);
					++k;
				}
				if (!f->is_output_) f->out_ = dalloc<float>(2 * rows * f->out_size_);
			}
			switch (t) {
			case isLinear:
				if (f->slots_.size() != 2 || f->slots_[1].rows != 1)
					throw std::invalid_argument(f->getName() + ": the weight operand must be a parameter CInput (stored once)");
				break;
			case isHadamard:
			case isResidual:
				if (f->slots_.size() != 2) throw std::invalid_argument(f->getName() + ": needs two inputs");
				if (t == isHadamard && f->slots_[0].rows < f->slots_[1].rows)
					throw std::invalid_argument(f->getName() + ": put the batched operand first, the parameter second");
				break;
			case isFourier:
				ck(cnet_cdft_plan(f->out_size_), "cnet_cdft_plan");
				break;
			case isTrianFourier:
				ck(cnet_ctriang_dft_plan(f->out_size_), "cnet_ctriang_dft_plan");
				break;
			case isSeqFourier: {
				SeqFourierTrans *q = (SeqFourierTrans *) f;
				if (f->slots_.size() != 1 || (int) rows != batch_ || batch_ % q->seq_ != 0)
					throw std::invalid_argument(f->getName() + ": transforms along groups of " + std::to_string(q->seq_) +
							" batch rows; the batch of " + std::to_string(batch_) + " must hold whole sequences of a batched operand");
				if (batch_ / q->seq_ > 65535) throw std::invalid_argument(f->getName() + ": more than 65535 sequences in a batch");
				ck(cnet_cdft_plan(q->seq_), "cnet_cdft_plan");
				ck(cnet_cdft_twiddle(q->seq_, &q->f_re_, &q->f_im_), "cnet_cdft_twiddle");
				q->f_ld_ = (q->seq_ + 3) / 4 * 4;
				break;
			}
			case isSoftMax:
				((SoftMax *) f)->d_s_ = dalloc<float>(rows);
				break;
			case isCrossEntropy: {
				CrossEntropy *c = (CrossEntropy *) f;
				c->d_s_ = dalloc<float>(rows);
				planLoss(c->loss_, (int) rows);
				c->d_argmax_ = dalloc<int32_t>(rows);
				c->d_norm_ = lazy_loss_rows_ ? NULL : dalloc<float>(2 * rows * f->input().length_);  // (else when first looked at)
				c->norm_current_ = false;
				break;
			}
			case isL2Out:
				planLoss(((L2Out *) f)->loss_, (int) rows);
				break;
			default: break;
			}
			if (t != isInput && t != isEmbedding && f->slots_.empty())
				throw std::invalid_argument(f->getName() + ": has no inputs");
		}
		// who reads the dz* planes of a slot on the device: the backward pass of its producer, when that is an input function
		// or the embedding table (they gather dz*), or a Residual that sums one of its operands over the batch
		for (auto f : func_list_)
			for (auto &sl : f->slots_) {
				CFunc *p = sl.producer;
				bool reads = !p || p->typeId() == isInput || p->typeId() == isEmbedding;
				if (p && p->typeId() == isResidual)
					for (auto q : p->prev_func_) reads = reads || q->rows_ != p->rows_;
				sl.star_on_device = reads;
			}
		planFusion();
		for (auto f : inputs_) {  // the gradient planes were cleared above
			f->pending_ = NULL;
			f->grad_clean_ = true;
		}
		d_labels_ = dalloc<int32_t>(batch_);
		ck(cnet_memset_zero(d_labels_, batch_ * sizeof(int32_t)), "zero");
		if (main_input_->typeId() == isInput) {
			stage_[0].z = main_input_->slots_[0].z;
			stage_[0].labels = d_labels_;
		}
		copyInputsToGpu();
	}

	// a FourierTrans whose operand is a data input that holds real samples right now
	bool realInputNow(CFunc *f) const {
		if (!real_transforms_ || f->typeId() != isFourier) return false;
		CFunc *p = f->slots_[0].producer;
		// Three quarters of the product are saved (half of the columns, and of the rest the two real products with the
		// imaginary plane), which pays once the product runs on the block kernels (784 long: 8.7 against 13.3 us at batch
		// 128, 21 against 35 at 512, 56 against 148 at 4096; 8.2 against 12.3 at batch 96; up to batch 64 both take the small-C
		// kernel and 8 us either way).
		const double n = f->out_size_;
		return p && p->typeId() == isInput && p->z_imag_zero_ && p->rows_ == f->rows_ && f->rows_ * n * n >= 5e7;
	}
	bool anyRealTransformNow() const {
		for (auto f : func_list_)
			if (realInputNow(f)) return true;
		return false;
	}
	void planFusion() {
		for (auto f : func_list_) {
			f->fused_next_ = NULL;
			f->loss_next_ = NULL;
			f->fwd_by_producer_ = false;
			f->bwd_by_consumer_now_ = false;
			f->fused_prev_ = 0;
			f->fused_gelu_slot_ = -1;
			f->bwd_by_consumer_ = false;
		}
		if (!fuse_layers_) return;
		for (auto f : func_list_) {
			const int t = f->typeId();
			if ((t != isHadamard && t != isLinear) || f->no_outputs() != 1 || f->slots_[0].rows != f->rows_) continue;
			CFunc *g = f->next_func_[0];
			if (g->typeId() != isGelu || g->rows_ != f->rows_ || g->slots_.size() != 1 || g->slots_[0].len != f->out_size_ ||
					g->out_size_ != f->out_size_)
				continue;
			if (t == isHadamard && g->no_outputs() != 1) continue;
			f->fused_next_ = g;
			g->fused_prev_ = t == isHadamard ? 2 : 1;
		}
		for (auto f : func_list_) {  // Linear -> CrossEntropy
			if (f->typeId() != isLinear || f->fused_next_ || f->no_outputs() != 1 || f->slots_[0].rows != f->rows_) continue;
			CFunc *c = f->next_func_[0];
			if (c->typeId() != isCrossEntropy || c->rows_ != f->rows_ || c->slots_.size() != 1 || c->slots_[0].producer != f ||
					c->slots_[0].len != f->out_size_)
				continue;
			f->loss_next_ = c;
		}
		for (auto f : func_list_) {  // FourierTrans -> Hadamard (shared row) -> CGelu
			if (f->typeId() != isFourier || f->no_outputs() != 1) continue;
			CFunc *h = f->next_func_[0];
			if (h->typeId() != isHadamard || !h->fused_next_ || h->rows_ != f->rows_ || h->slots_.size() != 2 || h->slots_[0].producer != f ||
					h->slots_[0].len != f->out_size_ || h->slots_[1].rows != 1 || h->out_size_ != f->out_size_)
				continue;
			f->fused_next_ = h;
		}
		for (auto f : func_list_) {
			if (f->typeId() != isResidual || f->no_outputs() < 1 || f->no_outputs() > 2) continue;
			if (f->slots_[0].rows != f->rows_ || f->slots_[1].rows != f->rows_) continue;
			for (int k = 0; k < 2 && f->fused_gelu_slot_ < 0; ++k) {
				CFunc *g = f->slots_[k].producer;
				if (!g || g->typeId() != isGelu || g->no_outputs() != 1 || g->fused_prev_ == 2 || g->rows_ != f->rows_ ||
						f->slots_[1 - k].producer == g || g->out_size_ != f->out_size_)
					continue;
				f->fused_gelu_slot_ = k;
				g->bwd_by_consumer_ = true;
			}
		}
	}

	// Whether the operand of the Linear f is the CGelu of a Hadamard gate with one shared row of weights that runs its backward
	// pass with that CGelu's (fused_prev_ == 2: the CGelu feeds f only) in this pass, on rows of the same count.
	bool gateBelow(CFunc *f) const {
		CFunc *g = f->slots_[0].producer;
		if (!g || g->typeId() != isGelu || g->fused_prev_ != 2 || g->rows_ != f->rows_ || f->slots_[0].len != g->out_size_) return false;
		CFunc *h = g->slots_[0].producer;
		return h && h->typeId() == isHadamard && h->fused_next_ == g && h->rows_ == f->rows_ && h->slots_.size() == 2 &&
				h->slots_[1].rows == 1 && h->slots_[0].rows == f->rows_ && !h->lazy_now_ && !h->lazy_skip_now_;
	}

	// z planes of slot k of node f (read in place from the producer)
	static const float *zre(CFunc *f, int k) { return f->slots_[k].producer->out_re(); }
	static const float *zim(CFunc *f, int k) { return f->slots_[k].producer->out_im(); }
	// the slot of consumer c that is fed by f (its gradient planes are f's upstream gradient)
	static CFunc::Slot &upstream(CFunc *f, int c) {
		CFunc *n = f->next_func_[c];
		for (auto &s : n->slots_)
			if (s.producer == f && s.offset == f->offset_[c]) return s;
		throw std::logic_error("broken wiring at " + f->getName());
	}

	// A short-rowed loss (a classifier head) costs less than the launch it rides on: forward pass and gradient go out as one
	// launch.  Not inside the recorded phases (the labels may change between a recorded forward and a recorded backward pass)
	// and not in the per-sample calls (upstream shows cleared gradients after forward()).
	bool lossFromForward(CFunc *c) const {
		return fuse_layers_ && conjugate_gradients_ && !use_graphs_ && !per_sample_call_ && (long) c->rows_ * c->input().length_ <= (1L << 18);
	}

	// The planes that the forward pass of the loss c, about to be queued, writes the normalised rows to: none when they can
	// wait until something looks (not in the recorded phases, whose replays the host does not see one by one, and not in
	// the per-sample calls, which fetch every node anyway).
	float *normPlanes(CrossEntropy *c) {
		const bool now = !lazy_loss_rows_ || use_graphs_ || in_train_step_ || per_sample_call_;
		if (now && !c->d_norm_) c->d_norm_ = dalloc<float>(2 * (size_t) c->rows_ * c->input().length_);
		c->norm_current_ = now;
		return now ? c->d_norm_ : NULL;
	}
	// the normalised rows of the last forward pass, written now if that pass left them out
	void materializeLossRows(CrossEntropy *c) {
		if (c->norm_current_) return;
		const int n = c->input().length_, rows = c->rows_;
		if (!c->d_norm_) c->d_norm_ = dalloc<float>(2 * (size_t) rows * n);
		if (!loss_scratch_ || loss_scratch_rows_ < rows) {
			loss_scratch_ = dalloc<float>(rows);
			loss_scratch_rows_ = rows;
		}
		// the kernel of the forward pass again, on the same z: the same row sums and predictions, and the rows; the losses of
		// this pass go nowhere (they depend on the labels, which may have moved on to the next batch)
		ck(cnet_cross_entropy_fwd(zre(c, 0), zim(c, 0), n, d_labels_, c->d_norm_, c->d_norm_ + (size_t) rows * n, n, c->d_s_, loss_scratch_,
				c->d_argmax_, rows, n), "cnet_cross_entropy_fwd");
		c->norm_current_ = true;
	}

	// ---- the forward pass of the layers that have more than one way to run ----
	// y = x w^T, with the CGelu or the loss on its rows in the same call where the plan says so
	void forwardLinear(CFunc *f) {
		const int rows = f->rows_;
		const int K = f->slots_[0].len, N = f->out_size_;
		if (CFunc *g = f->fused_next_) {  // the CGelu on its result is applied as the product is stored
			ck(cnet_clinear_cgelu_fwd(zre(f, 0), zim(f, 0), K, zre(f, 1), zim(f, 1), K, f->out_re(), f->out_im(), g->out_re(), g->out_im(),
					N, rows, K, N, 0), "cnet_clinear_cgelu_fwd");
			return;
		}
		if (f->loss_next_ && lossFromForward(f->loss_next_)) {  // the loss on its rows where the product is stored
			CrossEntropy *c = (CrossEntropy *) f->loss_next_;
			CFunc::Slot &sl = c->slots_[0];
			float *nr = normPlanes(c);
			ck(cnet_clinear_cross_entropy_fwd_bwd_sym(zre(f, 0), zim(f, 0), K, zre(f, 1), zim(f, 1), K, f->out_re(), f->out_im(), N, d_labels_,
					nr, nr ? nr + (size_t) rows * N : NULL, N, c->d_s_, lossTarget(c->loss_), c->d_argmax_, sl.g(0), sl.g(1), sl.gs(2),
					sl.gs(3), sl.len, rows, K, N), "cnet_clinear_cross_entropy_fwd_bwd_sym");
			c->grad_from_forward_ = true;
			c->fwd_by_producer_ = true;
			return;
		}
		ck(cnet_clinear_fwd(zre(f, 0), zim(f, 0), K, zre(f, 1), zim(f, 1), K, f->out_re(), f->out_im(), N, rows, K, N, 0),
				"cnet_clinear_fwd");
	}

	// y = x F: half the work on real samples, with the gate and activation above it in the same call where the plan says so
	void forwardFourier(CFunc *f) {
		const int rows = f->rows_;
		if (realInputNow(f)) {  // real samples: half the columns by the matrix product, the rest are their conjugates
			ck(cnet_cdft_fwd_real_input(zre(f, 0), zim(f, 0), f->out_size_, f->out_re(), f->out_im(), f->out_size_, rows, f->out_size_),
					"cnet_cdft_fwd_real_input");
			return;
		}
		if (CFunc *h = f->fused_next_) {  // the gate and the activation above it where the transform is stored
			CFunc *g = h->fused_next_;
			ck(cnet_cdft_hadamard_cgelu_fwd(zre(f, 0), zim(f, 0), f->out_size_, zre(h, 1), zim(h, 1), f->out_re(), f->out_im(), h->out_re(),
					h->out_im(), g->out_re(), g->out_im(), f->out_size_, rows, f->out_size_), "cnet_cdft_hadamard_cgelu_fwd");
			h->fwd_by_producer_ = true;
			return;
		}
		ck(cnet_cdft_fwd(zre(f, 0), zim(f, 0), f->out_size_, f->out_re(), f->out_im(), f->out_size_, rows, f->out_size_, 0),
				"cnet_cdft_fwd");
	}

	void forwardHadamard(CFunc *f) {
		const int rows = f->rows_;
		const int n = f->out_size_;
		if (f->fwd_by_producer_) {  // written by the transform below it in this pass
			f->fwd_by_producer_ = false;
			return;
		}
		if (CFunc *g = f->fused_next_) {  // the CGelu on its result in the same pass
			ck(cnet_hadamard_cgelu_fwd(zre(f, 0), zim(f, 0), n, zre(f, 1), zim(f, 1), f->slots_[1].rows == rows ? n : 0, f->out_re(),
					f->out_im(), n, g->out_re(), g->out_im(), n, rows, n), "cnet_hadamard_cgelu_fwd");
			return;
		}
		ck(cnet_hadamard_fwd(zre(f, 0), zim(f, 0), n, zre(f, 1), zim(f, 1), f->slots_[1].rows == rows ? n : 0, f->out_re(),
				f->out_im(), n, rows, n), "cnet_hadamard_fwd");
	}

	void forwardCrossEntropy(CFunc *f) {
		const int rows = f->rows_;
		CrossEntropy *c = (CrossEntropy *) f;
		const int n = f->input().length_;
		if (f->fwd_by_producer_) {  // written by the Linear below it in this pass
			f->fwd_by_producer_ = false;
			return;
		}
		float *nr = normPlanes(c);
		if (lossFromForward(f)) {
			CFunc::Slot &sl = f->slots_[0];
			ck(cnet_cross_entropy_fwd_bwd_sym(zre(f, 0), zim(f, 0), n, d_labels_, nr, nr ? nr + (size_t) rows * n : NULL, n, c->d_s_,
					lossTarget(c->loss_), c->d_argmax_, sl.g(0), sl.g(1), sl.gs(2), sl.gs(3), sl.len, rows, n), "cnet_cross_entropy_fwd_bwd_sym");
			c->grad_from_forward_ = true;
			return;
		}
		ck(cnet_cross_entropy_fwd(zre(f, 0), zim(f, 0), n, d_labels_, nr, nr ? nr + (size_t) rows * n : NULL, n, c->d_s_,
				lossTarget(c->loss_), c->d_argmax_, rows, n), "cnet_cross_entropy_fwd");
		c->grad_from_forward_ = false;
	}

	void nodeForward(CFunc *f) {
		const int rows = f->rows_;
		switch (f->typeId()) {
		case isInput: break;  // consumers read the node's z planes in place
		case isEmbedding: {
			CEmbedding *e = (CEmbedding *) f;
			const float *tab = f->slots_[0].z;
			ck(cnet_embedding_fwd(tab, tab + f->slots_[0].len, e->embedding_dim_, e->no_embeddings_, e->d_tokens_, f->out_re(),
					f->out_im(), f->out_size_, rows, e->no_out_tokens_), "cnet_embedding_fwd");
			break;
		}
		case isLinear: forwardLinear(f); break;
		case isFourier: forwardFourier(f); break;
		case isTrianFourier:
			ck(cnet_ctriang_dft_fwd(zre(f, 0), zim(f, 0), f->out_size_, f->out_re(), f->out_im(), f->out_size_, rows, f->out_size_, 0),
					"cnet_ctriang_dft_fwd");
			break;
		case isSeqFourier: {  // Y_g = F X_g for every sequence g: one strided-batched product, F shared (stride 0)
			SeqFourierTrans *q = (SeqFourierTrans *) f;
			const int S = q->seq_, n = f->out_size_;
			ck(cnet_cgemm_batched(0, 1, 0, 0, S, n, S, q->f_re_, q->f_im_, q->f_ld_, 0, zre(f, 0), zim(f, 0), n, (int64_t) S * n, f->out_re(),
					f->out_im(), n, (int64_t) S * n, rows / S, 0), "cnet_cgemm_batched");
			break;
		}
		case isCrelu:
			ck(cnet_crelu_fwd(zre(f, 0), zim(f, 0), f->out_size_, f->out_re(), f->out_im(), f->out_size_, rows, f->out_size_),
					"cnet_crelu_fwd");
			break;
		case isHadamard: forwardHadamard(f); break;
		case isGelu:
			if (f->fused_prev_) break;  // written by the Hadamard or the Linear below it
			ck(cnet_cgelu_fwd(zre(f, 0), zim(f, 0), f->out_size_, f->out_re(), f->out_im(), f->out_size_, rows, f->out_size_),
					"cnet_cgelu_fwd");
			break;
		case isResidual: {
			const int n = f->out_size_;
			// an operand that is a parameter (one row, e.g. a positional table) is added to every row
			ck(cnet_residual_fwd(zre(f, 0), zim(f, 0), f->slots_[0].rows == rows ? n : 0, zre(f, 1), zim(f, 1),
					f->slots_[1].rows == rows ? n : 0, f->out_re(), f->out_im(), n, rows, n), "cnet_residual_fwd");
			break;
		}
		case isSoftMax:
			ck(cnet_l2norm_fwd(zre(f, 0), zim(f, 0), f->out_size_, f->out_re(), f->out_im(), f->out_size_, ((SoftMax *) f)->d_s_, rows,
					f->out_size_), "cnet_l2norm_fwd");
			break;
		case isCrossEntropy: forwardCrossEntropy(f); break;
		case isL2Out:
			ck(cnet_l2out_fwd(zre(f, 0), zim(f, 0), f->input().length_, lossTarget(((L2Out *) f)->loss_), rows, f->input().length_),
					"cnet_l2out_fwd");
			break;
		default: throw std::logic_error(f->getName() + ": no device implementation");
		}
	}

	// ---- the backward pass of one layer for the gradient u of one consumer (acc: added to what an earlier consumer left) ----
	// dx = g w and dw = g^T x of a Linear (upstream gpu_linear_backward), with what the plan lets ride on the same call
	void backwardLinear(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		CFunc::Slot &w = f->slots_[1];
		const int K = a.len, N = f->out_size_;
		// (the input gradient of a lazy data input waits: see CFunc::lazy_bwd_)
		const bool to_data = a.producer->wants_grad_ && !f->lazy_skip_now_, to_weight = w.producer->wants_grad_;
		if (conjugate_gradients_ && to_data && to_weight && f->no_outputs() == 1 && gateBelow(f)) {
			// the operand is the CGelu of a Hadamard gate with a shared row: the gate's backward pass in the same call (one
			// launch at small batches: the workgroup that forms 16 columns of dx goes on to the gate)
			CFunc *g = a.producer, *h = g->slots_[0].producer;
			CFunc::Slot &hs = g->slots_[0], &hu = h->slots_[0], &hv = h->slots_[1];
			ck(cnet_clinear_hadamard_cgelu_bwd_sym(u.g(0), u.g(1), u.len, zre(f, 0), zim(f, 0), K, zre(f, 1), zim(f, 1), K, a.g(0), a.g(1),
					a.gs(2), a.gs(3), K, acc, w.g(0), w.g(1), w.gs(2), w.gs(3), K, acc, zre(h, 0), zim(h, 0), K, zre(h, 1), zim(h, 1), hs.g(0),
					hs.g(1), hs.gs(2), hs.gs(3), K, hu.g(0), hu.g(1), hu.gs(2), hu.gs(3), K, hv.g(0), hv.g(1), hv.gs(2), hv.gs(3), 0, rows, K, N),
					"cnet_clinear_hadamard_cgelu_bwd_sym");
			h->bwd_by_consumer_now_ = true;
			return;
		}
		if (conjugate_gradients_ && to_data && to_weight) {  // both gradients in one call (one launch when both products are small)
			ck(cnet_clinear_bwd_sym(u.g(0), u.g(1), u.len, zre(f, 0), zim(f, 0), K, zre(f, 1), zim(f, 1), K, a.g(0), a.g(1), a.gs(2),
					a.gs(3), K, acc, w.g(0), w.g(1), w.gs(2), w.gs(3), K, acc, rows, K, N), "cnet_clinear_bwd_sym");
			return;
		}
		if (conjugate_gradients_) {  // dz* = conj(dz): one product each, written to both pairs of planes
			if (to_data)
				ck(cnet_clinear_bwd_input_sym(u.g(0), u.g(1), u.len, zre(f, 1), zim(f, 1), K, a.g(0), a.g(1), a.gs(2), a.gs(3), K, rows, K,
						N, acc), "cnet_clinear_bwd_input_sym");
			if (to_weight)
				ck(cnet_clinear_bwd_weight_sym(u.g(0), u.g(1), u.len, zre(f, 0), zim(f, 0), K, w.g(0), w.g(1), w.gs(2), w.gs(3), K, rows, K,
						N, acc), "cnet_clinear_bwd_weight_sym");
			return;
		}
		if (to_data)
			ck(cnet_clinear_bwd_input(u.g(0), u.g(1), u.g(2), u.g(3), u.len, zre(f, 1), zim(f, 1), K, a.g(0), a.g(1), a.g(2), a.g(3), K,
					rows, K, N, acc), "cnet_clinear_bwd_input");
		if (to_weight)
			ck(cnet_clinear_bwd_weight(u.g(0), u.g(1), u.g(2), u.g(3), u.len, zre(f, 0), zim(f, 0), K, w.g(0), w.g(1), w.g(2), w.g(3), K,
					rows, K, N, acc), "cnet_clinear_bwd_weight");
	}

	// the backward pass of the transform is the transform of the gradients
	void backwardFourier(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		if (conjugate_gradients_)
			ck(cnet_cdft_bwd_sym(u.g(0), u.g(1), u.len, a.g(0), a.g(1), a.gs(2), a.gs(3), a.len, rows, a.len, acc), "cnet_cdft_bwd_sym");
		else
			ck(cnet_cdft_bwd(u.g(0), u.g(1), u.g(2), u.g(3), u.len, a.g(0), a.g(1), a.g(2), a.g(3), a.len, rows, a.len, acc),
					"cnet_cdft_bwd");
	}

	void backwardTrianFourier(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		if (conjugate_gradients_)
			ck(cnet_ctriang_dft_bwd_sym(u.g(0), u.g(1), u.len, a.g(0), a.g(1), a.gs(2), a.gs(3), a.len, rows, a.len, acc),
					"cnet_ctriang_dft_bwd_sym");
		else
			ck(cnet_ctriang_dft_bwd(u.g(0), u.g(1), u.g(2), u.g(3), u.len, a.g(0), a.g(1), a.g(2), a.g(3), a.len, rows, a.len, acc),
					"cnet_ctriang_dft_bwd");
	}

	void backwardSeqFourier(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		// dX_g.dz = F G_g.dz and dX_g.dz* = conj(F) G_g.dz* (F is symmetric).  Of a conjugate pair only the dz planes of G
		// hold values: dz* = conj(F) conj(G.dz), formed where something reads it on the device.
		SeqFourierTrans *q = (SeqFourierTrans *) f;
		const int S = q->seq_, n = f->out_size_;
		ck(cnet_cgemm_batched(0, 1, 0, 0, S, n, S, q->f_re_, q->f_im_, q->f_ld_, 0, u.g(0), u.g(1), u.len, (int64_t) S * u.len, a.g(0), a.g(1),
				a.len, (int64_t) S * a.len, rows / S, acc), "cnet_cgemm_batched");
		if (conjugate_gradients_) {
			if (a.gs(2))
				ck(cnet_cgemm_batched(0, 1, 1, 1, S, n, S, q->f_re_, q->f_im_, q->f_ld_, 0, u.g(0), u.g(1), u.len, (int64_t) S * u.len,
						a.g(2), a.g(3), a.len, (int64_t) S * a.len, rows / S, acc), "cnet_cgemm_batched");
		} else {
			ck(cnet_cgemm_batched(0, 1, 1, 0, S, n, S, q->f_re_, q->f_im_, q->f_ld_, 0, u.g(2), u.g(3), u.len, (int64_t) S * u.len, a.g(2),
					a.g(3), a.len, (int64_t) S * a.len, rows / S, acc), "cnet_cgemm_batched");
		}
	}

	void backwardCrelu(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		if (conjugate_gradients_) {
			ck(cnet_crelu_bwd_sym(zre(f, 0), zim(f, 0), a.len, u.g(0), u.g(1), u.len, a.g(0), a.g(1), a.gs(2), a.gs(3), a.len, rows, a.len,
					acc), "cnet_crelu_bwd_sym");
			return;
		}
		ck(cnet_crelu_bwd(zre(f, 0), zim(f, 0), a.len, u.g(0), u.g(1), u.g(2), u.g(3), u.len, a.g(0), a.g(1), a.g(2), a.g(3), a.len,
				rows, a.len, acc), "cnet_crelu_bwd");
	}

	// du = G v, dv = G u; with the CGelu above it in the same pass where the plan says so
	void backwardHadamard(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		CFunc::Slot &v = f->slots_[1];
		const int n = f->out_size_;
		if (f->bwd_by_consumer_now_) {  // done by the Linear above its CGelu in this pass
			f->bwd_by_consumer_now_ = false;
			return;
		}
		if (conjugate_gradients_ && f->fused_next_) {  // the backward pass of the CGelu above it in the same pass
			CFunc *g = f->fused_next_;
			CFunc::Slot &ug = upstream(g, 0), &h = g->slots_[0];
			ck(cnet_hadamard_cgelu_bwd_sym(zre(f, 0), zim(f, 0), n, zre(f, 1), zim(f, 1), v.rows == rows ? n : 0, ug.g(0), ug.g(1), ug.len,
					h.g(0), h.g(1), h.gs(2), h.gs(3), n, a.g(0), a.g(1), a.gs(2), a.gs(3), n, v.g(0), v.g(1), v.gs(2), v.gs(3), n, rows, n,
					acc), "cnet_hadamard_cgelu_bwd_sym");
			return;
		}
		if (conjugate_gradients_) {
			ck(cnet_hadamard_bwd_sym(zre(f, 0), zim(f, 0), n, zre(f, 1), zim(f, 1), v.rows == rows ? n : 0, u.g(0), u.g(1), u.len, a.g(0),
					a.g(1), a.gs(2), a.gs(3), n, v.g(0), v.g(1), v.gs(2), v.gs(3), n, rows, n, acc), "cnet_hadamard_bwd_sym");
			return;
		}
		ck(cnet_hadamard_bwd(zre(f, 0), zim(f, 0), n, zre(f, 1), zim(f, 1), v.rows == rows ? n : 0, u.g(0), u.g(1), u.g(2), u.g(3),
				u.len, a.g(0), a.g(1), a.g(2), a.g(3), n, v.g(0), v.g(1), v.g(2), v.g(3), n, rows, n, acc), "cnet_hadamard_bwd");
	}

	void backwardGelu(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		if (conjugate_gradients_ && (f->fused_prev_ == 2 || f->bwd_by_consumer_)) return;  // done by the Hadamard below it or the Residual above it
		if (conjugate_gradients_) {
			ck(cnet_cgelu_bwd_sym(zre(f, 0), zim(f, 0), a.len, u.g(0), u.g(1), u.len, a.g(0), a.g(1), a.gs(2), a.gs(3), a.len, rows, a.len,
					acc), "cnet_cgelu_bwd_sym");
			return;
		}
		ck(cnet_cgelu_bwd(zre(f, 0), zim(f, 0), a.len, u.g(0), u.g(1), u.g(2), u.g(3), u.len, a.g(0), a.g(1), a.g(2), a.g(3), a.len,
				rows, a.len, acc), "cnet_cgelu_bwd");
	}

	// the incoming gradient goes to both operands
	void backwardResidual(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		CFunc::Slot &v = f->slots_[1];
		const int n = f->out_size_;
		if (a.rows == rows && v.rows == rows && conjugate_gradients_) {
			ck(cnet_residual_bwd_sym(u.g(0), u.g(1), u.len, a.g(0), a.g(1), a.gs(2), a.gs(3), n, v.g(0), v.g(1), v.gs(2), v.gs(3), n, rows,
					n, acc), "cnet_residual_bwd_sym");
			return;
		}
		if (a.rows == rows && v.rows == rows) {
			ck(cnet_residual_bwd(u.g(0), u.g(1), u.g(2), u.g(3), u.len, a.g(0), a.g(1), a.g(2), a.g(3), n, v.g(0), v.g(1), v.g(2), v.g(3),
					n, rows, n, acc), "cnet_residual_bwd");
			return;
		}
		// a parameter operand receives the sum over the batch rows, a batched one a copy
		for (CFunc::Slot *s : {&a, &v})
			for (int p = 0; p < 4; ++p) {
				if (s->rows == 1 && rows > 1)
					ck(cnet_batch_sum(u.g(p), u.len, s->g(p), rows, n, acc), "cnet_batch_sum");
				else if (acc)
					ck(cnet_add2d(u.g(p), u.len, s->g(p), n, s->rows, n), "cnet_add2d");
				else
					ck(cnet_copy2d(u.g(p), u.len, s->g(p), n, s->rows, n), "cnet_copy2d");
			}
	}

	void backwardSoftMax(CFunc *f, CFunc::Slot &u, const int acc) {
		const int rows = f->rows_;
		CFunc::Slot &a = f->slots_[0];
		if (conjugate_gradients_) {
			ck(cnet_l2norm_bwd_sym(zre(f, 0), zim(f, 0), a.len, ((SoftMax *) f)->d_s_, u.g(0), u.g(1), u.len, a.g(0), a.g(1), a.gs(2),
					a.gs(3), a.len, rows, a.len, acc), "cnet_l2norm_bwd_sym");
			return;
		}
		ck(cnet_l2norm_bwd(zre(f, 0), zim(f, 0), a.len, ((SoftMax *) f)->d_s_, u.g(0), u.g(1), u.g(2), u.g(3), u.len, a.g(0), a.g(1),
				a.g(2), a.g(3), a.len, rows, a.len, acc), "cnet_l2norm_bwd");
	}

	// the gradient of a loss at its operand (upstream CrossEntropy::backward / L2Out::backward)
	void backwardLoss(CFunc *f, bool with_labels) {
		const int rows = f->rows_;
		CFunc::Slot &s = f->slots_[0];
		if (f->typeId() == isCrossEntropy) {
			if (!with_labels) return;  // upstream: CrossEntropy::backward() without a label does nothing
			CrossEntropy *c = (CrossEntropy *) f;
			if (conjugate_gradients_ && c->grad_from_forward_) return;  // written by the forward pass, with these labels
			if (conjugate_gradients_)
				ck(cnet_cross_entropy_bwd_sym(zre(f, 0), zim(f, 0), s.len, c->d_s_, d_labels_, s.g(0), s.g(1), s.gs(2), s.gs(3), s.len, rows,
						s.len), "cnet_cross_entropy_bwd_sym");
			else
				ck(cnet_cross_entropy_bwd(zre(f, 0), zim(f, 0), s.len, c->d_s_, d_labels_, s.g(0), s.g(1), s.g(2), s.g(3), s.len, rows, s.len),
						"cnet_cross_entropy_bwd");
			return;
		}
		if (conjugate_gradients_)
			ck(cnet_l2out_bwd_sym(zre(f, 0), zim(f, 0), s.len, s.g(0), s.g(1), s.gs(2), s.gs(3), s.len, rows, s.len, 0), "cnet_l2out_bwd_sym");
		else
			ck(cnet_l2out_bwd(zre(f, 0), zim(f, 0), s.len, s.g(0), s.g(1), s.g(2), s.g(3), s.len, rows, s.len, 0), "cnet_l2out_bwd");
	}

	// An input function gathers the dz* of its consumers (impl/cinput.h:54-65), and keeps adding until the next update.
	// Both dz* planes of a consumer's slot are adjacent and dense, as they are in the node's own block: one array per
	// consumer.  Nothing in the backward pass reads what an input function gathers, so the gathers of all of them
	// wait for the end of the pass and go out as one launch (flushGathers).
	void backwardInput(CFunc *f) {
		CFunc::Slot &own = f->slots_[0];
		if (f->defer_now_) return;  // the update will read the consumer's planes (see pending_)
		for (int c = 0; c < f->no_outputs(); ++c) {
			CFunc::Slot &u = upstream(f, c);
			if (c) flushGathers();  // one launch must not hold two additions into the same planes
			gather_src_.push_back(u.g(2));
			gather_dst_.push_back(own.g(2));
			gather_len_.push_back(2 * (int64_t) own.rows * own.len);
		}
	}

	void backwardEmbedding(CFunc *f) {
		CEmbedding *e = (CEmbedding *) f;
		CFunc::Slot &own = f->slots_[0];
		for (int c = 0; c < f->no_outputs(); ++c) {
			CFunc::Slot &u = upstream(f, c);
			ck(cnet_embedding_bwd(e->d_tokens_, u.g(2), u.g(3), u.len, own.g(2), own.g(3), e->embedding_dim_, e->no_embeddings_, f->rows_,
					e->no_out_tokens_, 1), "cnet_embedding_bwd");
		}
	}

	// a Residual that takes all its incoming gradients in one kernel: true when it did
	bool backwardResidualInOnePass(CFunc *f) {
		const int rows = f->rows_, n = f->out_size_;
		if (!conjugate_gradients_) return false;
		if (f->fused_gelu_slot_ >= 0) {  // one operand is a CGelu that feeds nothing else: its backward pass in the same kernel
			const int k = f->fused_gelu_slot_;
			CFunc *g = f->slots_[k].producer;
			CFunc::Slot &u0 = upstream(f, 0), &a = f->slots_[1 - k], &h = g->slots_[0];
			CFunc::Slot *u1 = f->no_outputs() == 2 ? &upstream(f, 1) : NULL;
			ck(cnet_residual_cgelu_bwd_sym(u0.g(0), u0.g(1), u0.len, u1 ? u1->g(0) : NULL, u1 ? u1->g(1) : NULL, u1 ? u1->len : 0, zre(g, 0),
					zim(g, 0), n, a.g(0), a.g(1), a.gs(2), a.gs(3), n, NULL, NULL, NULL, NULL, 0, h.g(0), h.g(1), h.gs(2), h.gs(3), n, rows, n),
					"cnet_residual_cgelu_bwd_sym");
			return true;
		}
		if (f->no_outputs() == 2 && f->slots_[0].rows == rows && f->slots_[1].rows == rows) {
			// a Residual feeding two consumers (the usual skip connection): both incoming gradients in one pass
			CFunc::Slot &u0 = upstream(f, 0), &u1 = upstream(f, 1), &a = f->slots_[0], &v = f->slots_[1];
			ck(cnet_residual_bwd_sym2(u0.g(0), u0.g(1), u0.len, u1.g(0), u1.g(1), u1.len, a.g(0), a.g(1), a.gs(2), a.gs(3), n, v.g(0), v.g(1),
					v.gs(2), v.gs(3), n, rows, n, 0), "cnet_residual_bwd_sym2");
			return true;
		}
		return false;
	}

	// Each consumer's contribution is added in turn (the per-consumer loops of the upstream layers); the first one
	// overwrites, so the planes never need zeroing between steps.  Nodes without consumers get zeros.
	void nodeBackward(CFunc *f, bool with_labels) {
		const int t = f->typeId();
		if (t == isCrossEntropy || t == isL2Out) return backwardLoss(f, with_labels);
		if ((t == isInput || t == isEmbedding) && !f->trainable_) return;  // nothing steps it: nothing to gather
		if (f->lazy_now_ || (f->lazy_skip_now_ && t != isLinear)) return;  // left out for now (see CFunc::lazy_bwd_)
		if (t == isInput) return backwardInput(f);
		if (t == isEmbedding) return backwardEmbedding(f);
		if (f->no_outputs() == 0) {
			for (auto &s : f->slots_) ck(cnet_memset_zero(s.grad, 4 * (size_t) s.rows * s.len * sizeof(float)), "zero");
			return;
		}
		// Gradients flow only towards input functions that are stepped: a layer none of whose operands leads to one is
		// skipped (all input functions are trainable unless CNet::setInputTrainable said otherwise, as upstream has it).
		if (!f->wants_grad_) return;
		if (t == isResidual && backwardResidualInOnePass(f)) return;
		for (int c = 0; c < f->no_outputs(); ++c) {
			CFunc::Slot &u = upstream(f, c);  // the gradient that consumer c left for this node
			const int acc = c > 0;
			switch (t) {
			case isLinear: backwardLinear(f, u, acc); break;
			case isFourier: backwardFourier(f, u, acc); break;
			case isTrianFourier: backwardTrianFourier(f, u, acc); break;
			case isSeqFourier: backwardSeqFourier(f, u, acc); break;
			case isCrelu: backwardCrelu(f, u, acc); break;
			case isHadamard: backwardHadamard(f, u, acc); break;
			case isGelu: backwardGelu(f, u, acc); break;
			case isResidual: backwardResidual(f, u, acc); break;
			case isSoftMax: backwardSoftMax(f, u, acc); break;
			default: throw std::logic_error(f->getName() + ": no device implementation");
			}
		}
	}

	// wants_grad_ of every function: input functions say it themselves, a layer wants gradients when one of its operands
	// does (func_list_ is in insertion order, producers first)
	void planGradients() {
		for (auto f : func_list_) {
			if (f->is_input_) {
				f->wants_grad_ = f->trainable_;
				continue;
			}
			f->wants_grad_ = false;
			for (auto &sl : f->slots_)
				if (sl.producer && sl.producer->wants_grad_) f->wants_grad_ = true;
		}
	}

	void requireAllocated(const char *who) const {
		if (!batch_) throw std::logic_error(std::string(who) + ": call allocateOnGpu(batch_size) first");
	}

public:
	// ---- host <-> device (upstream copyInputsToGpu / getInputsFromGpu, gpu/gpu_func.h:512-527, 543-574) ----
	bool copyInputsToGpu() {
		requireAllocated("copyInputsToGpu");
		for (auto f : inputs_) beforeFeed(f);  // first of all: work that was left out may still read weights that are replaced below
		for (auto f : inputs_) sendInputValues(f);
		return true;
	}
	// upstream inputToGpu (gpu/gpu_func.h:470-487): the host values (or token list) of ONE input function to the device
	bool inputToGpu(CFunc *input) {
		requireAllocated("inputToGpu");
		if (!input || !input->is_input_ || std::find(inputs_.begin(), inputs_.end(), input) == inputs_.end())
			throw std::invalid_argument("inputToGpu: not an input function of this net");
		for (auto f : inputs_) beforeFeed(f);
		sendInputValues(input);
		return true;
	}
	void sendInputValues(CFunc *f) {
		f->z_imag_zero_ = false;
		dataValuesWritten(f);
		CFunc::Slot &s = f->slots_[0];
		float *z = s.z;
		if (s.rows == 1) {
			ck(cnet_memcpy_h2d(z, f->mutable_input()->real_, 2 * (size_t) s.len * sizeof(float)), "cnet_memcpy_h2d");
		} else {  // the data input: the host view holds one sample, replicate it to every row (one copy for both planes)
			std::vector<float> rows(2 * (size_t) s.rows * s.len);
			for (int b = 0; b < s.rows; ++b) {
				std::copy(f->input().real_, f->input().real_ + s.len, rows.begin() + (size_t) b * s.len);
				std::copy(f->input().imag_, f->input().imag_ + s.len, rows.begin() + (size_t) (s.rows + b) * s.len);
			}
			ck(cnet_memcpy_h2d(z, rows.data(), rows.size() * sizeof(float)), "cnet_memcpy_h2d");
		}
		if (f->typeId() == isEmbedding) uploadTokens((CEmbedding *) f, NULL);
	}

	bool getInputsFromGpu() {
		requireAllocated("getInputsFromGpu");
		for (auto f : inputs_) fetch(f, 0);
		return true;
	}

	// Fill the per-sample host view of `f` (all six planes of its input block; for output functions also the output
	// block) from row `b` of the device planes.  Parameter operands always come from their single row.
	void fetch(CFunc *f, int b) {
		requireAllocated("fetch");
		if (b < 0 || b >= batch_) throw std::out_of_range("fetch: batch index");
		materializeLazy();
		if (f->pending_) flushPending();
		settleUploads();
		ck(cnet_sync(), "cnet_sync");
		Vars *v = f->mutable_input();
		for (auto &s : f->slots_) {
			const int row = s.rows == 1 ? 0 : b;
			const float *z_re, *z_im;
			if (s.producer) {
				z_re = s.producer->out_re() + (size_t) (s.producer->rows_ == 1 ? 0 : b) * s.len;
				z_im = s.producer->out_im() + (size_t) (s.producer->rows_ == 1 ? 0 : b) * s.len;
			} else {
				const float *z = s.z;
				z_re = z + (size_t) row * s.len;
				z_im = z + (size_t) (s.rows + row) * s.len;
			}
			ck(cnet_memcpy_d2h(v->real_ + s.offset, z_re, s.len * sizeof(float)), "cnet_memcpy_d2h");
			ck(cnet_memcpy_d2h(v->imag_ + s.offset, z_im, s.len * sizeof(float)), "cnet_memcpy_d2h");
			// the gradient of a Residual's CGelu operand is kept once, in the planes of the other operand (see fused_gelu_slot_)
			const bool alias = conjugate_gradients_ && f->fused_gelu_slot_ >= 0 && &s == &f->slots_[f->fused_gelu_slot_];
			const CFunc::Slot &gsrc = alias ? f->slots_[1 - f->fused_gelu_slot_] : s;
			for (int p = 0; p < 4; ++p)
				ck(cnet_memcpy_d2h(v->plane(2 + p) + s.offset, gsrc.g(p) + (size_t) row * s.len, s.len * sizeof(float)), "cnet_memcpy_d2h");
			if (conjugate_gradients_ && !gsrc.star_on_device) {
				// the pair is conjugate and nothing on the device reads its dz* half: it is formed here
				const float *dz_re = v->plane(2) + s.offset, *dz_im = v->plane(3) + s.offset;
				float *dzs_re = v->plane(4) + s.offset, *dzs_im = v->plane(5) + s.offset;
				for (int k = 0; k < s.len; ++k) {
					dzs_re[k] = dz_re[k];
					dzs_im[k] = -dz_im[k];
				}
			}
		}
		if (f->typeId() == isCrossEntropy) {
			CrossEntropy *c = (CrossEntropy *) f;
			const int n = f->input().length_;
			const int rb = f->rows_ == 1 ? 0 : b;  // an output that hangs off parameters only has one row
			materializeLossRows(c);
			ck(cnet_memcpy_d2h(c->output_.real_, c->d_norm_ + (size_t) rb * n, n * sizeof(float)), "cnet_memcpy_d2h");
			ck(cnet_memcpy_d2h(c->output_.imag_, c->d_norm_ + (size_t) (f->rows_ + rb) * n, n * sizeof(float)), "cnet_memcpy_d2h");
			int32_t am = 0;
			ck(cnet_memcpy_d2h(&am, c->d_argmax_ + rb, sizeof(am)), "cnet_memcpy_d2h");
			c->prediction_ = am;
		} else if (f->typeId() == isL2Out) {
			readLoss(((L2Out *) f)->loss_, ((L2Out *) f)->output_.real_, f->rows_ == 1 ? 0 : b, 1);
		}
	}
	void fetchAll(int b) {
		for (auto f : func_list_) fetch(f, b);
	}

	// ---- batched step (upstream gpuForward / gpuBackward / gpuUpdateInputs / getLoss,
	//      gpu/gpu_func.h:1088-1101, 491-495, 906-926; step semantics of cnet.cpp:104-150) ----
	bool gpuForward(InputFunc *inp, OutputFunc *outp, InputBatch &batch) {
		feedBatch(inp, outp, batch);
		return GpuForward();
	}
	// The steps upstream's gpuForward / gpuBackward / allocateOnGpu are made of, under their names, for code that calls
	// them one by one as upstream's GPU tests do (gpu/gpu_func.h:368-425, 532-541, 576-643): a batch and its labels to the
	// device without the pass; the two copies between a function and its clones, of which there are none here; the
	// allocation for `no_batches` samples side by side.
	void batchToGpu(InputFunc *inp, OutputFunc *outp, Batch *batch) {
		if (InputBatch *ib = dynamic_cast<InputBatch *>(batch)) {
			feedBatch(inp, outp, *ib);
		} else if (EmbeddingBatch *eb = dynamic_cast<EmbeddingBatch *>(batch)) {
			feedTokens(inp, outp, *eb);
		} else {
			throw std::invalid_argument("batchToGpu: needs an InputBatch or an EmbeddingBatch");
		}
	}
	void copyInputsToClones() {}
	void updateGradientsFromClones() {}
	std::string AllocateNet(int no_batches, bool &was_failure, bool print_graph = false) {
		was_failure = true;
		if (func_list_.empty()) return "AllocateNet error: 0 depth net.";
		if (batch_) return "Net already initialised on GPU.";
		if (print_graph) std::cout << toString();
		try {
			was_failure = !allocateOnGpu(no_batches);
		} catch (const std::exception &e) {
			return std::string("AllocateNet error: ") + e.what();
		}
		return was_failure ? "AllocateNet error" : "Allocated";
	}
	// forward + backward + update of one batch, replayed from ONE recorded graph: a step at small batch sizes is bound by
	// the cost of launching ~20 kernels one by one, not by the kernels.  The first call with each buffer of the data input
	// runs the three phases as usual (which also sizes the library's workspace), the second records them, later ones
	// replay; a change of the learning rate records again.  Same kernels, same arguments, same results as
	// gpuForward / gpuBackward / gpuUpdateInputs; the losses of the step are read with getLoss() whenever they are wanted
	// (every call of it waits for the device).
	void gpuTrainStep(InputFunc *inp, OutputFunc *outp, InputBatch &batch, float l_rate) {
		if (use_graphs_) throw std::logic_error("gpuTrainStep records the whole step itself: call useGraphs(false) first");
		feedBatch(inp, outp, batch);
		settleUploads();  // the recording below cannot hold a wait for the upload stream
		StepGraphs &g = graphs_[active_];
		// every step of this loop, queued or replayed, leaves its losses in the device buffer and decides what can wait the
		// way a recording does
		struct InStep {
			bool &flag;
			explicit InStep(bool &f) : flag(f) { flag = true; }
			~InStep() { flag = false; }
		} in_step(in_train_step_);
		auto eager = [&] {
			const bool was = use_graphs_;
			use_graphs_ = false;  // the phases launch (or record) their kernels themselves
			try {
				GpuForward();
				gpuBackward();
				gpuUpdateInputs(l_rate);
			} catch (...) {
				use_graphs_ = was;
				throw;
			}
			use_graphs_ = was;
		};
		// an update that also clears a first moment is not what a recording replays, nor is a step that finds gradients of
		// an earlier backward pass waiting for their update
		if (input_dz_dirty_ || !g.step_warm || !allCleanNonePending()) {
			eager();
			g.step_warm = true;
			return;
		}
		const bool real_now = anyRealTransformNow();
		if (g.step && (g.step_lr != l_rate || g.step_real != real_now)) {
			ck(cnet_graph_destroy(g.step), "cnet_graph_destroy");
			g.step = NULL;
		}
		g.step_real = real_now;
		if (!g.step) {
			ck(cnet_graph_begin(), "cnet_graph_begin");
			try {
				eager();
			} catch (...) {
				cnet_graph_end(NULL);
				throw;
			}
			ck(cnet_graph_end(&g.step), "cnet_graph_end");
			g.step_lr = l_rate;
		}
		ck(cnet_graph_launch(g.step), "cnet_graph_launch");
		for (auto f : inputs_) {  // what the steps inside the recording do to the host's picture of the inputs
			if (!f->trainable_) continue;
			f->z_imag_zero_ = false;
			if (!lazyEligible(f)) dataValuesWritten(f);  // stepped inside the recording
			if (lazyEligible(f)) {  // the recording was made in the usual state: its backward pass and update left these out
				for (auto c : f->next_func_)
					if (lazyKind(f, c)) c->lazy_owed_ = true;
				f->lazy_bwd_ = f->lazy_upd_ = true;
				f->lazy_lr_ = l_rate;
			}
		}
	}

private:
	// a batch for the main data input: switch to the buffer it was sent ahead to (gpuPrefetch), or copy it now
	void feedBatch(InputFunc *inp, OutputFunc *outp, InputBatch &batch) {
		requireAllocated("gpuForward");
		CInput *cin = dynamic_cast<CInput *>(inp);
		if (!cin) throw std::invalid_argument("gpuForward: this type of input is not supported with an InputBatch");
		if (cin != main_input_) throw std::invalid_argument("gpuForward: not the main input of the allocated net");
		if (batch.size() != batch_ || batch.noOfLabels() != batch_) throw std::invalid_argument("gpuForward: batch size differs from allocateOnGpu");
		if (batch.sampleDim() != cin->input().length_) throw std::invalid_argument("gpuForward: sample dimension differs from the input length");
		(void) outp;
		beforeFeed(cin);
		CFunc::Slot &s = cin->slots_[0];
		Stage &staged = stage_[nextStage()];
		if (staged.holds == &batch && staged.deferred) {  // nothing was sent ahead: the direct path below copies it on the compute stream
			staged.holds = NULL;
			staged.deferred = false;
		}
		if (staged.holds == &batch) {
			// the batch was sent ahead by gpuPrefetch(): switch the data input to the buffer it landed in.  Everything
			// queued so far may still read the buffer in use, so its retirement point is remembered for the next refill.
			checkLabels(batch.labelsPtr(), batch_);
			ck(cnet_compute_wait_ticket(staged.upload_ticket), "cnet_compute_wait_ticket");  // this batch's copies, nothing later
			ck(cnet_mark_compute(active_), "cnet_mark_compute");
			active_ = nextStage();
			staged.holds = NULL;
			cin->out_ = staged.z;
			s.z = staged.z;
			cin->z_imag_zero_ = staged.imag_zero;
			d_labels_ = staged.labels;
			labels_.assign(batch.labelsPtr(), batch.labelsPtr() + batch_);
			batch_labels_ = true;
			lossGradientsStale();
			return;
		}
		const size_t plane = (size_t) batch_ * s.len * sizeof(float);
		// one copy for both planes, which are one array here and there (upstream: two small copies per sample,
		// gpu/gpu_func.h:403-419)
		// (a batch of real samples sends its real plane only; the imaginary plane is cleared on the device)
		const bool real_only = batch.imagIsZero() && !send_zero_planes_;
		Stage &here = stage_[active_];
		const bool clear_imag = real_only && !here.imag_dev_zero;  // unless the plane is still clear from the last batch
		bool labels_set = false;
		if (gatherOnCompute(batch, plane)) {
			// the rows and their labels by one short kernel on the compute stream, behind the kernels that still read this buffer
			const DeviceDataset &ds = *batch.resident_;
			const size_t floats = (size_t) batch_ * s.len;
			checkLabels(batch.labelsPtr(), batch_);
			if (clear_imag) ck(cnet_memset_zero(s.z + floats, plane), "cnet_memset_zero");
			ck(cnet_gather_rows(s.z, s.len, (int64_t) floats, ds.z_, ds.dim_, (int64_t) ds.count_ * ds.dim_, ds.planes_, ds.count_, batch.indices_, d_labels_,
					ds.labels_dev_, batch_, s.len), "cnet_gather_rows");
			if (!real_only && ds.planes_ == 1) ck(cnet_memset_zero(s.z + floats, plane), "cnet_memset_zero");
			ck(cnet_copy_ticket(0, &batch.ticket_), "cnet_copy_ticket");
			labels_.assign(batch.labelsPtr(), batch.labelsPtr() + batch_);
			batch_labels_ = true;
			lossGradientsStale();
			labels_set = true;
		} else if (batch.resident_) {
			// The samples are on the device already: the upload stream, behind everything queued on the compute stream so far
			// (which may still read this buffer), copies the rows named by the indices; the compute stream waits for that.
			const DeviceDataset &ds = *batch.resident_;
			const size_t floats = (size_t) batch_ * s.len;
			ck(cnet_upload_wait_compute(), "cnet_upload_wait_compute");
			if (clear_imag) ck(cnet_upload_zero(s.z + floats, plane), "cnet_upload_zero");
			ck(cnet_upload_gather_rows(s.z, s.len, (int64_t) floats, ds.z_, ds.dim_, (int64_t) ds.count_ * ds.dim_, ds.planes_, ds.count_, batch.indices_,
					NULL, NULL, batch_, s.len), "cnet_upload_gather_rows");
			// a data set of real samples fills the real plane only; sendZeroPlanes has nothing to send here
			if (!real_only && ds.planes_ == 1) ck(cnet_upload_zero(s.z + floats, plane), "cnet_upload_zero");
			ck(cnet_copy_ticket(1, &batch.ticket_), "cnet_copy_ticket");
			ck(cnet_compute_wait_ticket(batch.ticket_), "cnet_compute_wait_ticket");
		} else if (batch.isPinned()) {
			ck(cnet_memcpy_h2d_async(s.z, batch.realDataPtr(), real_only ? plane : 2 * plane), "cnet_memcpy_h2d_async");
			if (clear_imag) ck(cnet_memset_zero(s.z + (size_t) batch_ * s.len, plane), "cnet_memset_zero");
			ck(cnet_copy_ticket(0, &batch.ticket_), "cnet_copy_ticket");
		} else {
			ck(cnet_memcpy_h2d(s.z, batch.realDataPtr(), real_only ? plane : 2 * plane), "cnet_memcpy_h2d");
			if (clear_imag) ck(cnet_memset_zero(s.z + (size_t) batch_ * s.len, plane), "cnet_memset_zero");
		}
		here.imag_dev_zero = batch.imagIsZero();  // zeros on the device, cleared there (now or earlier) or sent
		cin->z_imag_zero_ = batch.imagIsZero();
		if (!labels_set) setLabels(batch.labelsPtr(), batch_);
	}

public:
	// Send the NEXT batch to the device on the upload stream while the kernels of the current step run; the later
	// gpuForward(inp, outp, batch) with the same batch object then only switches buffers.  The data input is double
	// buffered on the device (the second buffer is allocated on the first call); at most one batch can be staged.  The
	// batch must be page-locked (built after the device library was initialised) and must not be refilled before its
	// gpuForward; clear() / add() on it wait for the copy.
	void gpuPrefetch(InputFunc *inp, InputBatch &batch) {
		requireAllocated("gpuPrefetch");
		CInput *cin = dynamic_cast<CInput *>(inp);
		if (!cin || cin != main_input_) throw std::invalid_argument("gpuPrefetch: not the main input of the allocated net");
		if (batch.size() != batch_ || batch.noOfLabels() != batch_ || batch.sampleDim() != cin->input().length_)
			throw std::invalid_argument("gpuPrefetch: batch shape differs from the allocated net");
		if (!batch.isPinned() && !batch.resident_) throw std::invalid_argument("gpuPrefetch: the batch is not in page-locked memory");
		checkLabels(batch.labelsPtr(), batch_);
		const int other = nextStage();
		Stage &st = stage_[other];
		if (st.holds) throw std::logic_error("gpuPrefetch: a staged batch is still waiting for its gpuForward");
		CFunc::Slot &s = cin->slots_[0];
		const size_t plane = (size_t) batch_ * s.len;
		if (gatherOnCompute(batch, plane * sizeof(float))) {  // nothing to send ahead: gpuForward copies the rows itself
			st.holds = &batch;
			st.deferred = true;
			return;
		}
		if (!st.z) {
			st.z = dalloc<float>(2 * plane);
			st.labels = dalloc<int32_t>(batch_);
		}
		if (!batch.resident_) {
			if (!st.host_labels) {
				void *h = NULL;
				ck(cnet_host_alloc(batch_ * sizeof(int32_t), &h), "cnet_host_alloc");
				st.host_labels = (int32_t *) h;
			}
			if (st.labels_ticket >= 0) ck(cnet_copy_wait(st.labels_ticket), "cnet_copy_wait");  // the previous copy has left host_labels
			std::copy(batch.labelsPtr(), batch.labelsPtr() + batch_, st.host_labels);
		}
		ck(cnet_upload_wait_marker(other), "cnet_upload_wait_marker");  // kernels of the step that last used this buffer
		// the two planes of a batch are one array on the host and on the device: one copy for both
		st.imag_zero = batch.imagIsZero();
		const bool real_only = st.imag_zero && !send_zero_planes_;
		// the plane is still clear when the last batch that landed here was real and nothing has stepped the values since
		if (real_only && !st.imag_dev_zero) ck(cnet_upload_zero(st.z + plane, plane * sizeof(float)), "cnet_upload_zero");
		if (batch.resident_) {
			// the samples and their labels are on the device already: one launch copies the rows that the indices name
			const DeviceDataset &ds = *batch.resident_;
			ck(cnet_upload_gather_rows(st.z, s.len, (int64_t) plane, ds.z_, ds.dim_, (int64_t) ds.count_ * ds.dim_, ds.planes_, ds.count_, batch.indices_,
					st.labels, ds.labels_dev_, batch_, s.len), "cnet_upload_gather_rows");
			if (!real_only && ds.planes_ == 1) ck(cnet_upload_zero(st.z + plane, plane * sizeof(float)), "cnet_upload_zero");
		} else {
			// the samples and their labels: one launch for a small batch, two queued copies for a large one
			ck(cnet_upload_pair(st.z, batch.realDataPtr(), (real_only ? 1 : 2) * plane * sizeof(float), st.labels, st.host_labels,
					batch_ * sizeof(int32_t)), "cnet_upload_pair");
		}
		st.imag_dev_zero = st.imag_zero;
		// one recorded point serves the host (the batch may be refilled, the staging of the labels reused) and the compute
		// stream (the forward pass of this batch)
		ck(cnet_copy_ticket(1, &batch.ticket_), "cnet_copy_ticket");
		st.upload_ticket = batch.ticket_;
		st.labels_ticket = batch.ticket_;
		st.holds = &batch;
	}
	// upload a batch into a CInput flagged with setIsBatched(true); labels of that batch are ignored
	void gpuSetInput(CInput *cin, InputBatch &batch) {
		requireAllocated("gpuSetInput");
		if (cin->rows_ != batch_ || batch.size() != batch_ || batch.sampleDim() != cin->input().length_)
			throw std::invalid_argument("gpuSetInput: " + cin->getName() + " is not a data input of this batch shape");
		if (batch.isResident())
			throw std::invalid_argument("gpuSetInput: a batch that names samples of a data set on the device feeds the main data input only (gpuForward / gpuPrefetch)");
		beforeFeed(cin);
		CFunc::Slot &s = cin->slots_[0];
		const size_t plane = (size_t) batch_ * s.len * sizeof(float);
		const bool real_only = batch.imagIsZero() && !send_zero_planes_;
		if (batch.isPinned() && !use_graphs_) {
			// On the upload stream, behind everything queued on the compute stream so far (the kernels that still use the
			// previous contents); the compute stream waits for it only in front of the first kernel that touches this
			// input, so the copy travels under the layers of the forward pass that come before it.
			ck(cnet_upload_wait_compute(), "cnet_upload_wait_compute");
			ck(cnet_upload_async(s.z, batch.realDataPtr(), real_only ? plane : 2 * plane), "cnet_upload_async");
			if (real_only) ck(cnet_upload_zero(s.z + (size_t) batch_ * s.len, plane), "cnet_upload_zero");
			ck(cnet_copy_ticket(1, &batch.ticket_), "cnet_copy_ticket");
			in_flight_.push_back(cin);
		} else if (batch.isPinned()) {  // queued behind the kernels that still read the previous contents; the host does not wait
			ck(cnet_memcpy_h2d_async(s.z, batch.realDataPtr(), real_only ? plane : 2 * plane), "cnet_memcpy_h2d_async");
			if (real_only) ck(cnet_memset_zero(s.z + (size_t) batch_ * s.len, plane), "cnet_memset_zero");
			ck(cnet_copy_ticket(0, &batch.ticket_), "cnet_copy_ticket");
		} else {
			ck(cnet_memcpy_h2d(s.z, batch.realDataPtr(), real_only ? plane : 2 * plane), "cnet_memcpy_h2d");
			if (real_only) ck(cnet_memset_zero(s.z + (size_t) batch_ * s.len, plane), "cnet_memset_zero");
		}
		cin->z_imag_zero_ = batch.imagIsZero();
		if (cin == main_input_) stage_[active_].imag_dev_zero = batch.imagIsZero();  // cleared or sent just now
	}
	bool gpuForward(InputFunc *inp, OutputFunc *outp, EmbeddingBatch &batch) {
		feedTokens(inp, outp, batch);
		return GpuForward();
	}
	void feedTokens(InputFunc *inp, OutputFunc *outp, EmbeddingBatch &batch) {
		requireAllocated("gpuForward");
		CEmbedding *emb = dynamic_cast<CEmbedding *>(inp);
		if (!emb || emb != main_input_) throw std::invalid_argument("gpuForward: the EmbeddingBatch needs the main CEmbedding input");
		if (batch.size() != batch_ || batch.noOfLabels() != batch_ || batch.sampleDim() != emb->no_out_tokens_)
			throw std::invalid_argument("gpuForward: batch shape differs from the allocated net");
		(void) outp;
		uploadTokens(emb, batch.tokensPtr());
		setLabels(batch.labelsPtr(), batch_);
	}
	bool GpuForward() {
		requireAllocated("GpuForward");
		materializeLazy();  // a forward pass on values that were not replaced reads what the update made of them
		if (use_graphs_) settleUploads();  // a recording cannot hold the wait
		{
			StepGraphs &g = graphs_[active_];  // a recording holds one of the two transforms of a data input
			const bool real_now = anyRealTransformNow();
			if (g.fwd && g.fwd_real != real_now) {
				ck(cnet_graph_destroy(g.fwd), "cnet_graph_destroy");
				g.fwd = NULL;
			}
			g.fwd_real = real_now;
		}
		runPhase(0, graphs_[active_].fwd, [&] {
			for (auto f : func_list_) {
				if (readsInFlight(f)) settleUploads();
				nodeForward(f);
			}
		});
		settleUploads();
		return true;
	}
	// spellings of upstream GpuNet (gpu/gpu_func.h:645-681).  GpuInfer is upstream's forward pass without the clearing of
	// gradients; no forward pass clears gradients here (the first contribution of a backward pass overwrites), so it is
	// the same pass.  GpuBackward's label applies when no batch has supplied labels, as upstream's does.
	std::string GpuForward(bool &was_failure) {
		was_failure = !GpuForward();
		return "";
	}
	std::string GpuInfer(bool &was_failure) { return GpuForward(was_failure); }
	std::string GpuBackward(int label, bool &was_failure) {
		requireAllocated("GpuBackward");
		if (!batch_labels_) {
			std::vector<int> all(batch_, label);
			setLabels(all.data(), batch_, false);
			for (auto f : outputs_)  // the loss on the device follows the label in use
				if (f->typeId() == isCrossEntropy) nodeForward(f);
		}
		was_failure = !gpuBackward();
		return "";
	}
	bool gpuBackward() {
		requireAllocated("gpuBackward");
		settleUploads();
		planGradients();
		materializeLazy();  // this pass overwrites the gradients a transform left out would start from
		flushPending();     // ... and the planes a deferred gradient sits in
		const bool nominal = planDeferral(true);
		auto body = [&] {
			gather_src_.clear();  // nothing is left over from a pass that threw
			gather_dst_.clear();
			gather_len_.clear();
			for (int k = (int) func_list_.size() - 1; k >= 0; --k) nodeBackward(func_list_[k], true);
			flushGathers();
		};
		// a recording stands for the usual state (every gradient deferred); a second pass before an update runs as it is
		if (nominal) runPhase(1, graphs_[active_].bwd, body);
		else body();
		noteDeferred();
		return true;
	}
	// z -= l_rate * dzs on every input function (the data input too, impl/cnet.h:413-421), then its gradients are cleared
	void gpuUpdateInputs(float l_rate) {
		requireAllocated("gpuUpdateInputs");
		settleUploads();
		StepGraphs &g = graphs_[active_];
		if (g.upd && g.upd_lr != l_rate) {  // the rate is frozen into a recording
			ck(cnet_graph_destroy(g.upd), "cnet_graph_destroy");
			g.upd = NULL;
		}
		g.upd_lr = l_rate;
		if (input_dz_dirty_) materializeLazy();  // the first moment of every input function is cleared here: all of them take part
		saveWeightsOwed();  // before the launch below changes them
		if (input_dz_dirty_)  // this update also clears the first moment: not what a recording made without it does
			for (auto &sg : graphs_)
				if (sg.upd) {
					ck(cnet_graph_destroy(sg.upd), "cnet_graph_destroy");
					sg.upd = NULL;
				}
		auto body = [&] {
			// every input function in one launch (two when some gradients are still with their consumers: those are read
			// there and nothing has to be cleared); the dz planes only hold something after an Adam-style step (its first
			// moment), so they are cleared only then
			for (int deferred = 0; deferred < 2; ++deferred) {
				std::vector<float *> zr, zi, dr, di;
				std::vector<int64_t> len;
				for (auto f : inputs_) {
					if (!f->trainable_ || f->lazy_bwd_ || (f->pending_ != NULL) != (deferred != 0)) continue;
					CFunc::Slot &s = f->slots_[0];
					const CFunc::Slot &gsrc = deferred ? *f->pending_ : s;
					const size_t n = (size_t) s.rows * s.len;
					zr.push_back(s.z);
					zi.push_back(s.z + n);
					dr.push_back(gsrc.g(2));
					di.push_back(gsrc.g(3));
					len.push_back((int64_t) n);
					if (input_dz_dirty_) ck(cnet_memset_zero(s.g(0), 2 * n * sizeof(float)), "zero");
				}
				if (zr.empty()) continue;
				ck(cnet_sgd_update_multi((int) zr.size(), zr.data(), zi.data(), dr.data(), di.data(), len.data(), l_rate, deferred ? 0 : 1),
						"cnet_sgd_update_multi");
			}
		};
		// a recording stands for the usual state: every gradient that can be is still with its consumer
		if (allPending()) runPhase(2, g.upd, body);
		else body();
		for (auto f : inputs_) {
			if (!f->trainable_) continue;
			if (!f->lazy_bwd_) dataValuesWritten(f);  // stepped by the launch above (or by its replay)
			if (f->lazy_bwd_ && !f->lazy_upd_) {  // its step waits with its backward pass
				f->lazy_upd_ = true;
				f->lazy_lr_ = l_rate;
			}
			f->pending_ = NULL;
			f->grad_clean_ = true;
			f->z_imag_zero_ = false;  // stepped: complex from here on
		}
		input_dz_dirty_ = false;
	}
	// Replay the kernels of GpuForward / gpuBackward / gpuUpdateInputs from recorded graphs instead of launching them
	// one by one (a step at small batch sizes is bound by launch overhead).  Each phase runs once as usual after this
	// call (which also sizes the library's workspace), is recorded on its next call and replayed from then on; there is
	// one recording per phase and per buffer of the data input.  Same kernels, same arguments, same results.
	void useGraphs(bool on) {
		requireAllocated("useGraphs");
		if (!on) dropGraphs();
		lossGradientsStale();  // a recorded backward pass holds the loss's own backward kernel
		if (on != use_graphs_) materializeLazy();  // what may wait differs between the two ways of running a pass
		use_graphs_ = on;
	}
	bool usingGraphs() const { return use_graphs_; }
	// Every backward pass starts at a CrossEntropy or an L2Out, whose loss is real: the gradient with respect to z* is then
	// the conjugate of the gradient with respect to z at every node, and the matrix products of Linear, FourierTrans and
	// TriangFourier compute the dz half only and write its conjugate to the dz* planes (half the matrix work of a backward
	// pass; same results to rounding).  Off: both halves are computed, as upstream does.  Recordings are dropped, since
	// they hold the kernels of the other setting.
	void conjugateGradients(bool on) {
		if (on != conjugate_gradients_ && batch_) {
			dropGraphs();
			materializeLazy();  // with the kernels of the setting the backward pass ran under
			lossGradientsStale();
		}
		conjugate_gradients_ = on;
	}
	bool conjugateGradients() const { return conjugate_gradients_; }
	// The block kernels of the matrix products (Linear, FourierTrans, TriangFourier; forward and backward) form a complex
	// product from three real ones instead of four (cnet_cgemm_set_products): a quarter of the matrix work less, the
	// imaginary parts rounded against the size of the whole entry instead of their own.  A setting of the device library,
	// shared by every net of the process; off unless CNET_CGEMM_3M=1 is in the environment.  Recordings of this net are
	// dropped, since they hold the kernels of the other setting.
	void threeProductGemm(bool on) {
		if (on != threeProductGemm() && batch_) {
			dropGraphs();
			materializeLazy();  // with the kernels of the setting the backward pass ran under
		}
		ck(cnet_cgemm_set_products(on ? 3 : 4), "cnet_cgemm_set_products");
	}
	bool threeProductGemm() const { return cnet_cgemm_get_products() == 3; }
	// Neighbouring layers that run as one kernel where the device layer has one (Hadamard or Linear followed by CGelu): same bits,
	// fewer passes over memory and fewer launches.  Off: one launch per layer.  Takes effect at the next allocateOnGpu,
	// or at once when the net is allocated (recordings are dropped).
	void fuseLayers(bool on) {
		if (on == fuse_layers_) return;
		fuse_layers_ = on;
		if (batch_) {
			dropGraphs();
			planFusion();
		}
	}
	bool fusingLayers() const { return fuse_layers_; }
	// A batch all of whose samples are real (InputBatch::imagIsZero: images, for instance) sends its real plane only and
	// the imaginary plane of the data input is cleared on the device: half the bytes over the link, the same values on
	// the device.  On: the plane of zeros travels like any other.
	void sendZeroPlanes(bool on) { send_zero_planes_ = on; }
	// The normalised rows of a CrossEntropy (its output values upstream, impl/crossent.h:38-59) are read by nothing on the
	// device.  By default the forward pass leaves them out and `fetch` writes them when asked (same kernel, same values);
	// off: every forward pass writes them.  At 8192 rows of 32768 the forward pass of the loss takes 0.33 instead of 1.27 ms.
	void lazyLossRows(bool on) { lazy_loss_rows_ = on; }
	// The loss kernels of a forward pass that is launched kernel by kernel store the per-row losses straight into page-locked
	// host memory (see OutLoss): getLoss and gpuQueueLoss then queue no copy.  Off: the losses stay in a device buffer and are
	// copied when asked for, as in a recorded forward pass.  Same values either way.
	void hostLosses(bool on) { host_losses_ = on; }
	// A FourierTrans applied to a data input that was fed real samples computes half of its columns and writes the others
	// as their conjugates (cnet_cdft_fwd_real_input); off: the whole product, whatever the samples.  Same values to rounding.
	void realTransforms(bool on) {
		if (on != real_transforms_ && batch_) dropGraphs();
		real_transforms_ = on;
	}
	// An input function with one consumer leaves the gradient of a backward pass in that consumer's planes until the update
	// reads it there (nothing is added to cleared planes and cleared again).  Off: every backward pass adds it to the input
	// function's own planes at once, as upstream does.  Same weights to the bit either way.
	void deferGathers(bool on) {
		if (on == defer_gathers_) return;
		if (batch_) {
			dropGraphs();
			materializeLazy();
			flushPending();
		}
		defer_gathers_ = on;
	}
	// A data input that feeds a FourierTrans or TriangFourier and nothing else: the backward pass of the transform and the
	// gather and step of the input (upstream steps data inputs like parameters, impl/cnet.h:413-421) produce values that
	// the next batch overwrites.  By default they are left out and done only if something looks first (fetch,
	// getInputsFromGpu, a forward pass on the same values, a second backward pass, an Adam-style step, the per-sample
	// calls), from the gradients the transform's consumers left; a new batch drops them.  Off: done at once, as upstream
	// does.  Same observable values either way.
	void lazyDataInputs(bool on) {
		if (on == lazy_inputs_) return;
		if (batch_) {
			dropGraphs();
			materializeLazy();
		}
		lazy_inputs_ = on;
	}
	// Upstream steps every input function, the data input included (impl/cnet.h:413-421), and therefore runs the backward
	// pass all the way down to it.  An input function marked not trainable is left alone by gpuUpdateInputs /
	// gpuAdamUpdate, gathers nothing, and the backward products that would only serve it are not computed (for the
	// 784 -> 10 net: the whole backward pass of the FourierTrans).  Losses and the steps of the other input functions are
	// unchanged to the bit.  Recordings are dropped.
	void setInputTrainable(InputFunc *inp, bool on) {
		CFunc *f = dynamic_cast<CFunc *>(inp);
		if (!f || !f->is_input_) throw std::invalid_argument("setInputTrainable: not an input function of this net");
		if (f->trainable_ != on && batch_) {
			dropGraphs();
			materializeLazy();
			flushPending();
		}
		f->trainable_ = on;
	}
	// The Adam-style step of upstream GpuNet::adamUpdate (gpu/gpu_func.h:503-510, gpu/kernels.cpp:494-514) on every input
	// function: the first moment lives in the node's dz planes, dz* is cleared, dz is kept.
	void gpuAdamUpdate(float l_rate, float beta, int t) {
		requireAllocated("gpuAdamUpdate");
		materializeLazy();
		for (auto f : inputs_) {
			if (!f->trainable_) continue;
			CFunc::Slot &s = f->slots_[0];
			const size_t n = (size_t) s.rows * s.len;
			float *z = s.z;
			const CFunc::Slot &gsrc = f->pending_ ? *f->pending_ : s;  // a gradient still with its consumer is read there
			ck(cnet_adam_update(z, z + n, s.g(0), s.g(1), gsrc.g(2), gsrc.g(3), (int64_t) n, l_rate, beta, t, f->pending_ ? 0 : 1),
					"cnet_adam_update");
			dataValuesWritten(f);
			f->pending_ = NULL;
			f->grad_clean_ = true;
			f->z_imag_zero_ = false;
		}
		input_dz_dirty_ = true;
	}
	float getLoss(OutputFunc *outp, Batch *batch) {
		requireAllocated("getLoss");
		CFunc *f = dynamic_cast<CFunc *>(outp);
		OutLoss *l = lossOf(f);
		if (!l) throw std::invalid_argument("getLoss: not supported for this output");
		std::vector<float> tmp(f->rows_);
		readLoss(*l, tmp.data(), 0, f->rows_);
		float loss = 0.f;
		for (float v : tmp) {
			loss += v;
			if (batch) batch->addLoss(v);
		}
		return loss / tmp.size();
	}
	// The same read in two halves, so that a training loop never waits for the step it has just queued: gpuQueueLoss sends
	// the per-row losses of the forward pass that was queued last to page-locked memory without waiting; getLoss(pending)
	// waits for that copy alone, typically one step later, when it has long arrived.  The host can then queue step k+1
	// before it looks at the loss of step k, and the device never runs dry between steps.  Up to kLossSlots reads may be
	// pending; an older one is overwritten.
	static constexpr int kLossSlots = OutLoss::kSlots;
	struct PendingLoss {
		int64_t ticket = -1, serial = -1;
		int rows = 0;
		const OutLoss *direct = NULL;  // the forward pass wrote to that output's own ring (serial counts its forward passes)
	};
	PendingLoss gpuQueueLoss(OutputFunc *outp) {
		requireAllocated("gpuQueueLoss");
		CFunc *f = dynamic_cast<CFunc *>(outp);
		OutLoss *l = lossOf(f);
		if (!l) throw std::invalid_argument("gpuQueueLoss: not supported for this output");
		PendingLoss p;
		p.rows = f->rows_;
		if (l->cur_on_host) {  // already on its way: the kernel stores into page-locked memory; only the point in the stream is marked
			p.serial = l->serial;
			p.direct = l;
			ck(cnet_copy_ticket(0, &p.ticket), "cnet_copy_ticket");
			return p;
		}
		if (!loss_ring_) {
			void *h = NULL;
			ck(cnet_host_alloc((size_t) kLossSlots * batch_ * sizeof(float), &h), "cnet_host_alloc");
			loss_ring_ = (float *) h;
		}
		p.serial = loss_queued_++;
		ck(cnet_memcpy_d2h_async(loss_ring_ + (size_t) (p.serial % kLossSlots) * batch_, l->dev, (size_t) p.rows * sizeof(float)),
				"cnet_memcpy_d2h_async");
		ck(cnet_copy_ticket(0, &p.ticket), "cnet_copy_ticket");
		return p;
	}
	float getLoss(const PendingLoss &p, Batch *batch) {
		if (p.serial < 0 || (p.direct ? !p.direct->host : !loss_ring_)) throw std::logic_error("getLoss: nothing was queued under this handle");
		if ((p.direct ? p.direct->serial - p.serial + 1 : loss_queued_ - p.serial) > kLossSlots)
			throw std::logic_error("getLoss: the queued losses were overwritten by later ones");
		ck(cnet_copy_wait(p.ticket), "cnet_copy_wait");
		const float *v = p.direct ? p.direct->host + (size_t) (p.serial % kLossSlots) * p.direct->rows
								  : loss_ring_ + (size_t) (p.serial % kLossSlots) * batch_;
		float loss = 0.f;
		for (int b = 0; b < p.rows; ++b) {
			loss += v[b];
			if (batch) batch->addLoss(v[b]);
		}
		return loss / p.rows;
	}
	// upstream GpuNet::getLoss(int label) (gpu/gpu_func.h:928-969): the loss of every output function, keyed by uid.
	// Upstream has one entry per clone, i.e. per batch row, each clone under a uid of its own; there are no clones here,
	// so an output's entry is the loss of batch row 0, which is the entry upstream's tests read (tests/gputests.h:64,
	// 416, 456).  Per-row losses come from getLoss(outp, &batch).  As upstream, the label of the batch wins over the
	// argument, and the CrossEntropy loss is formed on the host from z_label and S: -log(max(|z_label|^2 / S, 1e-15)).
	std::map<int, float> getLoss(int label) {
		requireAllocated("getLoss");
		std::map<int, float> ret;
		for (auto f : outputs_) {
			if (f->typeId() == isL2Out) {
				float v = 0.f;
				readLoss(((L2Out *) f)->loss_, &v, 0, 1);
				ret[f->uid()] = v;
			} else if (f->typeId() == isCrossEntropy) {
				const int lab = batch_labels_ ? labels_[0] : label;
				if (lab < 0 || lab >= f->input().length_) throw std::out_of_range("getLoss: label outside the CrossEntropy input");
				const float S = rowZeroOfCrossEntropy((CrossEntropy *) f);
				float prob = std::norm(f->input().z(lab)) / S;
				prob = (prob < 1e-15 ? 1e-15 : prob);
				ret[f->uid()] = -std::log(prob);
			}
		}
		return ret;
	}
	// upstream GpuNet::sample (gpu/gpu_func.h:971-1011): draws an index from the probabilities p_k = |z_k|^2 / S of the
	// first CrossEntropy output (batch row 0): the first k whose running sum of p reaches a uniform coin; if rounding
	// leaves the total below the coin, the most probable index.  0 for a net without a CrossEntropy output.
	int sample() {
		requireAllocated("sample");
		for (auto f : outputs_) {
			if (f->typeId() != isCrossEntropy) continue;
			const float S = rowZeroOfCrossEntropy((CrossEntropy *) f);
			const float coin = (float) rand_.randDouble();
			float c_val = 0.f, max = 0.f;
			int var_max = 0;
			for (int var = 0; var < f->input().length_; ++var) {
				const float p = std::norm(f->input().z(var)) / S;
				c_val += p;
				if (coin <= c_val) return var;
				if (max < p) {
					max = p;
					var_max = var;
				}
			}
			return var_max;
		}
		return 0;
	}
	void setRandSeed(uint64_t seed) { rand_ = SimpleRand(seed); }  // repeatable sample(); upstream seeds from clock()
	CFunc *findFirstOfType(int type_id) {  // impl/cnet.h:85-92
		for (auto f : func_list_)
			if (f->typeId() == type_id) return f;
		return NULL;
	}
	std::vector<int> getPredictions(OutputFunc *outp) {
		requireAllocated("getPredictions");
		CrossEntropy *c = dynamic_cast<CrossEntropy *>(outp);
		if (!c) throw std::invalid_argument("getPredictions: needs a CrossEntropy output");
		std::vector<int32_t> tmp(c->rows_);
		ck(cnet_memcpy_d2h(tmp.data(), c->d_argmax_, tmp.size() * sizeof(int32_t)), "cnet_memcpy_d2h");
		return std::vector<int>(tmp.begin(), tmp.end());
	}
	void checkLabels(const int *labels, int count) {
		if (count != batch_) throw std::invalid_argument("setLabels: one label per batch row");
		for (auto f : outputs_)
			if (f->typeId() == isCrossEntropy)
				for (int k = 0; k < count; ++k)
					if (labels[k] < 0 || labels[k] >= f->input().length_) throw std::out_of_range("setLabels: label outside the CrossEntropy input");
	}
	void setLabels(const int *labels, int count, bool from_batch = true) {
		requireAllocated("setLabels");
		checkLabels(labels, count);
		labels_.assign(labels, labels + count);
		batch_labels_ = from_batch;
		lossGradientsStale();
		ck(cnet_memcpy_h2d(d_labels_, labels, count * sizeof(int32_t)), "cnet_memcpy_h2d");
	}
	void sync() { ck(cnet_sync(), "cnet_sync"); }

	// upstream CNet::save / restore (gpu/gpu_func.h:1103-1111); defined in model_saver.hpp
	bool save(std::string file);
	bool restore(std::string file);

	// ---- per-sample API of upstream (CNet::forward / backward / updateInputs, gpu/gpu_func.h:1046-1056, 497-501):
	//      host views are the state, the arithmetic runs on the device with a batch of one ----
	void forward() { forwardOneSample(true); }
	// ComplexNet::infer (impl/cnet.h:379-389): the forward pass alone, the gradients stay as they are
	void infer() { forwardOneSample(false); }
	// ComplexNet::update (impl/cnet.h:413-421): a step at learning_rate / batch_size that also clears the inputs' gradients
	void update(float learning_rate, int batch_size) { updateInputs(learning_rate / batch_size); }
	void forwardOneSample(bool clear_gradients) {
		if (!batch_) allocateOnGpu(1);
		if (batch_ != 1) throw std::logic_error("forward(): the per-sample API needs allocateOnGpu(1); use gpuForward for batches");
		copyInputsToGpu();
		// upstream forward() clears the gradients of every non-input function (impl/cnet.h:372-374); the batched path
		// never needs that (first contribution overwrites), the per-sample views do
		materializeLazy();
		flushPending();  // before the planes a deferred gradient sits in are cleared
		if (clear_gradients)
			for (auto f : func_list_)
				if (!f->is_input_)
					for (auto &s : f->slots_) ck(cnet_memset_zero(s.grad, 4 * (size_t) s.rows * s.len * sizeof(float)), "zero");
		lossGradientsStale();
		per_sample_call_ = true;
		try {
			GpuForward();
		} catch (...) {
			per_sample_call_ = false;
			throw;
		}
		per_sample_call_ = false;
		fetchAll(0);
	}
	void backward(int label) {
		if (batch_ != 1) throw std::logic_error("backward(): call forward() first");
		if (label >= 0) setLabels(&label, 1, false);
		// the label only enters the backward pass of CrossEntropy; its forward outputs do not depend on it except
		// the device-side loss, which is refreshed here so getLoss() matches the label in use
		per_sample_call_ = true;
		try {
			for (auto f : outputs_)
				if (f->typeId() == isCrossEntropy) nodeForward(f);
		} catch (...) {
			per_sample_call_ = false;
			throw;
		}
		per_sample_call_ = false;
		materializeLazy();
		flushPending();
		planDeferral(false);  // every host view is read right after the pass: nothing to gain from deferring
		gather_src_.clear();
		gather_dst_.clear();
		gather_len_.clear();
		for (int k = (int) func_list_.size() - 1; k >= 0; --k) nodeBackward(func_list_[k], label >= 0);
		flushGathers();
		noteDeferred();
		fetchAll(0);
	}
	void backward() { backward(-1); }
	void updateInputs(float l_rate) {
		if (batch_ != 1) throw std::logic_error("updateInputs(): call forward() first");
		gpuUpdateInputs(l_rate);
		for (auto f : inputs_) fetch(f, 0);
	}

	// per-sample twin of ComplexNet::adamUpdate (impl/cnet.h:423-431)
	void adamUpdate(float learning_rate, int batch_size, float beta, int t) {
		if (batch_ != 1) throw std::logic_error("adamUpdate(): call forward() first");
		gpuAdamUpdate(learning_rate / batch_size, beta, t);
		for (auto f : inputs_) fetch(f, 0);
	}

private:
	// brings row 0 of a CrossEntropy node's input to its host view and returns that row's clamped S = sum |z|^2
	float rowZeroOfCrossEntropy(CrossEntropy *c) {
		fetch(c, 0);
		float S = 0.f;
		ck(cnet_memcpy_d2h(&S, c->d_s_, sizeof(float)), "cnet_memcpy_d2h");
		return S < 1e-15 ? 1e-15 : S;
	}
	void uploadTokens(CEmbedding *e, const int *batch_tokens) {
		std::vector<int32_t> buf((size_t) e->rows_ * e->no_out_tokens_, NO_TOKEN);
		if (batch_tokens) {
			std::copy(batch_tokens, batch_tokens + buf.size(), buf.begin());
		} else {  // the per-sample token list of setInput(), in every row
			for (int b = 0; b < e->rows_; ++b) std::copy(e->tokens_.begin(), e->tokens_.end(), buf.begin() + (size_t) b * e->no_out_tokens_);
		}
		// upstream asserts id < no_embeddings in setInput (impl/embed.h:84-100); anything below zero is padding
		for (int32_t id : buf)
			if (id >= e->no_embeddings_) throw std::out_of_range("token id " + std::to_string(id) + " outside the embedding table of " + e->getName());
		ck(cnet_memcpy_h2d(e->d_tokens_, buf.data(), buf.size() * sizeof(int32_t)), "cnet_memcpy_h2d");
	}
};

#endif  // CNET_AMD_HOST_NET_HPP_
