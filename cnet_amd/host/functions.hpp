// cnet_amd/host/functions.hpp
// The graph node (upstream impl/cfunc.h) and the layer classes of the dense complex path.  The layer arithmetic lives in the
// device library; a node carries the wiring, the per-sample host view and its device planes.  Included by cnet.hpp (after
// batches.hpp).
#ifndef CNET_AMD_HOST_FUNCTIONS_HPP_
#define CNET_AMD_HOST_FUNCTIONS_HPP_

// ---------------------------------------------------------------------------------------------------------------
// impl/cfunc.h: graph node.  The layer arithmetic lives in the device library; a node here carries the wiring, the
// per-sample host view and its device planes.
// ---------------------------------------------------------------------------------------------------------------
class OutputFunc {
	bool isMainOutput_ = false;
public:
	virtual ~OutputFunc() {}
	virtual int outputLength() = 0;
	virtual float loss(int label) = 0;
	virtual Vars *mutableOutput() = 0;
	bool isMainOutput() { return isMainOutput_; }
	void setIsMainOutput(bool v) { isMainOutput_ = v; }
};

class InputFunc {
	bool isMainInput_ = false;
public:
	virtual ~InputFunc() {}
	bool isMainInput() { return isMainInput_; }
	void setIsMainInput(bool v) { isMainInput_ = v; }
};

// node type ids of impl/cnet.h:31-44
const int isHadamard = 1, isEmbedding = 2, isLinear = 3, isFourier = 4, isCrossEntropy = 5, isResidual = 6, isSoftMax = 7,
		isInput = 8, isCrelu = 9, isGelu = 10, isL2Out = 11, isTrianFourier = 12;
// not an upstream type (and not part of its .mod format): SeqFourierTrans below
const int isSeqFourier = 64;

class CFunc {
	friend class CNet;
	Vars input_;
protected:
	int uid_ = 0;
	int out_size_;
	std::vector<CFunc *> prev_func_, next_func_;  // not owned
	std::vector<int> offset_;
	int depth_ = 0;
	bool is_input_ = false, is_output_ = false;
	int type_ = 0;
	SimpleRand rand_;

	// ---- device side (owned by CNet's plan) ----
	struct Slot {            // one producer feeding this node
		CFunc *producer = NULL;
		int offset = 0, len = 0, rows = 0;
		float *grad = NULL;  // 4 planes [rows][len]
		float *z = NULL;     // input functions only: their own 2 value planes [rows][len] (the parameter, the data batch, the table)
		float *g(int plane) const { return grad + (size_t) plane * rows * len; }
		// Under conjugate gradient pairs (CNet::conjugateGradients) the dz* planes of a slot are written on the device only
		// where something reads them there: input functions and the embedding table gather dz*.  Elsewhere they are the
		// conjugate of the dz planes by construction and fetch() forms them on the host.
		bool star_on_device = true;
		float *gs(int plane) const { return star_on_device ? g(plane) : NULL; }
	};
	std::vector<Slot> slots_;
	bool trainable_ = true;   // input functions: stepped by the update (CNet::setInputTrainable)
	bool wants_grad_ = true;  // a trainable input function lies below this node: gradients have to flow through it
	// A Hadamard whose only consumer is a CGelu that feeds one consumer itself runs with it as one pass each way
	// (cnet_hadamard_cgelu_*): fused_next_ of the Hadamard names the CGelu, fused_prev_ of the CGelu is 2.  A Linear whose
	// only consumer is a CGelu applies it when it stores its product (cnet_clinear_cgelu_fwd): fused_prev_ of the CGelu is
	// 1, its backward pass runs as usual.
	CFunc *fused_next_ = NULL;
	int fused_prev_ = 0;
	// A FourierTrans whose only consumer is such a Hadamard with a shared weight row hands all three layers to one call
	// (cnet_cdft_hadamard_cgelu_fwd: one launch at small batches): fused_next_ of the transform names the Hadamard, and
	// fwd_by_producer_ of the Hadamard says that the transform of this forward pass has written its planes and the CGelu's.
	bool fwd_by_producer_ = false;
	// A narrow Linear whose operand is the CGelu of a Hadamard gate with a shared row takes the backward pass of that pair
	// into its own call (cnet_clinear_hadamard_cgelu_bwd_sym): bwd_by_consumer_now_ of the Hadamard is then set for the pass.
	bool bwd_by_consumer_now_ = false;
	// A Linear that feeds nothing but a CrossEntropy hands its product and the loss (forward pass and gradient) to one call
	// (cnet_clinear_cross_entropy_fwd_bwd_sym: one launch for a narrow head) whenever the loss would write its gradient from
	// its forward pass anyway: loss_next_ of the Linear names the CrossEntropy, whose fwd_by_producer_ is then set per pass.
	CFunc *loss_next_ = NULL;
	// A Residual one of whose operands (slot fused_gelu_slot_) is a CGelu that feeds nothing else runs the CGelu's backward
	// pass inside its own (cnet_residual_cgelu_bwd_sym) under conjugate gradient pairs; bwd_by_consumer_ of the CGelu is
	// set.  The gradient of that operand equals the gradient of the other one and is not stored a second time: fetch()
	// reads it from there.
	int fused_gelu_slot_ = -1;
	bool bwd_by_consumer_ = false;
	// Input functions with one consumer: the dz* of a backward pass is not added to the node's own planes at once.  While
	// those planes are clear (grad_clean_: nothing gathered since the last update) the gradient stays where the consumer's
	// backward pass wrote it (pending_), and the update reads it from there, which saves a pass that adds it to zeros and
	// the pass that clears it again.  Anything that looks at the node's planes or overwrites the consumer's first brings
	// them up to date (CNet::flushPending).  defer_now_ is the decision for the pass that is being queued.
	Slot *pending_ = NULL;
	bool grad_clean_ = false;
	bool defer_now_ = false;
	// input functions: the imaginary plane on the device is known to hold +0 only (a batch of real samples was fed and
	// nothing has stepped or overwritten the values since); a FourierTrans on it then takes cnet_cdft_fwd_real_input
	bool z_imag_zero_ = false;
	// Data inputs (one row per sample) that feed a FourierTrans / TriangFourier or the data operand of a Linear: the part
	// of that consumer's backward pass that only serves the data input (the whole backward pass of a transform, the
	// input-gradient product of a Linear), the gather and the update of the input are work whose results the next batch
	// overwrites.  They are left out (lazy_bwd_: a backward pass has skipped them; lazy_upd_: an update at rate lazy_lr_
	// has skipped them too) and done later, from the gradients the consumer's consumers left, if anything looks before the
	// next batch arrives (CNet::materializeLazy).  lazy_now_ (on the input) / lazy_skip_now_ (on the consumer) are the
	// decisions for the pass that is being queued; lazy_owed_ (on the consumer) says that a pass has skipped its share.
	// A Linear whose weights an update changes in the meantime keeps their old values in w_saved_ (w_saved_valid_).
	bool lazy_bwd_ = false, lazy_upd_ = false, lazy_now_ = false, lazy_skip_now_ = false, lazy_owed_ = false;
	float lazy_lr_ = 0.f;
	float *w_saved_ = NULL;
	bool w_saved_valid_ = false;
	int rows_ = 0;           // batch rows of this node's output (1 for parameter nodes)
	float *out_ = NULL;      // 2 planes [rows][out_size]: what consumers read
	float *out_re() const { return out_; }
	float *out_im() const { return out_ + (size_t) rows_ * out_size_; }

public:
	CFunc(Uid uid, InSize in_size, OutSize out_size) : input_(in_size.value()), uid_(uid.value()), out_size_(out_size.value()) {}
	CFunc(InSize in_size, OutSize out_size) : input_(in_size.value()), out_size_(out_size.value()) {}
	virtual ~CFunc() {}
	void setRandSeed(uint64_t seed) { rand_ = SimpleRand(seed); }
	bool isInput() { return is_input_; }
	bool isOutput() { return is_output_; }
	int getType() const { return type_; }
	int outSize() { return out_size_; }
	const Vars &input() const { return input_; }
	Vars *mutable_input() { return &input_; }
	const Vars &output() { assert(next_func_.size()); return next_func_[0]->input(); }
	const Vars &output(int i) { return next_func_[i]->input(); }
	Vars *mutable_output() { assert(next_func_.size()); return next_func_[0]->mutable_input(); }
	Vars *mutable_output(int i) { assert(i >= 0 && i < (int) next_func_.size()); return next_func_[i]->mutable_input(); }
	int uid() { return uid_; }
	int depth() { return depth_; }
	CFunc *next(int i) const { return next_func_[i]; }
	int offset(int i) { return offset_[i]; }
	int no_outputs() const { return (int) next_func_.size(); }
	int no_previous_func() const { return (int) prev_func_.size(); }
	CFunc *previous(int i) { return prev_func_[i]; }
	virtual int sizeInBytes() const { return (int) input_.size_in_bytes(); }
	// upstream's per-class operator== (impl/linear.h:135-151, impl/cinput.h:90-114 and the like): the same kind of function
	// with the same uid, sizes and consumers; input functions also hold the same values
	virtual bool operator==(const CFunc &rhs) const {
		if (typeId() != rhs.typeId() || uid_ != rhs.uid_ || input_.length_ != rhs.input_.length_ || out_size_ != rhs.out_size_ ||
				no_outputs() != rhs.no_outputs())
			return false;
		for (int i = 0; i < no_outputs(); ++i)
			if (next(i)->uid_ != rhs.next(i)->uid_) return false;
		if (is_input_)
			for (int i = 0; i < input_.length_; ++i)
				if (input_.real_[i] != rhs.input_.real_[i] || input_.imag_[i] != rhs.input_.imag_[i]) return false;
		return true;
	}
	bool operator!=(const CFunc &rhs) const { return !(*this == rhs); }
	virtual std::string getName() = 0;
	virtual int typeId() const = 0;

	// impl/cfunc.h:195-201
	virtual void init_inputs() {
		for (int i = 0; i < input_.length_; ++i) {
			float re = (float) rand_.randDouble() - 0.5;
			input_.real_[i] = re / input_.length_;
			input_.imag_[i] = sqrt(1 - re * re) / input_.length_;
		}
	}
	// the host view as text (impl/cfunc.h:158-209): values, values in rows of in_len, both gradients
	virtual void printInput() {
		std::cout << getName() << ": ";
		for (int i = 0; i < input_.length_; ++i) std::cout << i << ": " << input_.z(i) << ", ";
		std::cout << std::endl;
	}
	virtual void printInput2D(int in_len) { printInput2D(in_len, 0, input_.length_); }
	virtual void printInput2D(int in_len, int offset, int len) {
		assert(in_len > 0 && offset >= 0 && offset + len <= input_.length_);
		std::cout << getName() << ": " << std::endl;
		for (int i = 0; i < len; ++i) {
			std::cout << (offset + i) << ": " << input_.z(offset + i) << ", ";
			if (i % in_len == in_len - 1) std::cout << std::endl;
		}
		std::cout << std::endl;
	}
	virtual void printGradient() {
		std::cout << getName() << ": ";
		for (int i = 0; i < input_.length_; ++i) std::cout << i << "\tdz: " << input_.dz(i) << ", ";
		std::cout << std::endl << getName() << ": ";
		for (int i = 0; i < input_.length_; ++i) std::cout << i << "\tdz_star: " << input_.dz_star(i) << ", ";
		std::cout << std::endl;
	}
	// impl/cfunc.h:211-224
	void addOutput(CFunc *next, int offset) {
		assert(next && offset >= 0);
		if (next->input().length_ < offset + out_size_)
			throw std::invalid_argument("add: " + next->getName() + " input is shorter than offset + output of " + getName());
		next_func_.push_back(next);
		offset_.push_back(offset);
		if (next->depth_ <= depth_) next->depth_ = depth_ + 1;
	}
};

class CInput : public CFunc, public InputFunc {
	bool batched_ = false;
public:
	// A second per-sample data input (e.g. regression targets).  Upstream's GPU path knows exactly one data input
	// ("Only one main input supported", impl/cnet.h:541-544); flagging a CInput before allocateOnGpu() gives it batch
	// rows as well, filled with CNet::gpuSetInput().
	void setIsBatched(bool v) { batched_ = v; }
	bool isBatched() const { return batched_; }
	CInput(Uid uid, OutSize out) : CFunc(uid, InSize(out.value()), out) { is_input_ = true; }
	CInput(OutSize out) : CFunc(InSize(out.value()), out) { is_input_ = true; }
	std::string getName() override { return "Input_" + std::to_string(uid_); }
	int typeId() const override { return ::isInput; }
	void setInput(InputBatch &batch, int b) {
		assert(batch.sampleDim() == input().length_);
		if (batch.isResident()) throw std::logic_error("CInput::setInput: the samples of this batch are on the device, not in the batch");
		std::copy(batch.realDataPtr(b), batch.realDataPtr(b) + input().length_, mutable_input()->real_);
		std::copy(batch.imagDataPtr(b), batch.imagDataPtr(b) + input().length_, mutable_input()->imag_);
	}
};

class Linear : public CFunc {
	int in1_len, in2_len;
public:
	Linear(Uid uid, InSize in1, InSize in2) : CFunc(uid, InSize(in1.value() + in2.value()), OutSize(in2.value() / in1.value())),
			in1_len(in1.value()), in2_len(in2.value()) { assert(in2.value() % in1.value() == 0); }
	Linear(InSize in1, InSize in2) : CFunc(InSize(in1.value() + in2.value()), OutSize(in2.value() / in1.value())),
			in1_len(in1.value()), in2_len(in2.value()) { assert(in2.value() % in1.value() == 0); }
	int firstInputLength() { return in1_len; }
	int secondInputLength() { return in2_len; }
	std::string getName() override { return "Linear_" + std::to_string(uid_); }
	int typeId() const override { return isLinear; }
};

class FourierTrans : public CFunc {
public:
	FourierTrans(Uid uid, InSize n) : CFunc(uid, n, OutSize(n.value())) {}
	FourierTrans(InSize n) : CFunc(n, OutSize(n.value())) {}
	std::string getName() override { return "FourierTrans_" + std::to_string(uid_); }
	int typeId() const override { return isFourier; }
};

// Not an upstream layer: a FourierTrans along an axis upstream's API cannot address.  Upstream transforms the flat vector
// of ONE sample (impl/ft.h:37-80), and a Linear there acts on the whole flattened sample; a model that treats the positions
// of a sequence alike (the same Linear for every token) has no spelling.  With one token per sample it has: an
// EmbeddingBatch of batch x seq one-token samples, CEmbedding(dim, 1, vocab), and Hadamard / Linear / CGelu /
// CrossEntropy as they are, row by row.  What is then missing is the one layer that mixes the tokens of a sequence, and
// that is this one: the batch rows are taken in groups of `seq` consecutive rows (the positions of one sequence), and
// each of the n channels is transformed along its group,
//     y[g seq + p][c] = (1 / sqrt(seq)) sum_q x[g seq + q][c] e^{-2 pi i p q / seq},
// FourierTrans(seq) applied to every (sequence, channel) column; backward dz = F g.dz, dz* = conj(F) g.dz* along the same
// axis (impl/ft.h:57-79).  On the device one strided-batched matrix product against the seq x seq twiddle planes.
// The batch must hold whole sequences (allocateOnGpu(B) with B a multiple of seq); the per-sample calls, which see one
// row, refuse a net that contains it.  ModelSaver refuses it as well (upstream's file format has no such record).
class SeqFourierTrans : public CFunc {
	friend class CNet;
	int seq_;
	const float *f_re_ = NULL, *f_im_ = NULL;  // device: the twiddle planes of length seq (owned by the device library)
	int f_ld_ = 0;
public:
	SeqFourierTrans(Uid uid, InSize n, int seq) : CFunc(uid, n, OutSize(n.value())), seq_(seq) { assert(seq > 0); }
	SeqFourierTrans(InSize n, int seq) : CFunc(n, OutSize(n.value())), seq_(seq) { assert(seq > 0); }
	int seq() const { return seq_; }
	std::string getName() override { return "SeqFourierTrans_" + std::to_string(uid_); }
	int typeId() const override { return isSeqFourier; }
};

class Hadamard : public CFunc {
public:
	Hadamard(Uid uid, InSize a, InSize b) : CFunc(uid, InSize(a.value() + b.value()), OutSize(a.value())) { assert(a.value() == b.value()); }
	Hadamard(InSize a, InSize b) : CFunc(InSize(a.value() + b.value()), OutSize(a.value())) { assert(a.value() == b.value()); }
	std::string getName() override { return "Hadamard_" + std::to_string(uid_); }
	int typeId() const override { return isHadamard; }
};

class CGelu : public CFunc {
public:
	CGelu(Uid uid, InSize n) : CFunc(uid, n, OutSize(n.value())) {}
	CGelu(InSize n) : CFunc(n, OutSize(n.value())) {}
	std::string getName() override { return "CGelu_" + std::to_string(uid_); }
	int typeId() const override { return isGelu; }
};

// impl/relu.h:12-30
class CRelu : public CFunc {
public:
	CRelu(Uid uid, InSize n) : CFunc(uid, n, OutSize(n.value())) {}
	CRelu(InSize n) : CFunc(n, OutSize(n.value())) {}
	std::string getName() override { return "CRelu_" + std::to_string(uid_); }
	int typeId() const override { return isCrelu; }
};

// impl/ft.h:115-137
class TriangFourier : public CFunc {
public:
	TriangFourier(Uid uid, InSize n) : CFunc(uid, n, OutSize(n.value())) {}
	TriangFourier(InSize n) : CFunc(n, OutSize(n.value())) {}
	std::string getName() override { return "TriangFourier_" + std::to_string(uid_); }
	int typeId() const override { return isTrianFourier; }
};

class Residual : public CFunc {
public:
	Residual(Uid uid, InSize n) : CFunc(uid, InSize(2 * n.value()), OutSize(n.value())) {}
	Residual(Uid uid, InSize a, InSize b) : CFunc(uid, InSize(2 * a.value()), OutSize(a.value())) { assert(a.value() == b.value()); }
	Residual(InSize n) : CFunc(InSize(2 * n.value()), OutSize(n.value())) {}
	Residual(InSize a, InSize b) : CFunc(InSize(2 * a.value()), OutSize(a.value())) { assert(a.value() == b.value()); }
	std::string getName() override { return "Res_" + std::to_string(uid_); }
	int typeId() const override { return isResidual; }
};

class SoftMax : public CFunc {
	friend class CNet;
	float *d_s_ = NULL;  // device: sum |z|^2 per row
public:
	SoftMax(Uid uid, InSize n) : CFunc(uid, n, OutSize(n.value())) {}
	SoftMax(InSize n) : CFunc(n, OutSize(n.value())) {}
	std::string getName() override { return "SoftMax_" + std::to_string(uid_); }
	int typeId() const override { return isSoftMax; }
};

// Where the per-row losses of an output function go.  A forward pass that is launched kernel by kernel writes them straight
// into page-locked host memory (a ring of slots, one per forward pass: the kernel's stores travel over the link, no copy
// is queued); a forward pass inside a recording writes to the device buffer, since a replay cannot move to the next slot.
struct OutLoss {
	static constexpr int kSlots = 4;
	float *dev = NULL;        // device: [rows]
	float *host = NULL;       // page-locked: [kSlots][rows]
	int rows = 0;
	int64_t serial = -1;      // forward passes that have written to the ring so far, minus one
	const float *cur = NULL;  // where the last forward pass wrote
	bool cur_on_host = false;
};

class CrossEntropy : public CFunc, public OutputFunc {
	friend class CNet;
	Vars output_;
	int prediction_ = 0;                    // argmax of the fetched sample, computed on the device
	float *d_s_ = NULL;                     // device: [rows]
	OutLoss loss_;
	// The gradient planes hold what a backward pass with the current labels would write: the forward pass wrote it in the
	// same launch (cnet_cross_entropy_fwd_bwd_sym), and the backward pass of this node then has nothing to do.
	bool grad_from_forward_ = false;
	int32_t *d_argmax_ = NULL;
	float *d_norm_ = NULL;                  // device: normalised z, 2 planes [rows][n]
	// Nothing on the device reads the normalised rows: the loss, the prediction and the gradient come from z and its row
	// sums.  A forward pass launched kernel by kernel therefore leaves them out (a pass that only reads, a quarter of the time
	// on long rows) and notes it here; they are written when something looks (CNet::fetch), from the same z, by the same
	// kernel.  d_norm_ itself is allocated then.
	bool norm_current_ = false;
public:
	CrossEntropy(Uid uid, InSize n) : CFunc(uid, n, OutSize(1)), output_(n.value()) { is_output_ = true; }
	CrossEntropy(InSize n) : CFunc(n, OutSize(1)), output_(n.value()) { is_output_ = true; }
	std::string getName() override { return "CrossEntropy_" + std::to_string(uid_); }
	int typeId() const override { return isCrossEntropy; }
	// impl/crossent.h:38-59: accessors over the normalised output of the last fetched sample
	float getProbability(int label) { return std::pow(output_.real_[label], 2) + std::pow(output_.imag_[label], 2); }
	float loss(int label) override {
		assert(label >= 0 && label < input().length_);
		float v = getProbability(label);
		v = (v < 1e-15 ? 1e-15 : v);
		return -std::log(v);
	}
	int get_prediction() { return prediction_; }
	void printProbabilities() {  // impl/crossent.h:43-48
		for (int k = 0; k < input().length_; ++k) std::cout << std::setprecision(9) << k << ": " << getProbability(k) << ", ";
		std::cout << std::endl;
	}
	int sizeInBytes() const override { return (int) (input().size_in_bytes() + output_.size_in_bytes()); }
	int outputLength() override { return output_.length_; }
	Vars *mutableOutput() override { return &output_; }
};

class L2Out : public CFunc, public OutputFunc {
	friend class CNet;
	Vars output_;
	OutLoss loss_;
public:
	L2Out(Uid uid, InSize n) : CFunc(uid, n, OutSize(1)), output_(1) { is_output_ = true; }
	L2Out(InSize n) : CFunc(n, OutSize(1)), output_(1) { is_output_ = true; }
	std::string getName() override { return "L2Out_" + std::to_string(uid_); }
	int typeId() const override { return isL2Out; }
	float loss() { return output_.real_[0]; }
	float loss(int) override { return output_.real_[0]; }
	int sizeInBytes() const override { return (int) (input().size_in_bytes() + output_.size_in_bytes()); }
	int outputLength() override { return output_.length_; }
	Vars *mutableOutput() override { return &output_; }
};

class CEmbedding : public CFunc, public InputFunc {
	friend class CNet;
	int embedding_dim_, no_embeddings_, no_out_tokens_;
	std::vector<int> tokens_;
	int32_t *d_tokens_ = NULL;  // device: [rows][no_out_tokens]
public:
	CEmbedding(Uid uid, int dim, int max_out_tokens, int no_embeddings)
			: CFunc(uid, InSize(no_embeddings * dim), OutSize(max_out_tokens * dim)), embedding_dim_(dim),
			  no_embeddings_(no_embeddings), no_out_tokens_(max_out_tokens) { is_input_ = true; }
	CEmbedding(int dim, int max_out_tokens, int no_embeddings)
			: CFunc(InSize(no_embeddings * dim), OutSize(max_out_tokens * dim)), embedding_dim_(dim),
			  no_embeddings_(no_embeddings), no_out_tokens_(max_out_tokens) { is_input_ = true; }
	int embeddingDim() { return embedding_dim_; }
	int noEmbeddings() { return no_embeddings_; }
	int noOutTokens() { return no_out_tokens_; }
	std::string getName() override { return "Embedding " + std::to_string(uid_); }
	int typeId() const override { return isEmbedding; }
	bool operator==(const CFunc &rhs) const override {  // impl/embed.h:161-197: also the shape of the table and the token list
		const CEmbedding *e = dynamic_cast<const CEmbedding *>(&rhs);
		return e && CFunc::operator==(rhs) && embedding_dim_ == e->embedding_dim_ && no_embeddings_ == e->no_embeddings_ &&
				no_out_tokens_ == e->no_out_tokens_ && tokens_ == e->tokens_;
	}
	void setInput(const std::vector<int> &list) {
		tokens_.clear();
		for (auto id : list) {
			assert(id < no_embeddings_);
			tokens_.push_back(id);
		}
		assert(tokens_.size() && (int) tokens_.size() <= no_out_tokens_);
	}
	void setInput(std::initializer_list<int> list) { setInput(std::vector<int>(list)); }
	// impl/embed.h:56-74, 208-222: the table row by row, the token list, and both in short
	void printEmbedding() {
		for (int t = 0; t < no_embeddings_; ++t) {
			std::cout << t << ":\t";
			for (int i = 0; i < embedding_dim_; ++i) std::cout << input().z(t * embedding_dim_ + i) << ", ";
			std::cout << std::endl;
		}
	}
	void printTokens() {
		std::cout << "Tokens:\t";
		for (auto t : tokens_) std::cout << t << ", ";
		std::cout << std::endl;
	}
	void printInput() override {
		std::cout << getName() << " on CPU:\n\t tokens: ";
		for (auto t : tokens_) std::cout << t << ",";
		std::cout << std::endl << "\t embeddings: ";
		for (int i = 0; i < std::min(16, input().length_); ++i) std::cout << i / embedding_dim_ << ": " << input().z(i) << ", ";
		std::cout << std::endl;
	}
	void init_inputs() override {  // impl/embed.h:101-107
		for (int i = 0; i < input().length_; ++i) {
			float re = (float) rand_.randDouble() - 0.5;
			mutable_input()->real_[i] = re / sqrt(embedding_dim_);
			mutable_input()->imag_[i] = sqrt(1 - re * re) / sqrt(embedding_dim_);
		}
	}
};

#endif  // CNET_AMD_HOST_FUNCTIONS_HPP_
