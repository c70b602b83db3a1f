// cnet_amd/host/batches.hpp
// Batches of samples as upstream's impl/batch.h hands them to the net, held in page-locked memory for the device pipeline,
// and a data set kept in device memory.  Included by cnet.hpp (after vars.hpp).
#ifndef CNET_AMD_HOST_BATCHES_HPP_
#define CNET_AMD_HOST_BATCHES_HPP_

// ---------------------------------------------------------------------------------------------------------------
// impl/batch.h
// ---------------------------------------------------------------------------------------------------------------
const int NO_TOKEN = -1;

class Batch {
	friend class CNet;
protected:
	std::vector<float> losses_;
	std::vector<int> labels_;
	std::vector<int> sizes_;
	int current_pos_ = 0, batch_size_ = 0, sample_dim_ = 0;
	void addLoss(float loss) { losses_.push_back(loss); }
public:
	Batch() {}
	Batch(int batch_size, int sample_dim) : batch_size_(batch_size), sample_dim_(sample_dim) {}
	virtual ~Batch() {}
	int size() { return batch_size_; }
	int sampleDim() { return sample_dim_; }
	float loss(int i) { return losses_[i]; }
	int noOfLabels() const { return (int) labels_.size(); }
	const int *labelsPtr() const { return &labels_[0]; }
	int label(int i) { return labels_[i]; }
};

// A data set kept on the device: the samples as planes [count][dim] (the imaginary plane only if some sample has an imaginary
// part other than +0) and their labels.  A batch assembled out of it (InputBatch::gatherResident, BatchedDataReader::
// storeOnDevice) names its samples by index; gpuForward / gpuPrefetch then send the indices, 4 bytes per sample, and the
// device copies the rows out of its own memory (cnet_upload_gather_rows) instead of receiving them over the link again in
// every epoch.  No counterpart upstream, whose batches always travel from host memory (gpu/gpu_func.h:403-419).  Must outlive
// every batch that refers to it and every step that such a batch was fed to.
class DeviceDataset {
	friend class CNet;
	friend class InputBatch;
	float *z_ = NULL;             // device: planes_ x [count][dim]
	int32_t *labels_dev_ = NULL;  // device: [count]
	std::vector<int> labels_;
	int count_ = 0, dim_ = 0, planes_ = 1;
	static void must(int rc, const char *what) {
		if (rc != CNET_OK) throw std::runtime_error(std::string(what) + " failed (" + std::to_string(rc) + "): " + cnet_last_error());
	}

public:
	// re, im: [count][dim] on the host (im may be NULL: real samples); labels: [count]
	DeviceDataset(const float *re, const float *im, const int *labels, int count, int dim) : labels_(labels, labels + count), count_(count), dim_(dim) {
		if (count <= 0 || dim <= 0) throw std::invalid_argument("DeviceDataset: no samples");
		const size_t plane = (size_t) count * dim;
		bool complex_samples = false;
		if (im) {
			uint32_t acc = 0;
			for (size_t k = 0; k < plane; ++k) {
				uint32_t w;
				std::memcpy(&w, im + k, sizeof(w));
				acc |= w;
			}
			complex_samples = acc != 0;
		}
		planes_ = complex_samples ? 2 : 1;
		void *p = NULL;
		must(cnet_alloc((size_t) planes_ * plane * sizeof(float), &p), "cnet_alloc");
		z_ = (float *) p;
		must(cnet_alloc((size_t) count * sizeof(int32_t), &p), "cnet_alloc");
		labels_dev_ = (int32_t *) p;
		must(cnet_memcpy_h2d(z_, re, plane * sizeof(float)), "cnet_memcpy_h2d");
		if (complex_samples) must(cnet_memcpy_h2d(z_ + plane, im, plane * sizeof(float)), "cnet_memcpy_h2d");
		std::vector<int32_t> l32(labels, labels + count);
		must(cnet_memcpy_h2d(labels_dev_, l32.data(), (size_t) count * sizeof(int32_t)), "cnet_memcpy_h2d");
	}
	DeviceDataset(const DeviceDataset &) = delete;
	DeviceDataset &operator=(const DeviceDataset &) = delete;
	~DeviceDataset() {
		cnet_upload_sync();  // a batch may still be on its way out of these planes
		cnet_sync();
		cnet_free(z_);
		cnet_free(labels_dev_);
	}
	int size() const { return count_; }
	int sampleDim() const { return dim_; }
	int label(int i) const { return labels_[i]; }
	bool imagIsZero() const { return planes_ == 1; }  // every sample is real
};

// Two [batch x dim] planes in page-locked host memory when the device library is initialised (pageable otherwise), so
// a batch goes to the device as one asynchronous copy per plane (upstream: two pageable copies per sample,
// gpu/gpu_func.h:403-419).  Movable and reusable: clear() empties it for the next fill without giving the memory back.
class InputBatch : public Batch {
	friend class CNet;
	float *real_data_ = NULL, *imag_data_ = NULL;  // [batch][dim] each, one allocation
	bool pinned_ = false;
	int64_t ticket_ = -1;     // >= 0: a copy queued from these planes may not have finished; what the host waits for
	// Some sample added since the last clear() has an imaginary part that is not +0: while this is false the imaginary plane
	// holds nothing but zeros and need not travel to the device (real-valued data such as images: half the upload).
	bool imag_nonzero_ = false;
	// every element of the imaginary plane, filled rows or not, holds +0: rows of real samples then need no write at all
	bool imag_clean_ = false;
	// The samples of this batch are rows of a data set on the device (gatherResident): indices_[k] names the row of sample k,
	// the planes above are not filled.
	const DeviceDataset *resident_ = NULL;
	int32_t *indices_ = NULL;  // [batch], page-locked, allocated at the first gatherResident
	static bool anyBitSet(const float *p, size_t n) {
		uint32_t acc = 0;
		for (size_t k = 0; k < n; ++k) {
			uint32_t w;
			std::memcpy(&w, p + k, sizeof(w));
			acc |= w;
		}
		return acc != 0;
	}

	void allocate() {
		const size_t bytes = 2 * (size_t) batch_size_ * sample_dim_ * sizeof(float);
		if (!bytes) return;
		void *p = NULL;
		if (cnet_host_alloc(bytes, &p) == CNET_OK && p) {
			pinned_ = true;
		} else {
			p = ::operator new(bytes);
			pinned_ = false;
		}
		real_data_ = (float *) p;
		imag_data_ = real_data_ + (size_t) batch_size_ * sample_dim_;
		std::fill(imag_data_, imag_data_ + (size_t) batch_size_ * sample_dim_, 0.f);
		imag_clean_ = true;
	}
	void release() {
		if (indices_) cnet_host_free(indices_);  // (a batch of dimension 0 has indices and no planes)
		indices_ = NULL;
		if (!real_data_) return;
		if (pinned_) cnet_host_free(real_data_);  // waits for copies still reading it
		else ::operator delete(real_data_);
		real_data_ = imag_data_ = NULL;
	}
	void settle() {  // before the host writes the planes again
		if (ticket_ >= 0) {  // waits for that copy only: a copy out of another batch may still be running
			if (cnet_copy_wait(ticket_) != CNET_OK) {
				cnet_upload_sync();
				cnet_sync();
			}
			ticket_ = -1;
		}
	}
	void noteImag(bool some_bit_set) {
		if (!some_bit_set) return;
		imag_nonzero_ = true;
		imag_clean_ = false;
	}
	float *rowRe() { return real_data_ + (size_t) current_pos_ * sample_dim_; }
	float *rowIm() { return imag_data_ + (size_t) current_pos_ * sample_dim_; }
	void finishRow(int filled, int label) {
		if (resident_) throw std::logic_error("InputBatch: the batch holds samples of a data set on the device; clear() it first");
		std::fill(rowRe() + filled, rowRe() + sample_dim_, 0.f);  // padding with 0s
		std::fill(rowIm() + filled, rowIm() + sample_dim_, 0.f);
		labels_.push_back(label);
		sizes_.push_back(filled);
		current_pos_++;
	}

public:
	InputBatch() : Batch() {}
	InputBatch(int batch_size, int sample_dim) : Batch(batch_size, sample_dim) { allocate(); }
	InputBatch(const InputBatch &o) : Batch(o) {
		allocate();
		if (o.real_data_) std::copy(o.real_data_, o.real_data_ + 2 * (size_t) batch_size_ * sample_dim_, real_data_);
		imag_nonzero_ = o.imag_nonzero_;
		imag_clean_ = o.imag_clean_;
		if (o.resident_ && o.indices_) {
			void *p = NULL;
			if (cnet_host_alloc((size_t) batch_size_ * sizeof(int32_t), &p) == CNET_OK && p) {
				indices_ = (int32_t *) p;
				std::copy(o.indices_, o.indices_ + current_pos_, indices_);  // only the filled entries hold values
				resident_ = o.resident_;
			}
		}
	}
	InputBatch(InputBatch &&o) noexcept : Batch(std::move(o)), real_data_(o.real_data_), imag_data_(o.imag_data_), pinned_(o.pinned_),
			ticket_(o.ticket_), imag_nonzero_(o.imag_nonzero_), imag_clean_(o.imag_clean_), resident_(o.resident_), indices_(o.indices_) {
		o.real_data_ = o.imag_data_ = NULL;
		o.indices_ = NULL;
		o.resident_ = NULL;
	}
	InputBatch &operator=(InputBatch &&o) noexcept {
		if (this != &o) {
			release();
			Batch::operator=(std::move(o));
			real_data_ = o.real_data_;
			imag_data_ = o.imag_data_;
			pinned_ = o.pinned_;
			ticket_ = o.ticket_;
			imag_nonzero_ = o.imag_nonzero_;
			imag_clean_ = o.imag_clean_;
			resident_ = o.resident_;
			indices_ = o.indices_;
			o.real_data_ = o.imag_data_ = NULL;
			o.indices_ = NULL;
			o.resident_ = NULL;
		}
		return *this;
	}
	InputBatch &operator=(const InputBatch &) = delete;
	~InputBatch() override { release(); }

	bool isPinned() const { return pinned_; }
	// empty the batch for refilling; the planes are kept
	void clear() {
		settle();
		losses_.clear();
		labels_.clear();
		sizes_.clear();
		current_pos_ = 0;
		imag_nonzero_ = false;
		resident_ = NULL;
	}
	// every imaginary part added so far is +0: the samples are real
	bool imagIsZero() const { return !imag_nonzero_; }
	void add(const std::vector<std::complex<float> > &sample, int label) {
		assert(current_pos_ < batch_size_ && (int) sample.size() <= sample_dim_);
		settle();
		float *re = rowRe(), *im = rowIm();
		for (size_t k = 0; k < sample.size(); ++k) {
			re[k] = sample[k].real();
			im[k] = sample[k].imag();
		}
		noteImag(anyBitSet(im, sample.size()));
		finishRow((int) sample.size(), label);
	}
	void add(std::initializer_list<std::complex<float> > list, int label) {
		add(std::vector<std::complex<float> >(list), label);
	}
	// bulk variant for callers that already hold the two planes of one sample
	void add(const float *re, const float *im, int n, int label) {
		assert(current_pos_ < batch_size_ && n <= sample_dim_);
		settle();
		std::copy(re, re + n, rowRe());
		std::copy(im, im + n, rowIm());
		noteImag(anyBitSet(im, (size_t) n));
		finishRow(n, label);
	}
	// Fill the next `count` rows from planar sample storage ([sample][dim] re and im): row k takes sample index[k] and
	// label labels[index[k]].  The rows are independent copies, spread over the host threads when built with OpenMP (a
	// batch of 4096 x 784 is 25 MB; one thread assembles it no faster than the device trains on it).
	// im == NULL: every sample is real (the reader knows); the imaginary rows then only need clearing if something else
	// than +0 has been in the plane since it was last all zeros.
	void gather(const float *re, const float *im, const int *labels, const int *index, int count) {
		assert(current_pos_ + count <= batch_size_);
		if (resident_) throw std::logic_error("InputBatch: the batch holds samples of a data set on the device; clear() it first");
		settle();
		const size_t dim = (size_t) sample_dim_;
		float *dst_re = rowRe(), *dst_im = rowIm();
		const bool clear_im = !im && !imag_clean_;
		int nonzero = 0;
#pragma omp parallel for schedule(static) reduction(| : nonzero) if ((size_t) count * dim >= (1u << 18))
		for (int k = 0; k < count; ++k) {
			std::memcpy(dst_re + k * dim, re + index[k] * dim, dim * sizeof(float));
			if (im) {
				std::memcpy(dst_im + k * dim, im + index[k] * dim, dim * sizeof(float));
				nonzero |= anyBitSet(dst_im + k * dim, dim) ? 1 : 0;
			} else if (clear_im) {
				std::memset(dst_im + k * dim, 0, dim * sizeof(float));
			}
		}
		noteImag(nonzero != 0);
		if (clear_im && current_pos_ == 0 && count == batch_size_) imag_clean_ = true;  // every row of the plane was cleared just now
		for (int k = 0; k < count; ++k) {
			labels_.push_back(labels[index[k]]);
			sizes_.push_back(sample_dim_);
		}
		current_pos_ += count;
	}
	// The next `count` samples of the batch are rows index[0 .. count) of a data set on the device: only the indices and the
	// labels are noted here, the planes of this batch stay as they are.  A batch is filled either this way, from one data
	// set, or with add() / gather(), not both.
	void gatherResident(const DeviceDataset &ds, const int *index, int count) {
		assert(current_pos_ + count <= batch_size_);
		if (ds.sampleDim() != sample_dim_) throw std::invalid_argument("InputBatch::gatherResident: sample dimension differs from the data set");
		if ((current_pos_ > 0 && resident_ != &ds) || (resident_ && resident_ != &ds))
			throw std::logic_error("InputBatch::gatherResident: the batch already holds samples from elsewhere");
		settle();  // the indices of the last fill may still be read
		if (!indices_) {
			void *p = NULL;
			if (cnet_host_alloc((size_t) batch_size_ * sizeof(int32_t), &p) != CNET_OK || !p)
				throw std::runtime_error("InputBatch::gatherResident: no page-locked memory for the indices (is the device library initialised?)");
			indices_ = (int32_t *) p;
		}
		resident_ = &ds;
		for (int k = 0; k < count; ++k) {
			if (index[k] < 0 || index[k] >= ds.size()) throw std::out_of_range("InputBatch::gatherResident: no such sample in the data set");
			indices_[current_pos_ + k] = index[k];
			labels_.push_back(ds.label(index[k]));
			sizes_.push_back(sample_dim_);
		}
		if (!ds.imagIsZero()) imag_nonzero_ = true;
		current_pos_ += count;
	}
	bool isResident() const { return resident_ != NULL; }
	const float *realDataPtr() const { return real_data_; }
	const float *imagDataPtr() const { return imag_data_; }
	const float *realDataPtr(int b) const { return real_data_ + (size_t) b * sample_dim_; }
	const float *imagDataPtr(int b) const { return imag_data_ + (size_t) b * sample_dim_; }
	// one sample's planes as vectors (impl/batch.h:171-183)
	std::vector<float> realData(int b) const { return std::vector<float>(realDataPtr(b), realDataPtr(b) + sample_dim_); }
	std::vector<float> imagData(int b) const { return std::vector<float>(imagDataPtr(b), imagDataPtr(b) + sample_dim_); }
};

class EmbeddingBatch : public Batch {
	friend class CNet;
	std::vector<int> token_;
	int counter_ = 0;
public:
	EmbeddingBatch() : Batch() {}
	EmbeddingBatch(int batch_size, int sample_dim) : Batch(batch_size, sample_dim) {}
	void add(const std::vector<int> &sample, int label) {
		assert(current_pos_ < batch_size_);
		token_.insert(token_.end(), sample.begin(), sample.end());
		while (token_.size() < (size_t) (1 + current_pos_) * sample_dim_) token_.push_back(NO_TOKEN);  // padding with -1s
		labels_.push_back(label);
		sizes_.push_back((int) sample.size());
		current_pos_++;
		counter_ += (int) sample.size();
	}
	int noOfTokens() const { return (int) token_.size(); }
	// impl/batch.h:112-122: tokens (padding aside) and labels folded into 0 .. mod - 1
	void scale(int mod) {
		for (auto &t : token_)
			if (t >= 0) t %= mod;
		for (auto &l : labels_) l %= mod;
	}
	const int *tokensPtr() const { return &token_[0]; }
	int tokenCount() { return counter_; }
};

#endif  // CNET_AMD_HOST_BATCHES_HPP_
