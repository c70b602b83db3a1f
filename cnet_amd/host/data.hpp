// cnet_amd/host/data.hpp -- batched sample readers with the interface of upstream's data/data.h:28-165
// (BatchedDataReader, MnistDataReader), laid out for the device pipeline of cnet.hpp.
//
// Upstream keeps one std::vector<std::complex<float>> per sample and copies element by element into a fresh batch.
// Here all samples sit in two contiguous planes [count x dim] (re, im); a shuffle permutes an index table, and a batch is
// filled with one memcpy per sample and plane straight into the page-locked planes of an InputBatch, which then goes to
// the device as one asynchronous copy per plane (CNet::gpuForward / gpuPrefetch).
#ifndef CNET_AMD_HOST_DATA_HPP_
#define CNET_AMD_HOST_DATA_HPP_

#include <algorithm>
#include <fstream>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include "cnet.hpp"

class BatchedDataReader {
	int current_ = 0;
	std::vector<float> re_, im_;  // [count][dim]
	std::vector<int> labels_;
	std::vector<int> order_;      // position -> sample
	std::vector<int> pick_;       // samples of the batch being assembled
	bool imag_all_zero_ = true;   // no sample added so far has an imaginary part other than +0 (images): batches skip that plane
	std::shared_ptr<DeviceDataset> on_device_;  // the samples as they were at storeOnDevice(), kept in device memory (copies of the reader share it)
	void noteImag(const float *im, size_t n) {
		uint32_t acc = 0;
		for (size_t k = 0; k < n; ++k) {
			uint32_t w;
			std::memcpy(&w, im + k, sizeof(w));
			acc |= w;
		}
		if (acc) imag_all_zero_ = false;
	}

protected:
	int sample_dim_ = 0;

public:
	BatchedDataReader(int sample_dim) : sample_dim_(sample_dim) {}
	virtual ~BatchedDataReader() {}

	int size() { return (int) labels_.size(); }
	int sampleDim() const { return sample_dim_; }

	void shuffle() {  // data/data.h:47-51
		std::random_device rd;
		shuffle(rd());
	}
	void shuffle(unsigned seed) {  // repeatable variant
		std::default_random_engine rng(seed);
		std::shuffle(order_.begin(), order_.end(), rng);
	}

	bool hasNextBatch(int batch_size) { return current_ + batch_size <= (int) labels_.size(); }

	// data/data.h:57-66: the next batch_size samples in the current order, wrapping around at the end
	InputBatch nextBatch(int batch_size) {
		InputBatch batch(batch_size, sample_dim_);
		nextBatch(batch);
		return batch;
	}
	// refill an existing batch (its page-locked planes are reused; waits if a copy from them is still running)
	void nextBatch(InputBatch &batch) {
		assert(labels_.size() && batch.sampleDim() == sample_dim_);
		batch.clear();
		pick_.resize(batch.size());
		for (int i = 0; i < batch.size(); ++i) {
			pick_[i] = order_[current_];
			current_ = (current_ + 1) % (int) labels_.size();
		}
		if (on_device_)
			batch.gatherResident(*on_device_, pick_.data(), batch.size());
		else
			batch.gather(re_.data(), imag_all_zero_ ? NULL : im_.data(), labels_.data(), pick_.data(), batch.size());
	}

	// Keep a copy of all samples and labels in device memory (the device library must be initialised): the batches of
	// nextBatch() then only name their samples, and CNet::gpuForward / gpuPrefetch copy them on the device instead of
	// sending them over the link again in every epoch.  Same samples, same order, same results.  Samples added afterwards
	// are not part of the copy until the next call; releaseDevice() goes back to batches that carry their samples.  The
	// reader must outlive the steps its batches were fed to.
	void storeOnDevice() {
		assert(labels_.size());
		on_device_.reset();
		on_device_.reset(new DeviceDataset(re_.data(), imag_all_zero_ ? NULL : im_.data(), labels_.data(), (int) labels_.size(), sample_dim_));
	}
	void releaseDevice() { on_device_.reset(); }
	bool storedOnDevice() const { return on_device_ != NULL; }

	void add(const std::vector<std::complex<float> > &data, int label) {
		assert((int) data.size() <= sample_dim_);
		const size_t at = re_.size();
		re_.resize(at + sample_dim_, 0.f);
		im_.resize(at + sample_dim_, 0.f);
		for (size_t k = 0; k < data.size(); ++k) {
			re_[at + k] = data[k].real();
			im_[at + k] = data[k].imag();
		}
		noteImag(&im_[at], data.size());
		order_.push_back((int) labels_.size());
		labels_.push_back(label);
	}
	void addPlanes(const float *re, const float *im, int label) {
		re_.insert(re_.end(), re, re + sample_dim_);
		im_.insert(im_.end(), im, im + sample_dim_);
		noteImag(im, (size_t) sample_dim_);
		order_.push_back((int) labels_.size());
		labels_.push_back(label);
	}
	void reserve(size_t count) {
		re_.reserve(count * sample_dim_);
		im_.reserve(count * sample_dim_);
		labels_.reserve(count);
		order_.reserve(count);
	}
	// sample `index` in insertion order
	const float *realOf(int index) const { return &re_[(size_t) index * sample_dim_]; }
	const float *imagOf(int index) const { return &im_[(size_t) index * sample_dim_]; }
	int labelOf(int index) const { return labels_[index]; }

	virtual bool readData() = 0;
};

// The MNIST idx files (images: 16-byte header, labels: 8-byte header, one byte per pixel / label), data/data.h:86-165.
// As upstream, a pixel byte is read through a plain `char` and becomes BOTH the real and the imaginary part of the
// input (data/data.h:129-132); on the platforms upstream builds for `char` is signed, so bytes above 127 arrive as
// negative values.  That conversion is kept so that models trained by upstream see the inputs they were trained on.
class MnistDataReader : public BatchedDataReader {
	std::vector<signed char> local_data_, local_labels_;
	bool is_open_ = false;
	int current_indx_ = 0, max_count_ = 0;

public:
	MnistDataReader() : BatchedDataReader(28 * 28) {}

	bool Open(std::string image_file, std::string label_file, int count) {
		is_open_ = false;
		std::ifstream images(image_file.c_str(), std::ios::in | std::ios::binary);
		if (images.fail()) {
			std::cerr << "Cannot open " << image_file << std::endl;
			return false;
		}
		std::ifstream labels(label_file.c_str(), std::ios::in | std::ios::binary);
		if (labels.fail()) {
			std::cerr << "Cannot open " << label_file << std::endl;
			return false;
		}
		if (count < 0) return false;
		char header[16];
		if (!images.read(header, 16) || !labels.read(header, 8)) return false;
		local_data_.resize((size_t) count * 28 * 28);
		local_labels_.resize(count);
		if (!images.read((char *) local_data_.data(), (std::streamsize) local_data_.size())) return false;
		if (!labels.read((char *) local_labels_.data(), count)) return false;
		max_count_ = count;
		current_indx_ = 0;
		is_open_ = true;
		return true;
	}

	bool readData() override {
		assert(is_open_);
		reserve(max_count_);
		std::vector<float> px(28 * 28);
		while (current_indx_ < max_count_) {
			for (int k = 0; k < 28 * 28; ++k) px[k] = (float) local_data_[(size_t) current_indx_ * 28 * 28 + k];
			addPlanes(px.data(), px.data(), (int) local_labels_[current_indx_]);
			current_indx_++;
		}
		return true;
	}
};

#endif  // CNET_AMD_HOST_DATA_HPP_
