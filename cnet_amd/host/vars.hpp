// cnet_amd/host/vars.hpp
// Sizes, ids, the random generator of parameter initialisation and the per-sample host view of a node's planes: the small
// types of upstream's impl/sizes.h, utils/myrand.h and impl/vars.h that the rest of the facade is written in.  Included by cnet.hpp.
#ifndef CNET_AMD_HOST_VARS_HPP_
#define CNET_AMD_HOST_VARS_HPP_

// ---------------------------------------------------------------------------------------------------------------
// impl/sizes.h
// ---------------------------------------------------------------------------------------------------------------
class Size {
	int value_;
public:
	Size(int value) : value_(value) {}
	unsigned int value() { return value_; }
};
class InSize {
	unsigned int value_;
public:
	InSize(int value) : value_(value) {}
	unsigned int value() { return value_; }
};
class OutSize {
	unsigned int value_;
public:
	OutSize(int value) : value_(value) {}
	unsigned int value() { return value_; }
};
class Uid {
	int value_;
public:
	Uid(int value) : value_(value) {}
	int value() { return value_; }
};

// ---------------------------------------------------------------------------------------------------------------
// utils/myrand.h: xorshift64* and the polar normal, for reproducible parameter initialisation
// ---------------------------------------------------------------------------------------------------------------
class SimpleRand {
	uint64_t state_;
	double lastVal_;
public:
	SimpleRand(uint64_t seed = 88172645463325252ULL) : state_(0x2545F4914F6CDD1DULL ^ seed), lastVal_(0.0) {}
	uint64_t randUint64() {
		uint64_t x = state_;
		x ^= x >> 12;
		x ^= x << 25;
		x ^= x >> 27;
		state_ = x;
		return x * 0x2545F4914F6CDD1DULL;
	}
	double randDouble() { return 5.42101086242752217E-20 * randUint64(); }
	double normal(double mu, double sig) {
		if (lastVal_ == 0.) {
			double v1, v2, rsq;
			do {
				v1 = 2.0 * randDouble() - 1.0;
				v2 = 2.0 * randDouble() - 1.0;
				rsq = v1 * v1 + v2 * v2;
			} while (rsq >= 1.0 || rsq == 0.0);
			double fac = sqrt(-2.0 * log(rsq) / rsq);
			lastVal_ = v1 * fac;
			return mu + sig * v2 * fac;
		}
		double fac = lastVal_;
		lastVal_ = 0.;
		return mu + sig * fac;
	}
};

// ---------------------------------------------------------------------------------------------------------------
// impl/vars.h: six contiguous planes on the host (the per-sample view)
// ---------------------------------------------------------------------------------------------------------------
class Vars {
public:
	int length_ = 0;
	float *real_ = NULL, *imag_ = NULL, *dz_real_ = NULL, *dz_imag_ = NULL, *dz_star_real_ = NULL, *dz_star_imag_ = NULL;

	Vars() {}
	explicit Vars(int length) : length_(length) {
		assert(length > 0);
		real_ = new float[(size_t) length_ * 6];
		bind();
		std::fill(real_, real_ + (size_t) length_ * 6, 0.0f);
	}
	Vars(const Vars &o) : length_(o.length_) {
		if (!o.real_) return;
		real_ = new float[(size_t) length_ * 6];
		bind();
		std::copy(o.real_, o.real_ + (size_t) length_ * 6, real_);
	}
	Vars &operator=(const Vars &) = delete;
	virtual ~Vars() { delete[] real_; }

	void zero_gradients() { std::fill(dz_real_, dz_real_ + (size_t) length_ * 4, 0.0f); }
	void zero_input() { std::fill(real_, real_ + (size_t) length_ * 2, 0.0f); }
	std::complex<float> z(int i) const { return std::complex<float>(real_[i], imag_[i]); }
	std::complex<float> dz(int i) const { return std::complex<float>(dz_real_[i], dz_imag_[i]); }
	std::complex<float> dz_star(int i) const { return std::complex<float>(dz_star_real_[i], dz_star_imag_[i]); }
	void zSetValue(int i, std::complex<float> v) { real_[i] = v.real(); imag_[i] = v.imag(); }
	void dzSetValue(int i, std::complex<float> v) { dz_real_[i] = v.real(); dz_imag_[i] = v.imag(); }
	void dz_starSetValue(int i, std::complex<float> v) { dz_star_real_[i] = v.real(); dz_star_imag_[i] = v.imag(); }
	void zero_dZ() { std::fill(dz_real_, dz_real_ + (size_t) length_ * 2, 0.0f); }
	void zero_dZ_star() { std::fill(dz_star_real_, dz_star_real_ + (size_t) length_ * 2, 0.0f); }
	// the first max_len values / gradients as text (impl/vars.h:123-145)
	std::string zToString(int max_len) const { return listed(real_, max_len); }
	std::string dzToString(int max_len) const { return listed(dz_real_, max_len); }
	std::string dz_starToString(int max_len) const { return listed(dz_star_real_, max_len); }
	unsigned long long size_in_bytes() const { return 6ULL * length_ * sizeof(float); }
	float *plane(int p) { return real_ + (size_t) p * length_; }
private:
	std::string listed(const float *re, int max_len) const {  // re and the plane after it: one complex value per index
		std::ostringstream oss;
		for (int i = 0; i < std::min(length_, max_len); ++i) oss << std::complex<float>(re[i], re[length_ + i]) << ", ";
		return oss.str();
	}
	void bind() {
		imag_ = real_ + length_;
		dz_real_ = imag_ + length_;
		dz_imag_ = dz_real_ + length_;
		dz_star_real_ = dz_imag_ + length_;
		dz_star_imag_ = dz_star_real_ + length_;
	}
};

// impl/vars.h:165-177: sum of |z|^2 over the values, and its root
inline float norm(const Vars &v) {
	float sum = 0;
	for (int i = 0; i < v.length_; ++i) sum += v.real_[i] * v.real_[i] + v.imag_[i] * v.imag_[i];
	return sum;
}
inline float abs(const Vars &v) { return std::sqrt(norm(v)); }

#endif  // CNET_AMD_HOST_VARS_HPP_
