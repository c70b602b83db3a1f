// cnet_amd/host/model_saver.hpp -- reads and writes upstream CNet's .mod model files for the facade's CNet.
//
// Same class name and methods as upstream's ModelSaver (impl/model_saver.h:483-967): Save / Restore on a file,
// SaveToString / RestoreFromString on a byte string.  The stream is upstream's, byte for byte:
//
//   int32 magic 0xABCDE0EE
//   per function, in insertion order:
//     int32 type id (impl/cnet.h:31-44), uid, input length, output size, number of producers, producer uids
//     CInput      : float32 re[len], im[len]
//     CEmbedding  : int32 dim, slots, vocab ; float32 re[len], im[len]
//     Linear      : int32 in1, in2
//   every int32 and float32 big-endian (impl/model_saver.h:60-76, 392-416).
//
// A model trained by upstream on its CPU or CUDA path loads here and runs on the device after allocateOnGpu(); a net
// trained here is written back with getInputsFromGpu() + Save and loads in upstream.  Included by cnet.hpp.
#ifndef CNET_AMD_HOST_MODEL_SAVER_HPP_
#define CNET_AMD_HOST_MODEL_SAVER_HPP_

#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

const int magicNo = 0xABCDE0EE;

class ModelSaver {
	static void put32(std::string &o, uint32_t v) {
		char b[4] = {(char) (v >> 24), (char) (v >> 16), (char) (v >> 8), (char) v};
		o.append(b, 4);
	}
	static void putFloats(std::string &o, const float *p, int n) {
		const size_t at = o.size();
		o.resize(at + 4 * (size_t) n);
		for (int k = 0; k < n; ++k) {
			uint32_t u;
			memcpy(&u, p + k, 4);
			char *b = &o[at + 4 * (size_t) k];
			b[0] = (char) (u >> 24);
			b[1] = (char) (u >> 16);
			b[2] = (char) (u >> 8);
			b[3] = (char) u;
		}
	}
	struct Cursor {
		const std::string &s;
		size_t pos = 0;
		explicit Cursor(const std::string &str) : s(str) {}
		bool get32(int *v) {
			if (pos + 4 > s.size()) return false;
			const unsigned char *b = (const unsigned char *) s.data() + pos;
			*v = (int) (((uint32_t) b[0] << 24) | ((uint32_t) b[1] << 16) | ((uint32_t) b[2] << 8) | (uint32_t) b[3]);
			pos += 4;
			return true;
		}
		bool getFloats(float *p, int n) {
			if (n < 0 || pos + 4 * (size_t) n > s.size()) return false;
			for (int k = 0; k < n; ++k) {
				int v = 0;
				get32(&v);
				memcpy(p + k, &v, 4);
			}
			return true;
		}
	};

	static void writeFuncInfo(std::string &o, CFunc *f) {  // impl/model_saver.h:533-542
		put32(o, (uint32_t) f->uid());
		put32(o, (uint32_t) f->input().length_);
		put32(o, (uint32_t) f->outSize());
		put32(o, (uint32_t) f->no_previous_func());
		for (int k = 0; k < f->no_previous_func(); ++k) put32(o, (uint32_t) f->previous(k)->uid());
	}

public:
	virtual ~ModelSaver() {}

	std::string SaveToString(CNet &net) {
		std::string o;
		put32(o, (uint32_t) magicNo);
		for (auto f : net.functionList()) {
			const int t = f->typeId();
			switch (t) {
			case isInput: case isHadamard: case isLinear: case isEmbedding: case isFourier: case isTrianFourier: case isResidual:
			case isCrossEntropy: case isL2Out: case isSoftMax: case isCrelu: case isGelu: break;
			default: std::cerr << "Cannot save " << f->getName() << std::endl; return "";
			}
			put32(o, (uint32_t) t);
			writeFuncInfo(o, f);
			if (t == isEmbedding) {
				CEmbedding *e = (CEmbedding *) f;
				put32(o, (uint32_t) e->embeddingDim());
				put32(o, (uint32_t) e->noOutTokens());
				put32(o, (uint32_t) e->noEmbeddings());
			}
			if (t == isInput || t == isEmbedding) {
				putFloats(o, f->input().real_, f->input().length_);
				putFloats(o, f->input().imag_, f->input().length_);
			}
			if (t == isLinear) {
				put32(o, (uint32_t) ((Linear *) f)->firstInputLength());
				put32(o, (uint32_t) ((Linear *) f)->secondInputLength());
			}
		}
		return o;
	}

	bool Save(CNet &net, std::string file) {
		std::string blob = SaveToString(net);
		if (blob.empty()) return false;
		std::ofstream out(file, std::ofstream::out | std::ofstream::trunc | std::ofstream::binary);
		if (!out) {
			std::cerr << "Cannot open: \"" << file << "\"" << std::endl;
			return false;
		}
		out.write(blob.data(), (std::streamsize) blob.size());
		out.close();
		return (bool) out;
	}

	// Appends the stored functions to `net` with their stored uids (upstream restores into an empty net).  Returns false
	// on a wrong magic number, an unknown type id, a truncated record or a record that does not fit the graph (upstream
	// asserts on the last two).
	bool RestoreFromString(CNet &net, const std::string &input) {
		Cursor in(input);
		int current = 0;
		if (!in.get32(&current) || current != magicNo) {
			std::cerr << "not a CNet model: magic " << std::hex << current << std::dec << std::endl;
			return false;
		}
		try {
			while (in.get32(&current)) {
				int uid, in_size, out_size, no_prev;
				if (!in.get32(&uid) || !in.get32(&in_size) || !in.get32(&out_size) || !in.get32(&no_prev)) return false;
				if (uid <= 0 || in_size < 0 || out_size < 0 || no_prev < 0 || (size_t) no_prev > input.size()) return false;
				std::vector<int> prev(no_prev);
				for (auto &p : prev)
					if (!in.get32(&p)) return false;
				if ((current == isInput || current == isEmbedding) && 8 * (size_t) in_size > input.size() - in.pos) return false;
				switch (current) {  // constructor arguments as upstream's Restore* members choose them
				case isInput:
					net.add(new CInput(Uid(uid), OutSize(in_size)), prev);
					if (!in.getFloats(net[uid]->mutable_input()->real_, in_size) || !in.getFloats(net[uid]->mutable_input()->imag_, in_size))
						return false;
					break;
				case isEmbedding: {
					int dim, slots, vocab;
					if (!in.get32(&dim) || !in.get32(&slots) || !in.get32(&vocab)) return false;
					if (dim <= 0 || slots <= 0 || vocab <= 0 || (long) dim * vocab != in_size) return false;
					net.add(new CEmbedding(Uid(uid), dim, slots, vocab), prev);
					if (!in.getFloats(net[uid]->mutable_input()->real_, in_size) || !in.getFloats(net[uid]->mutable_input()->imag_, in_size))
						return false;
					break;
				}
				case isLinear: {
					int in1, in2;
					if (!in.get32(&in1) || !in.get32(&in2)) return false;
					if (in1 <= 0 || in2 <= 0 || in2 % in1) return false;
					net.add(new Linear(Uid(uid), InSize(in1), InSize(in2)), prev);
					break;
				}
				case isHadamard: net.add(new Hadamard(Uid(uid), InSize(out_size), InSize(out_size)), prev); break;
				case isFourier: net.add(new FourierTrans(Uid(uid), InSize(in_size)), prev); break;
				case isTrianFourier: net.add(new TriangFourier(Uid(uid), InSize(in_size)), prev); break;
				case isResidual: net.add(new Residual(Uid(uid), InSize(out_size)), prev); break;
				case isSoftMax: net.add(new SoftMax(Uid(uid), InSize(in_size)), prev); break;
				case isCrossEntropy: net.add(new CrossEntropy(Uid(uid), InSize(in_size)), prev); break;
				case isL2Out: net.add(new L2Out(Uid(uid), InSize(in_size)), prev); break;
				case isCrelu: net.add(new CRelu(Uid(uid), InSize(out_size)), prev); break;
				case isGelu: net.add(new CGelu(Uid(uid), InSize(out_size)), prev); break;
				default: std::cerr << "Cannot restore layer of ID: " << current << std::endl; return false;
				}
			}
		} catch (const std::exception &e) {
			std::cerr << "Cannot restore: " << e.what() << std::endl;
			return false;
		}
		return true;
	}

	bool Restore(CNet &net, std::string file) {
		std::ifstream in(file, std::ifstream::in | std::ifstream::binary);
		if (!in) {
			std::cerr << "Cannot restore: cannot open: " << file << std::endl;
			return false;
		}
		std::ostringstream all;
		all << in.rdbuf();
		return RestoreFromString(net, all.str());
	}
};

// upstream CNet::save / restore (gpu/gpu_func.h:1103-1111): the host views are what is written, so a net that was trained
// on the device is saved after getInputsFromGpu()
inline bool CNet::save(std::string file) {
	ModelSaver saver;
	return saver.Save(*this, file);
}
inline bool CNet::restore(std::string file) {
	ModelSaver saver;
	return saver.Restore(*this, file);
}

#endif  // CNET_AMD_HOST_MODEL_SAVER_HPP_
