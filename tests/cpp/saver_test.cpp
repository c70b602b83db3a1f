// Host-only test of the facade's ModelSaver (cnet_amd/host/model_saver.hpp) against .mod files written by upstream
// CNet's own ModelSaver (tests/golden/*.mod, made by tests/golden/make_golden.py) and against the CPU oracle's reader.
// Makes no device call.  Usage: saver_test <dir with readme_net.mod and token_net.mod> <scratch dir>
#include <cstdio>
#include <fstream>
#include <sstream>

#include "cnet_amd/host/cnet.hpp"
#include "cnet_amd/host/data.hpp"
#include "oracle/cnet_oracle.hpp"

static int g_fail = 0;
static void expect(const std::string &what, bool ok) {
	printf("%s %s\n", ok ? "PASS" : "FAIL", what.c_str());
	if (!ok) g_fail++;
}

static std::string slurp(const std::string &path) {
	std::ifstream in(path, std::ifstream::binary);
	std::ostringstream all;
	all << in.rdbuf();
	return all.str();
}

// structure and parameters of a facade net against an oracle net restored from the same stream
static bool same_net(CNet &net, orc::Net &on) {
	if (net.functionList().size() != on.nodes().size()) return false;
	for (size_t k = 0; k < on.nodes().size(); ++k) {
		CFunc *f = net.functionList()[k];
		const orc::Node *nd = on.nodes()[k];
		if (f->uid() != nd->uid || f->typeId() != nd->kind || f->input().length_ != nd->in.n || f->outSize() != nd->out_size) return false;
		if (f->no_previous_func() != (int) nd->prev.size()) return false;
		for (size_t q = 0; q < nd->prev.size(); ++q)
			if (f->previous((int) q)->uid() != nd->prev[q]->uid) return false;
		if (f->no_outputs() != (int) nd->next.size()) return false;
		for (size_t q = 0; q < nd->next.size(); ++q)
			if (f->next((int) q)->uid() != nd->next[q]->uid || f->offset((int) q) != nd->offset[q]) return false;
		if (f->isInput() && memcmp(f->input().real_, nd->in.re, 2 * sizeof(float) * nd->in.n)) return false;
	}
	return true;
}

int main(int argc, char **argv) {
	if (argc < 3) {
		printf("usage: saver_test <golden dir> <scratch dir>\n");
		return 2;
	}
	const std::string dir = argv[1], tmp = argv[2];
	ModelSaver saver;
	for (const char *name : {"readme_net.mod", "token_net.mod"}) {
		const std::string blob = slurp(dir + "/" + name);
		expect(std::string(name) + ": fixture present", blob.size() > 100);
		CNet net;
		expect(std::string(name) + ": Restore(file)", saver.Restore(net, dir + "/" + name));
		orc::Net on;
		expect(std::string(name) + ": oracle reader accepts it", on.restore(blob));
		expect(std::string(name) + ": functions, wiring, offsets and parameters as stored", same_net(net, on));
		expect(std::string(name) + ": SaveToString reproduces the upstream bytes", saver.SaveToString(net) == blob);
		expect(std::string(name) + ": CNet::save writes them too", net.save(tmp + "/again.mod") && slurp(tmp + "/again.mod") == blob);
		CNet third;
		expect(std::string(name) + ": CNet::restore reads its own file", third.restore(tmp + "/again.mod") && same_net(third, on));
		// new functions added after a restore continue the uid sequence (impl/cnet.h:228-246)
		int uid = third.add(new CInput(OutSize(3)));
		expect(std::string(name) + ": uid counter continues after the stored uids", uid == (int) on.nodes().size() + 1);
	}
	{  // a net built through the API round-trips through a string
		CNet net;
		auto x = net.add(new CInput(OutSize(6)));
		auto f = net.add(new FourierTrans(InSize(6)), {x});
		auto t = net.add(new TriangFourier(InSize(6)), {f});
		auto r = net.add(new CRelu(InSize(6)), {t});
		auto g = net.add(new CGelu(InSize(6)), {r});
		auto s = net.add(new SoftMax(InSize(6)), {g});
		auto w = net.add(new CInput(Uid(40), OutSize(12)));
		auto l = net.add(new Linear(InSize(6), InSize(12)), {s, w});
		net.add(new L2Out(InSize(2)), {l});
		net.init_inputs(3);
		std::string blob = saver.SaveToString(net);
		CNet back;
		expect("API-built net: RestoreFromString", saver.RestoreFromString(back, blob));
		expect("API-built net: same bytes again", saver.SaveToString(back) == blob);
		expect("API-built net: explicit uid kept", back[40] && back[40]->input().length_ == 12 && back[w]->typeId() == isInput);
		orc::Net on;
		expect("API-built net: the oracle reads the facade's stream", on.restore(blob) && same_net(back, on) && on.save() == blob);

		// refusals
		CNet n1, n2, n3, n4;
		expect("wrong magic number is refused", !saver.RestoreFromString(n1, std::string("\x01\x02\x03\x04", 4) + blob.substr(4)));
		expect("truncated parameter block is refused", !saver.RestoreFromString(n2, blob.substr(0, 40)));
		std::string bad = blob;
		bad[7] = 99;  // type id of the first record
		expect("unknown type id is refused", !saver.RestoreFromString(n3, bad));
		expect("missing file is refused", !saver.Restore(n4, tmp + "/does_not_exist.mod"));
		expect("empty string is refused", !saver.RestoreFromString(n4, ""));
	}
	{  // MNIST idx reader and batching (upstream data/data.h:28-165), host only: the batch planes are pageable here
		const int count = 10;
		std::string img = tmp + "/images.idx3-ubyte", lab = tmp + "/labels.idx1-ubyte";
		{
			std::ofstream fi(img, std::ofstream::binary), fl(lab, std::ofstream::binary);
			const unsigned char hi[16] = {0, 0, 8, 3, 0, 0, 0, 10, 0, 0, 0, 28, 0, 0, 0, 28}, hl[8] = {0, 0, 8, 1, 0, 0, 0, 10};
			fi.write((const char *) hi, 16);
			fl.write((const char *) hl, 8);
			for (int s = 0; s < count; ++s) {
				for (int k = 0; k < 784; ++k) fi.put((char) (unsigned char) ((s * 31 + k * 7) & 255));
				fl.put((char) (s % 10));
			}
		}
		MnistDataReader reader;
		expect("MNIST reader: missing file is refused", !reader.Open(tmp + "/nope", lab, count));
		expect("MNIST reader: asking for more samples than the file holds is refused", !reader.Open(img, lab, count + 1));
		expect("MNIST reader: Open + readData", reader.Open(img, lab, count) && reader.readData() && reader.size() == count);
		bool ok = true;
		for (int s = 0; s < count; ++s)
			for (int k = 0; k < 784; ++k) {
				// a pixel byte read through a signed char becomes the real AND the imaginary part (data/data.h:129-132)
				float want = (float) (signed char) (unsigned char) ((s * 31 + k * 7) & 255);
				ok = ok && reader.realOf(s)[k] == want && reader.imagOf(s)[k] == want;
			}
		expect("MNIST reader: pixel conversion, labels", ok && reader.labelOf(3) == 3 && reader.labelOf(9) == 9);
		expect("hasNextBatch", reader.hasNextBatch(10) && !reader.hasNextBatch(11));
		InputBatch b = reader.nextBatch(4);
		expect("nextBatch(4): shape, labels, first rows", b.size() == 4 && b.sampleDim() == 784 && b.noOfLabels() == 4 && b.label(2) == 2 &&
				std::equal(b.realDataPtr(1), b.realDataPtr(1) + 784, reader.realOf(1)) && !b.isPinned());
		reader.nextBatch(b);
		expect("refill continues with samples 4..7", b.label(0) == 4 && b.label(3) == 7 && std::equal(b.imagDataPtr(3), b.imagDataPtr(3) + 784, reader.imagOf(7)));
		reader.nextBatch(b);
		expect("wrap-around at the end of the data (8, 9, 0, 1)", b.label(0) == 8 && b.label(1) == 9 && b.label(2) == 0 && b.label(3) == 1);
		reader.shuffle(5);
		std::vector<int> seen(10, 0);
		InputBatch all(10, 784);
		// two positions were consumed after the wrap: the next ten positions still cover every sample once
		reader.nextBatch(all);
		bool rows_match = true;
		for (int r = 0; r < 10; ++r) {
			seen[all.label(r)]++;
			rows_match = rows_match && std::equal(all.realDataPtr(r), all.realDataPtr(r) + 784, reader.realOf(all.label(r)));
		}
		bool perm = true, moved = false;
		for (int r = 0; r < 10; ++r) {
			perm = perm && seen[r] == 1;
			moved = moved || all.label(r) != (r + 2) % 10;
		}
		expect("shuffle(seed) is a permutation that keeps rows and labels together", perm && moved && rows_match);
		// short samples are zero padded, as InputBatch::add upstream (impl/batch.h)
		InputBatch pad(2, 5);
		pad.add({{1.f, 2.f}, {3.f, 4.f}}, 7);
		pad.add({{5.f, 6.f}}, 1);
		expect("InputBatch pads short samples with zeros", pad.realDataPtr(0)[1] == 3.f && pad.imagDataPtr(0)[1] == 4.f && pad.realDataPtr(0)[2] == 0.f &&
				pad.realDataPtr(1)[0] == 5.f && pad.imagDataPtr(1)[4] == 0.f && pad.label(0) == 7);
		InputBatch moved_to = std::move(pad);
		expect("InputBatch moves", moved_to.realDataPtr(1)[0] == 5.f && moved_to.size() == 2);
	}
	printf("saver: %d failure(s)\n", g_fail);
	return g_fail ? 1 : 0;
}
