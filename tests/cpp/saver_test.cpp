// Host-only test of the facade's ModelSaver (cnet_amd/host/model_saver.hpp) against .mod files written by upstream
// CNet's own ModelSaver (tests/golden/*.mod, made by tests/golden/make_golden.py) and against the CPU oracle's reader.
// Makes no device call.  Usage: saver_test <dir with readme_net.mod and token_net.mod> <scratch dir>
#include <cstdio>
#include <fstream>
#include <sstream>

#include "cnet_amd/host/cnet.hpp"
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
	printf("saver: %d failure(s)\n", g_fail);
	return g_fail ? 1 : 0;
}
