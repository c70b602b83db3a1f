"""Writes a stand-in for the device library, generated from include/cnet_hip.h: every entry point exists and succeeds, memory
calls work on host memory, and the graph calls keep track of the handles they gave out (a replay or a destroy of a handle
that is not alive aborts).  Nothing is computed.  The C++ facade built against it runs its whole control flow on the CPU,
under AddressSanitizer, which is what tests/test_host_facade_stub.py does.

    python tests/cpp/make_stub_backend.py <header> <output .cpp>
"""
import re
import sys


def generate(header_path, out_path):
    text = re.sub(r'/\*.*?\*/', '', open(header_path).read(), flags=re.S)
    decls = re.findall(r'\n((?:int|void \*|const char \*)\s*cnet_\w+\s*\([^;]*?\));', text)
    special = {'cnet_graph_end', 'cnet_graph_launch', 'cnet_graph_destroy', 'cnet_graph_begin', 'cnet_alloc', 'cnet_host_alloc',
               'cnet_free', 'cnet_host_free', 'cnet_memcpy_h2d', 'cnet_memcpy_d2h', 'cnet_memcpy_d2d', 'cnet_memcpy_h2d_async',
               'cnet_memcpy_d2h_async', 'cnet_upload_async', 'cnet_upload_zero', 'cnet_upload_pair', 'cnet_upload_gather_rows', 'cnet_gather_rows', 'cnet_memset_zero', 'cnet_last_error', 'cnet_stream',
               'cnet_get_device_info'}
    out = ['#include "cnet_hip.h"\n#include <cstdio>\n#include <cstdlib>\n#include <cstring>\n#include <set>\nextern "C" {\n']
    seen = set()
    for d in decls:
        name = re.search(r'(cnet_\w+)', d).group(1)
        seen.add(name)
        if name not in special:
            out.append(d.strip() + ' { return 0; }\n')
    missing = special - seen
    assert not missing, "the header no longer declares %s" % sorted(missing)
    out.append('''static std::set<void *> live;
static bool recording = false;
int cnet_graph_begin(void) { if (recording) { fprintf(stderr, "stub: nested cnet_graph_begin\\n"); abort(); } recording = true; return 0; }
int cnet_graph_end(void **g) { if (!recording) return -2; recording = false; if (g) { *g = malloc(8); live.insert(*g); } return 0; }
int cnet_graph_launch(void *g) { if (!live.count(g)) { fprintf(stderr, "stub: launch of a graph that is not alive\\n"); abort(); } *(volatile char *) g; return 0; }
int cnet_graph_destroy(void *g) { if (!g) return 0; if (!live.count(g)) { fprintf(stderr, "stub: destroy of a graph that is not alive\\n"); abort(); } live.erase(g); free(g); return 0; }
int cnet_alloc(size_t b, void **o) { *o = calloc(b ? b : 1, 1); return 0; }
int cnet_host_alloc(size_t b, void **o) { *o = calloc(b ? b : 1, 1); return 0; }
int cnet_free(void *p) { free(p); return 0; }
int cnet_host_free(void *p) { free(p); return 0; }
int cnet_memcpy_h2d(void *d, const void *s, size_t b) { memcpy(d, s, b); return 0; }
int cnet_memcpy_d2h(void *d, const void *s, size_t b) { memcpy(d, s, b); return 0; }
int cnet_memcpy_d2d(void *d, const void *s, size_t b) { memmove(d, s, b); return 0; }
int cnet_memcpy_h2d_async(void *d, const void *s, size_t b) { memcpy(d, s, b); return 0; }
int cnet_memcpy_d2h_async(void *d, const void *s, size_t b) { memcpy(d, s, b); return 0; }
int cnet_upload_async(void *d, const void *s, size_t b) { memcpy(d, s, b); return 0; }
int cnet_upload_zero(void *d, size_t b) { memset(d, 0, b); return 0; }
int cnet_upload_pair(void *d0, const void *s0, size_t b0, void *d1, const void *s1, size_t b1) { if (b0) memcpy(d0, s0, b0); if (b1) memcpy(d1, s1, b1); return 0; }
int cnet_upload_gather_rows(float *d, int64_t ldd, int64_t dps, const float *s, int64_t lds, int64_t sps, int planes, int src_rows,
		const int32_t *idx, int32_t *dl, const int32_t *sl, int rows, int cols) {
	for (int p = 0; p < planes; ++p)
		for (int r = 0; r < rows; ++r) {
			if (idx[r] < 0 || idx[r] >= src_rows) { fprintf(stderr, "stub: gather index outside the table\\n"); abort(); }
			memcpy(d + p * dps + (int64_t) r * ldd, s + p * sps + (int64_t) idx[r] * lds, cols * sizeof(float));
		}
	if (dl) for (int r = 0; r < rows; ++r) dl[r] = sl[idx[r]];
	return 0;
}
int cnet_gather_rows(float *d, int64_t ldd, int64_t dps, const float *s, int64_t lds, int64_t sps, int planes, int src_rows,
		const int32_t *idx, int32_t *dl, const int32_t *sl, int rows, int cols) {
	return cnet_upload_gather_rows(d, ldd, dps, s, lds, sps, planes, src_rows, idx, dl, sl, rows, cols);
}
int cnet_memset_zero(void *d, size_t b) { memset(d, 0, b); return 0; }
const char *cnet_last_error(void) { return "stub"; }
void *cnet_stream(void) { return 0; }
int cnet_get_device_info(cnet_device_info *o) { memset(o, 0, sizeof(*o)); return 0; }
}
''')
    open(out_path, 'w').write(''.join(out))


if __name__ == "__main__":
    generate(sys.argv[1], sys.argv[2])
