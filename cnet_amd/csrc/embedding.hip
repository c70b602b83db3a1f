// CEmbedding: row gather with zero padding, and the deterministic dzs scatter-add.
#include "common.hpp"

#include <hipcub/hipcub.hpp>

namespace {

constexpr int TPB = 256;

// y[row][slot*dim + d] = table[token][d], zeros for token < 0   (impl/embed.h:109-131 upstream).  An id >= vocab, which
// upstream rejects with an assert on the host, is treated as padding here: a wrong id must not become a wild access.
template <int V>
__global__ __launch_bounds__(TPB) void embedding_fwd_kernel(const float *__restrict__ tr, const float *__restrict__ ti, int dim,
		const int *__restrict__ tokens, float *__restrict__ yr, float *__restrict__ yi, long ldy, long positions, int slots, int vocab) {
	const long dv = dim / V;
	const long idx = (long) blockIdx.x * TPB + threadIdx.x;
	if (idx >= positions * dv) return;
	const long pos = idx / dv;
	const int d = (int) (idx - pos * dv) * V;
	int tok = tokens[pos];
	if (tok >= vocab) tok = -1;
	const long row = pos / slots, slot = pos - row * slots;
	const long dst = row * ldy + slot * dim + d;
	if (V == 4) {
		float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
		if (tok >= 0) {
			a = *reinterpret_cast<const float4 *>(tr + (long) tok * dim + d);
			b = *reinterpret_cast<const float4 *>(ti + (long) tok * dim + d);
		}
		*reinterpret_cast<float4 *>(yr + dst) = a;
		*reinterpret_cast<float4 *>(yi + dst) = b;
	} else {
		yr[dst] = tok >= 0 ? tr[(long) tok * dim + d] : 0.f;
		yi[dst] = tok >= 0 ? ti[(long) tok * dim + d] : 0.f;
	}
}

__global__ __launch_bounds__(TPB) void iota_kernel(int *__restrict__ p, long n) {
	const long i = (long) blockIdx.x * TPB + threadIdx.x;
	if (i < n) p[i] = (int) i;
}

// keys/pos: token ids sorted ascending (stable), pos = original (row, slot) position.  One workgroup per sorted
// index; only the head of a run of equal tokens works: it adds the run's dzs rows in position order.
__global__ __launch_bounds__(TPB) void embedding_bwd_kernel(const int *__restrict__ keys, const int *__restrict__ pos, long n,
		const float *__restrict__ gr, const float *__restrict__ gi, long ldg, int slots, int dim, int vocab, float *__restrict__ dr,
		float *__restrict__ di) {
	const long i = blockIdx.x;
	const int tok = keys[i];
	if (tok < 0 || tok >= vocab) return;
	if (i > 0 && keys[i - 1] == tok) return;
	for (int d = threadIdx.x; d < dim; d += TPB) {
		float ar = dr[(long) tok * dim + d], ai = di[(long) tok * dim + d];
		for (long j = i; j < n && keys[j] == tok; ++j) {
			const long p = pos[j];
			const long row = p / slots, slot = p - row * slots;
			ar += gr[row * ldg + slot * dim + d];
			ai += gi[row * ldg + slot * dim + d];
		}
		dr[(long) tok * dim + d] = ar;
		di[(long) tok * dim + d] = ai;
	}
}

}  // namespace

using namespace cnet;

extern "C" {

int cnet_memset_zero(void *dst, size_t bytes);

int cnet_embedding_fwd(const float *table_re, const float *table_im, int dim, int vocab, const int32_t *tokens, float *y_re,
		float *y_im, int64_t ldy, int rows, int slots) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && slots > 0 && dim > 0 && vocab > 0);
	if (!rows) return CNET_OK;
	CNET_CHECK_ARG(table_re && table_im && tokens && y_re && y_im && ldy >= (int64_t) slots * dim);
	const long positions = (long) rows * slots;
	const bool vec = dim % 4 == 0 && ldy % 4 == 0 && aligned16(table_re) && aligned16(table_im) && aligned16(y_re) && aligned16(y_im);
	const long work = positions * (dim / (vec ? 4 : 1));
	dim3 grid((unsigned) ((work + TPB - 1) / TPB));
	if (vec)
		hipLaunchKernelGGL(embedding_fwd_kernel<4>, grid, dim3(TPB), 0, rt().stream, table_re, table_im, dim, tokens, y_re, y_im, (long) ldy,
				positions, slots, vocab);
	else
		hipLaunchKernelGGL(embedding_fwd_kernel<1>, grid, dim3(TPB), 0, rt().stream, table_re, table_im, dim, tokens, y_re, y_im, (long) ldy,
				positions, slots, vocab);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_embedding_bwd(const int32_t *tokens, const float *g_dzs_re, const float *g_dzs_im, int64_t ldg, float *table_dzs_re,
		float *table_dzs_im, int dim, int vocab, int rows, int slots, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(rows >= 0 && slots > 0 && dim > 0 && vocab > 0);
	CNET_CHECK_ARG(tokens && g_dzs_re && g_dzs_im && table_dzs_re && table_dzs_im && ldg >= (int64_t) slots * dim);
	if (!accumulate) {
		int rc = cnet_memset_zero(table_dzs_re, (size_t) vocab * dim * sizeof(float));
		if (rc) return rc;
		rc = cnet_memset_zero(table_dzs_im, (size_t) vocab * dim * sizeof(float));
		if (rc) return rc;
	}
	if (!rows) return CNET_OK;
	const long n = (long) rows * slots;
	CNET_CHECK_ARG(n < (1L << 31));
	// stable radix sort of (token, position): equal tokens stay in (row, slot) order
	size_t sort_bytes = 0;
	CNET_HIP(hipcub::DeviceRadixSort::SortPairs(nullptr, sort_bytes, (const int *) nullptr, (int *) nullptr, (const int *) nullptr,
			(int *) nullptr, (int) n, 0, 32, rt().stream));
	const size_t ints = ((size_t) n + 63) / 64 * 64;
	char *ws = (char *) workspace(3 * ints * sizeof(int) + sort_bytes + 256);
	if (!ws) return CNET_ERR_OUT_OF_MEMORY;
	int *pos_in = (int *) ws, *keys_out = pos_in + ints, *pos_out = keys_out + ints;
	void *sort_ws = (void *) (pos_out + ints);
	hipLaunchKernelGGL(iota_kernel, dim3((unsigned) ((n + TPB - 1) / TPB)), dim3(TPB), 0, rt().stream, pos_in, n);
	CNET_LAUNCH_CHECK();
	CNET_HIP(hipcub::DeviceRadixSort::SortPairs(sort_ws, sort_bytes, (const int *) tokens, keys_out, (const int *) pos_in, pos_out, (int) n, 0,
			32, rt().stream));
	hipLaunchKernelGGL(embedding_bwd_kernel, dim3((unsigned) n), dim3(TPB), 0, rt().stream, keys_out, pos_out, n, g_dzs_re, g_dzs_im,
			(long) ldg, slots, dim, vocab, table_dzs_re, table_dzs_im);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

}  // extern "C"
