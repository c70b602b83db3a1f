// Internal declarations shared by the translation units of libcnet_hip.so.
#ifndef CNET_CSRC_COMMON_HPP_
#define CNET_CSRC_COMMON_HPP_

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdlib>
#include <cstdio>

#include "cnet_hip.h"

namespace cnet {

struct Runtime {
	bool ready = false;
	int device = -1;
	hipStream_t own_stream = nullptr;
	hipStream_t stream = nullptr;   // the stream in use (own_stream unless the caller supplied one)
	// host -> device uploads that overlap compute run on their own stream (default priority, like the compute stream);
	// the two events order the streams against each other
	hipStream_t upload_stream = nullptr;
	hipEvent_t upload_done = nullptr, compute_done = nullptr;
	static constexpr int kMarkers = 8;
	hipEvent_t marker[kMarkers] = {};  // caller-numbered points of the compute stream
	hipEvent_t upload_marker[kMarkers] = {};  // caller-numbered points of the upload stream
	// tickets: points of either stream the HOST can wait for one by one (has this copy left its page-locked source?).
	// A ring of events per stream; a slot that was reused stands for a later point of the same stream, so waiting on it
	// can only wait longer, never too short.
	static constexpr int kTickets = 32;
	hipEvent_t ticket_event[2][kTickets] = {};
	int64_t tickets_issued[2] = {0, 0};
	bool capturing = false;  // between cnet_graph_begin and cnet_graph_end: nothing may allocate or wait
	hipDeviceProp_t prop;
	// grow-only scratch for two-stage deterministic reductions (never allocated inside a hot loop twice
	// for the same size)
	void *workspace = nullptr;
	size_t workspace_bytes = 0;
	// a second buffer of the same kind, for an operand that a product reads while it may itself use the workspace for partial
	// sums (the folded samples of the transform of real input)
	void *operand_workspace = nullptr;
	size_t operand_workspace_bytes = 0;
	// A recorded graph holds the workspace address it was recorded with: while any recording exists, a workspace that
	// has to grow is retired (kept until shutdown) instead of freed.
	// Each live recording is kept as (executable, the graph it was instantiated from): the template graph lives as long
	// as its executable, so that nothing that still walks its nodes (a tracing tool) finds them gone, and shutdown can
	// destroy what the caller left behind.
	int graphs_alive = 0;
	static constexpr int kGraphs = 256;
	hipGraphExec_t graph_exec[kGraphs] = {};
	hipGraph_t graph_template[kGraphs] = {};
	static constexpr int kRetired = 16;
	void *retired[kRetired] = {};
	int retired_count = 0;
};

Runtime &rt();
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char *what);
// returns nullptr (and records the error) when the allocation fails
void *workspace(size_t bytes);
void *operand_workspace(size_t bytes);  // the second buffer (Runtime::operand_workspace); same rules
// every hipFuncSetAttribute the matrix kernels need, made once, outside any stream capture (cgemm.hip)
int cgemm_prime_attributes();

#define CNET_REQUIRE_INIT()                                                              \
	do {                                                                                 \
		if (!cnet::rt().ready) return cnet::fail(CNET_ERR_NOT_INITIALIZED, "%s: cnet_init() has not been called", __func__); \
	} while (0)

// entry points that wait for the device or allocate cannot be recorded into a graph
#define CNET_NOT_IN_CAPTURE()                                                                                                \
	do {                                                                                                                     \
		if (cnet::rt().capturing) return cnet::fail(CNET_ERR_UNSUPPORTED, "%s: not allowed between cnet_graph_begin and cnet_graph_end", __func__); \
	} while (0)

#define CNET_HIP(call)                                             \
	do {                                                           \
		hipError_t e__ = (call);                                   \
		if (e__ != hipSuccess) return cnet::hip_fail(e__, #call);  \
	} while (0)

#define CNET_CHECK_ARG(cond)                                                                   \
	do {                                                                                       \
		if (!(cond)) return cnet::fail(CNET_ERR_INVALID_ARGUMENT, "%s: requirement failed: %s", __func__, #cond); \
	} while (0)

#define CNET_LAUNCH_CHECK()                                            \
	do {                                                               \
		hipError_t e__ = hipGetLastError();                            \
		if (e__ != hipSuccess) return cnet::hip_fail(e__, __func__);   \
	} while (0)

// Second stage of the deterministic column sums: adds `count` partial values that lie `stride` floats apart, in index
// order, requesting eight of them before the first is added (the additions stay sequential, the loads overlap).
__device__ __forceinline__ float ordered_sum(const float *__restrict__ first, long stride, int count) {
	float s = 0.f;
	int k = 0;
	for (; k + 8 <= count; k += 8) {
		float v[8];
#pragma unroll
		for (int u = 0; u < 8; ++u) v[u] = first[(long) (k + u) * stride];
#pragma unroll
		for (int u = 0; u < 8; ++u) s += v[u];
	}
	for (; k < count; ++k) s += first[(long) k * stride];
	return s;
}

// tanh-GELU of one real plane value and its derivative (impl/relu.h:119-131 upstream); shared by the elementwise kernels
// and the matrix-product epilogue that applies the CGelu of a Linear's result, so both give the same bits.
// With a = sqrt(2/pi) (t + 0.044715 t^3) and e = exp(-2a): (1 + tanh a)/2 = 1/(1 + e) and 1/(2 cosh^2 a) = 2e/(1 + e)^2,
// so one hardware exponential and one reciprocal (about 1 ulp each) stand in for tanhf and coshf of the CPU path, without
// the cancellation of 1 + tanh a for negative a.  a is kept above -43 so that e stays finite (e = inf would give inf * 0).
__device__ __forceinline__ float gelu_gate(float t, float &e) {
	const float c = 0.7978845608028654f;  // sqrt(2/pi)
	const float arg = fmaxf(c * (t + 0.044715f * t * t * t), -43.0f);
	e = __builtin_amdgcn_exp2f(-2.8853900817779268f * arg);  // exp(-2 arg) = 2^(-2 log2(e) arg)
	return __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ float gelu_value(float t) {
	float e;
	return t * gelu_gate(t, e);
}

__device__ __forceinline__ float gelu_slope(float t) {
	const float c = 0.7978845608028654f;
	float e;
	const float sig = gelu_gate(t, e);
	const float half_sech2 = 2.0f * ((e * sig) * sig);
	return sig + t * half_sech2 * c * (1.0f + 3.0f * 0.044715f * t * t);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The cache policy of a launch that touches `planes` fp32 planes of `elems` elements each.  Operands that fit the 256 MB
// memory-side cache together are left there for the next kernel (plain accesses: with hints the next kernel no longer
// finds them and loses up to 20 %).  Beyond that everything streams from and to HBM, and which side carries the streaming
// hint decides up to 30 % of the rate.  Measured kernel by kernel at [8192 x 4096] (the same ranking on three machines,
// with the operands in other buffers and at other offsets), ms under: the hint on loads and stores (1) / plain loads,
// streaming stores (2) / streaming loads, device-scope stores (3) / no hints:
//   two planes read:    CGelu forward .086 / .074 / .076 / .097; Hadamard + CGelu forward (four written) .137 / .113 / .138 / .149;
//                       Residual backward of a pair (four written) .144 / .113 / .147 / .155; L2Out backward .142 / .113 / .148 / .162
//   four read, two written: CGelu backward of a pair .129 / .152 / .116 / .152; shared-weight Hadamard backward of a pair
//                       .132 / .146 / .121 / .158; SoftMax backward of a pair .129 / .141 / .115 / .148; but Residual forward
//                       .109 / .144 / .136 / .150
//   six read, four written: CGelu backward .221 / .251 / .249 / .257; Residual + CGelu backward of a pair .222 / .245 / .228 / .239
//   four read and written (the SGD step) .179 / .187 / .178 / .195; six (the Adam-style step) .279 / .318 / .304 / .315
// A probe kernel that only moves R planes to W planes ranks the three the same way.  `when_streaming` is the caller's entry
// of that table.
constexpr int ST_BOTH = 1, ST_STORES = 2, ST_LOADS = 3;
inline int stream_policy(int when_streaming, int planes, long elems) {
	static const int forced = [] {
		const char *e = getenv("CNET_STREAM_POLICY");  // tuning override: 0..3 for every launch beyond the cache size
		return e ? atoi(e) : -1;
	}();
	static const long cache_bytes = [] {
		const char *e = getenv("CNET_STREAM_MIN_MB");  // tuning override of the footprint from which a launch counts as streaming
		return (e ? atol(e) : 256L) << 20;
	}();
	if ((long) planes * elems * 4 <= cache_bytes) return 0;
	return forced >= 0 && forced <= 3 ? forced : when_streaming;
}


}  // namespace cnet

#endif
