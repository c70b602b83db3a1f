// Lifetime, memory and stream entry points of libcnet_hip.so.
#include "common.hpp"

#include <cstring>
#include <map>
#include <string>

namespace cnet {

static thread_local char g_error[1024] = "";
static Runtime g_rt;

Runtime &rt() { return g_rt; }

int fail(int code, const char *fmt, ...) {
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(g_error, sizeof(g_error), fmt, ap);
	va_end(ap);
	return code;
}

int hip_fail(hipError_t e, const char *what) {
	snprintf(g_error, sizeof(g_error), "HIP error %d (%s) in %s", (int) e, hipGetErrorString(e), what);
	return e == hipErrorOutOfMemory ? CNET_ERR_OUT_OF_MEMORY : CNET_ERR_HIP;
}

// one grow-only buffer (see Runtime::workspace): at least `bytes` long, or nullptr with the error recorded
static void *grown(void *&buf, size_t &have, size_t bytes) {
	Runtime &r = rt();
	if (bytes <= have) return buf;
	if (r.capturing) {
		fail(CNET_ERR_UNSUPPORTED, "the workspace would have to grow while a graph is being recorded: run the same calls once before recording");
		return nullptr;
	}
	if (buf) {
		if (r.graphs_alive > 0) {  // a recording may replay kernels that use the old buffer
			if (r.retired_count == Runtime::kRetired) {
				fail(CNET_ERR_UNSUPPORTED, "the workspace had to grow %d times while recorded graphs exist: destroy the graphs first", Runtime::kRetired);
				return nullptr;
			}
			r.retired[r.retired_count++] = buf;
		} else {
			// queued kernels may still read the old buffer
			hipStreamSynchronize(r.stream);
			hipFree(buf);
		}
		buf = nullptr;
		have = 0;
	}
	size_t want = bytes + bytes / 2;
	hipError_t e = hipMalloc(&buf, want);
	if (e != hipSuccess) {
		hip_fail(e, "workspace hipMalloc");
		buf = nullptr;
		return nullptr;
	}
	have = want;
	return buf;
}

void *workspace(size_t bytes) { return grown(rt().workspace, rt().workspace_bytes, bytes); }

void *operand_workspace(size_t bytes) { return grown(rt().operand_workspace, rt().operand_workspace_bytes, bytes); }

void release_twiddles();  // cdft.hip
int init_static_scratch(int device);  // reduce.hip

// destroys whatever streams and events exist (also the leftovers of an initialisation that failed half-way)
static void destroy_streams(Runtime &r) {
	if (r.upload_stream) {
		hipStreamSynchronize(r.upload_stream);
		hipStreamDestroy(r.upload_stream);
	}
	if (r.upload_done) hipEventDestroy(r.upload_done);
	if (r.compute_done) hipEventDestroy(r.compute_done);
	for (auto &m : r.marker) {
		if (m) hipEventDestroy(m);
		m = nullptr;
	}
	for (auto &m : r.upload_marker) {
		if (m) hipEventDestroy(m);
		m = nullptr;
	}
	for (auto &ring : r.ticket_event)
		for (auto &e : ring) {
			if (e) hipEventDestroy(e);
			e = nullptr;
		}
	r.tickets_issued[0] = r.tickets_issued[1] = 0;
	if (r.own_stream) hipStreamDestroy(r.own_stream);
	r.upload_stream = r.own_stream = r.stream = nullptr;
	r.upload_done = r.compute_done = nullptr;
}

static int create_streams(Runtime &r) {
	CNET_HIP(hipStreamCreateWithFlags(&r.own_stream, hipStreamNonBlocking));
	r.stream = r.own_stream;
	CNET_HIP(hipStreamCreateWithFlags(&r.upload_stream, hipStreamNonBlocking));
	CNET_HIP(hipEventCreateWithFlags(&r.upload_done, hipEventDisableTiming));
	CNET_HIP(hipEventCreateWithFlags(&r.compute_done, hipEventDisableTiming));
	for (auto &m : r.marker) CNET_HIP(hipEventCreateWithFlags(&m, hipEventDisableTiming));
	for (auto &m : r.upload_marker) CNET_HIP(hipEventCreateWithFlags(&m, hipEventDisableTiming));
	for (auto &ring : r.ticket_event)
		for (auto &e : ring) CNET_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
	return CNET_OK;
}

}  // namespace cnet

using namespace cnet;

extern "C" {

int cnet_init(int device) {
	Runtime &r = rt();
	if (r.ready) {
		if (r.device == device) return CNET_OK;
		return fail(CNET_ERR_INVALID_ARGUMENT, "cnet_init: already initialised on device %d", r.device);
	}
	int count = 0;
	CNET_HIP(hipGetDeviceCount(&count));
	if (device < 0 || device >= count) return fail(CNET_ERR_INVALID_ARGUMENT, "cnet_init: device %d of %d", device, count);
	CNET_HIP(hipSetDevice(device));
	CNET_HIP(hipGetDeviceProperties(&r.prop, device));
	if (strncmp(r.prop.gcnArchName, "gfx950", 6) != 0)
		return fail(CNET_ERR_UNSUPPORTED, "cnet_init: kernels are built for gfx950 only, device is %s", r.prop.gcnArchName);
	const int rc = create_streams(r);
	if (rc != CNET_OK) {
		destroy_streams(r);
		return rc;
	}
	const int rc_scratch = init_static_scratch(device);
	if (rc_scratch != CNET_OK) {
		destroy_streams(r);
		return rc_scratch;
	}
	r.device = device;
	r.ready = true;
	return CNET_OK;
}

int cnet_shutdown(void) {
	Runtime &r = rt();
	if (!r.ready) return CNET_OK;
	int rc = CNET_OK;
	if (r.capturing) {  // an open recording is ended and dropped: the stream cannot be waited for while it records
		hipGraph_t open_graph = nullptr;
		(void) hipStreamEndCapture(r.stream, &open_graph);
		if (open_graph) (void) hipGraphDestroy(open_graph);
		(void) hipGetLastError();
		r.capturing = false;
	}
	hipError_t sync_err = hipStreamSynchronize(r.stream);
	if (sync_err != hipSuccess) rc = hip_fail(sync_err, "cnet_shutdown: hipStreamSynchronize");
	// recordings the caller did not destroy: their handles die with the library's buffers
	for (int k = 0; k < Runtime::kGraphs; ++k) {
		if (r.graph_exec[k]) (void) hipGraphExecDestroy(r.graph_exec[k]);
		if (r.graph_template[k]) (void) hipGraphDestroy(r.graph_template[k]);
		r.graph_exec[k] = nullptr;
		r.graph_template[k] = nullptr;
	}
	release_twiddles();
	if (r.workspace) hipFree(r.workspace);
	r.workspace = nullptr;
	r.workspace_bytes = 0;
	if (r.operand_workspace) hipFree(r.operand_workspace);
	r.operand_workspace = nullptr;
	r.operand_workspace_bytes = 0;
	for (int k = 0; k < r.retired_count; ++k) hipFree(r.retired[k]);
	r.retired_count = 0;
	r.graphs_alive = 0;
	destroy_streams(r);
	r.ready = false;
	r.device = -1;
	return rc;
}

int cnet_get_device_info(cnet_device_info *out) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(out != nullptr);
	Runtime &r = rt();
	memset(out, 0, sizeof(*out));
	snprintf(out->name, sizeof(out->name), "%s", r.prop.name);
	snprintf(out->arch, sizeof(out->arch), "%s", r.prop.gcnArchName);
	out->compute_units = r.prop.multiProcessorCount;
	out->clock_khz = r.prop.clockRate;
	out->wavefront_size = r.prop.warpSize;
	out->lds_bytes_per_block = (int) r.prop.maxSharedMemoryPerMultiProcessor;
	out->hbm_bytes = (int64_t) r.prop.totalGlobalMem;
	out->fp32_matrix_peak_tflops = 256.0 * r.prop.multiProcessorCount * (r.prop.clockRate * 1e3) / 1e12;
	return CNET_OK;
}

const char *cnet_last_error(void) { return g_error; }

void *cnet_stream(void) { return rt().ready ? (void *) rt().stream : nullptr; }

int cnet_set_stream(void *hip_stream) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	Runtime &r = rt();
	CNET_HIP(hipStreamSynchronize(r.stream));
	r.stream = hip_stream ? (hipStream_t) hip_stream : r.own_stream;
	return CNET_OK;
}

int cnet_sync(void) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_HIP(hipStreamSynchronize(rt().stream));
	return CNET_OK;
}

int cnet_alloc(size_t bytes, void **out) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_CHECK_ARG(out != nullptr);
	*out = nullptr;
	if (bytes == 0) return CNET_OK;
	CNET_HIP(hipMalloc(out, bytes));
	return CNET_OK;
}

int cnet_free(void *ptr) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	if (!ptr) return CNET_OK;
	CNET_HIP(hipStreamSynchronize(rt().stream));
	CNET_HIP(hipFree(ptr));
	return CNET_OK;
}

int cnet_memcpy_h2d(void *dst, const void *host_src, size_t bytes) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	if (!bytes) return CNET_OK;
	CNET_CHECK_ARG(dst && host_src);
	// pageable source: hipMemcpyAsync stages and returns after the copy was consumed from the host buffer
	CNET_HIP(hipMemcpyAsync(dst, host_src, bytes, hipMemcpyHostToDevice, rt().stream));
	CNET_HIP(hipStreamSynchronize(rt().stream));
	return CNET_OK;
}

// page-locked ranges handed out by cnet_host_alloc: only these may be read by a kernel directly (cnet_upload_pair); a
// pointer into pageable memory there would be a memory fault on the device instead of an error code
static std::map<uintptr_t, size_t> &pinned_ranges() {
	static std::map<uintptr_t, size_t> ranges;
	return ranges;
}
static bool in_pinned_range(const void *p, size_t bytes) {
	if (!bytes) return true;
	auto &ranges = pinned_ranges();
	auto it = ranges.upper_bound((uintptr_t) p);
	if (it == ranges.begin()) return false;
	--it;
	return (uintptr_t) p + bytes <= it->first + it->second;
}

int cnet_host_alloc(size_t bytes, void **out) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_CHECK_ARG(out != nullptr);
	*out = nullptr;
	if (bytes == 0) return CNET_OK;
	CNET_HIP(hipHostMalloc(out, bytes, hipHostMallocDefault));
	pinned_ranges()[(uintptr_t) *out] = bytes;
	return CNET_OK;
}

int cnet_host_free(void *ptr) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	if (!ptr) return CNET_OK;
	// copies queued from this buffer must have left it
	CNET_HIP(hipStreamSynchronize(rt().stream));
	CNET_HIP(hipStreamSynchronize(rt().upload_stream));
	pinned_ranges().erase((uintptr_t) ptr);
	CNET_HIP(hipHostFree(ptr));
	return CNET_OK;
}

int cnet_memcpy_h2d_async(void *dst, const void *pinned_src, size_t bytes) {
	CNET_REQUIRE_INIT();
	if (!bytes) return CNET_OK;
	CNET_CHECK_ARG(dst && pinned_src);
	CNET_HIP(hipMemcpyAsync(dst, pinned_src, bytes, hipMemcpyHostToDevice, rt().stream));
	return CNET_OK;
}

int cnet_memcpy_d2h_async(void *pinned_dst, const void *src, size_t bytes) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // a recording would replay the copy into the same host address
	if (!bytes) return CNET_OK;
	CNET_CHECK_ARG(pinned_dst && src);
	CNET_HIP(hipMemcpyAsync(pinned_dst, src, bytes, hipMemcpyDeviceToHost, rt().stream));
	return CNET_OK;
}

int cnet_upload_async(void *dst, const void *pinned_src, size_t bytes) {
	CNET_REQUIRE_INIT();
	if (!bytes) return CNET_OK;
	CNET_CHECK_ARG(dst && pinned_src);
	CNET_HIP(hipMemcpyAsync(dst, pinned_src, bytes, hipMemcpyHostToDevice, rt().upload_stream));
	return CNET_OK;
}

// two regions of page-locked host memory to the device in one launch: the lanes read the host memory over the link
__global__ __launch_bounds__(256) void upload_pair_kernel(uint32_t *__restrict__ d0, const uint32_t *__restrict__ s0, long words0,
		long vec0, uint32_t *__restrict__ d1, const uint32_t *__restrict__ s1, long words1) {
	const long i = (long) blockIdx.x * blockDim.x + threadIdx.x, stride = (long) gridDim.x * blockDim.x;
	for (long k = i; k < vec0; k += stride) reinterpret_cast<uint4 *>(d0)[k] = reinterpret_cast<const uint4 *>(s0)[k];
	for (long k = 4 * vec0 + i; k < words0; k += stride) d0[k] = s0[k];
	for (long k = i; k < words1; k += stride) d1[k] = s1[k];
}

int cnet_upload_pair(void *dst0, const void *pinned_src0, size_t bytes0, void *dst1, const void *pinned_src1, size_t bytes1) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // work on the upload stream: never part of a recording
	CNET_CHECK_ARG((bytes0 == 0 || (dst0 && pinned_src0)) && (bytes1 == 0 || (dst1 && pinned_src1)));
	CNET_CHECK_ARG(bytes0 % 4 == 0 && bytes1 % 4 == 0);
	if (!bytes0 && !bytes1) return CNET_OK;
	Runtime &r = rt();
	// Small batches: a copy queued through the runtime costs the host 3-5 us each and takes the copy engine's start-up time
	// to arrive; one kernel launch that reads the page-locked memory directly does both regions.  Large ones stay with the
	// copy engine, which moves them without occupying compute units.
	if (bytes0 + bytes1 <= (1u << 20) && in_pinned_range(pinned_src0, bytes0) && in_pinned_range(pinned_src1, bytes1)) {
		const long words0 = (long) (bytes0 / 4), words1 = (long) (bytes1 / 4);
		const long vec0 = aligned16(dst0) && aligned16(pinned_src0) ? words0 / 4 : 0;
		const long threads = std::max(vec0 + (words0 - 4 * vec0), words1);
		const unsigned blocks = (unsigned) std::min<long>((threads + 255) / 256, 1024);
		hipLaunchKernelGGL(upload_pair_kernel, dim3(blocks), dim3(256), 0, r.upload_stream, (uint32_t *) dst0, (const uint32_t *) pinned_src0,
				words0, vec0, (uint32_t *) dst1, (const uint32_t *) pinned_src1, words1);
		CNET_LAUNCH_CHECK();
		return CNET_OK;
	}
	if (bytes0) CNET_HIP(hipMemcpyAsync(dst0, pinned_src0, bytes0, hipMemcpyHostToDevice, r.upload_stream));
	if (bytes1) CNET_HIP(hipMemcpyAsync(dst1, pinned_src1, bytes1, hipMemcpyHostToDevice, r.upload_stream));
	return CNET_OK;
}

// rows of a table on the device into a batch buffer, with their labels: each wavefront of workgroup (x, p) copies one row,
// idx[4 x + wavefront], of plane p (its lanes read the index over the link in one request)
__global__ __launch_bounds__(256) void gather_rows_kernel(float *__restrict__ dst, long ldd, long dst_plane, const float *__restrict__ src,
		long lds, long src_plane, int src_rows, const int32_t *__restrict__ idx, int32_t *__restrict__ dst_labels,
		const int32_t *__restrict__ src_labels, int rows, int cols, int vec) {
	const int r = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
	if (r >= rows) return;
	const int i = min(max(idx[r], 0), src_rows - 1);
	const float *s = src + (long) blockIdx.y * src_plane + (long) i * lds;
	float *d = dst + (long) blockIdx.y * dst_plane + (long) r * ldd;
	if (vec) {
		for (int c = lane * 4; c < cols; c += 256) *reinterpret_cast<float4 *>(d + c) = *reinterpret_cast<const float4 *>(s + c);
	} else {
		for (int c = lane; c < cols; c += 64) d[c] = s[c];
	}
	if (blockIdx.y == 0 && lane == 0 && dst_labels) dst_labels[r] = src_labels[i];
}

static int gather_rows_on(hipStream_t stream, const char *who, float *dst, int64_t ldd, int64_t dst_plane_stride, const float *src, int64_t lds,
		int64_t src_plane_stride, int planes, int src_rows, const int32_t *pinned_idx, int32_t *dst_labels, const int32_t *src_labels, int rows,
		int cols);

int cnet_upload_gather_rows(float *dst, int64_t ldd, int64_t dst_plane_stride, const float *src, int64_t lds, int64_t src_plane_stride,
		int planes, int src_rows, const int32_t *pinned_idx, int32_t *dst_labels, const int32_t *src_labels, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // work on the upload stream: never part of a recording
	return gather_rows_on(rt().upload_stream, "cnet_upload_gather_rows", dst, ldd, dst_plane_stride, src, lds, src_plane_stride, planes, src_rows,
			pinned_idx, dst_labels, src_labels, rows, cols);
}

int cnet_gather_rows(float *dst, int64_t ldd, int64_t dst_plane_stride, const float *src, int64_t lds, int64_t src_plane_stride, int planes,
		int src_rows, const int32_t *pinned_idx, int32_t *dst_labels, const int32_t *src_labels, int rows, int cols) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // the indices are read when the kernel runs: a replay would read whatever the buffer holds then
	return gather_rows_on(rt().stream, "cnet_gather_rows", dst, ldd, dst_plane_stride, src, lds, src_plane_stride, planes, src_rows, pinned_idx,
			dst_labels, src_labels, rows, cols);
}

static int gather_rows_on(hipStream_t stream, const char *who, float *dst, int64_t ldd, int64_t dst_plane_stride, const float *src, int64_t lds,
		int64_t src_plane_stride, int planes, int src_rows, const int32_t *pinned_idx, int32_t *dst_labels, const int32_t *src_labels, int rows,
		int cols) {
	const bool shape_ok = rows >= 0 && rows <= 65535 * 32 && cols > 0 && src_rows > 0 && (planes == 1 || planes == 2);
	if (shape_ok && !rows) return CNET_OK;
	const bool args_ok = shape_ok && dst && src && pinned_idx && ldd >= cols && lds >= cols && (dst_labels == nullptr) == (src_labels == nullptr) &&
			(planes == 1 || (dst_plane_stride >= (int64_t) (rows - 1) * ldd + cols && src_plane_stride >= (int64_t) (src_rows - 1) * lds + cols));
	if (!args_ok)
		return fail(CNET_ERR_INVALID_ARGUMENT, "%s: rows, cols, table rows > 0, 1 or 2 planes, pointers given, leading dimensions >= cols, planes that "
				"do not overlap, and both label arrays or neither", who);
	// the kernel reads the indices where they are: anything but memory from cnet_host_alloc would be a fault on the device
	if (!in_pinned_range(pinned_idx, (size_t) rows * sizeof(int32_t)))
		return fail(CNET_ERR_INVALID_ARGUMENT, "%s: the indices do not lie in memory from cnet_host_alloc", who);
	for (int r = 0; r < rows; ++r)
		if (pinned_idx[r] < 0 || pinned_idx[r] >= src_rows)
			return fail(CNET_ERR_INVALID_ARGUMENT, "%s: index %d of row %d outside the table of %d rows", who, pinned_idx[r], r, src_rows);
	const bool vec = cols % 4 == 0 && ldd % 4 == 0 && lds % 4 == 0 && dst_plane_stride % 4 == 0 && src_plane_stride % 4 == 0 && aligned16(dst) &&
			aligned16(src);
	dim3 grid((unsigned) ((rows + 3) / 4), (unsigned) planes);
	hipLaunchKernelGGL(gather_rows_kernel, grid, dim3(256), 0, stream, dst, (long) ldd, (long) dst_plane_stride, src, (long) lds,
			(long) src_plane_stride, src_rows, pinned_idx, dst_labels, src_labels, rows, cols, vec ? 1 : 0);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

int cnet_upload_zero(void *dst, size_t bytes) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // a fill on the upload stream: never part of a recording
	if (!bytes) return CNET_OK;
	CNET_CHECK_ARG(dst != nullptr);
	CNET_HIP(hipMemsetAsync(dst, 0, bytes, rt().upload_stream));
	return CNET_OK;
}

int cnet_upload_wait_compute(void) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // would pull the upload stream into the recording
	CNET_HIP(hipEventRecord(rt().compute_done, rt().stream));
	CNET_HIP(hipStreamWaitEvent(rt().upload_stream, rt().compute_done, 0));
	return CNET_OK;
}

int cnet_mark_compute(int marker) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_CHECK_ARG(marker >= 0 && marker < Runtime::kMarkers);
	CNET_HIP(hipEventRecord(rt().marker[marker], rt().stream));
	return CNET_OK;
}

// `stream` waits for the point that `ev` stands for.  A point that has been reached already needs no wait, and asking
// costs the host a tenth of what queueing a wait across streams does (0.5 against 5-8 us); in a training loop that is
// the usual case for both directions (the buffer about to be refilled was retired two steps ago, the batch about to be
// used landed a step ago).
static int wait_unless_reached(hipStream_t stream, hipEvent_t ev) {
	const hipError_t q = hipEventQuery(ev);
	if (q == hipSuccess) return CNET_OK;
	(void) hipGetLastError();  // "not ready" is an answer, not a failure to carry into the next call
	CNET_HIP(hipStreamWaitEvent(stream, ev, 0));
	return CNET_OK;
}

int cnet_upload_wait_marker(int marker) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_CHECK_ARG(marker >= 0 && marker < Runtime::kMarkers);
	// a marker that was never set does not hold anything back
	return wait_unless_reached(rt().upload_stream, rt().marker[marker]);
}

int cnet_mark_upload(int marker) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_CHECK_ARG(marker >= 0 && marker < Runtime::kMarkers);
	CNET_HIP(hipEventRecord(rt().upload_marker[marker], rt().upload_stream));
	return CNET_OK;
}

int cnet_compute_wait_upload_marker(int marker) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // would pull the upload stream into the recording
	CNET_CHECK_ARG(marker >= 0 && marker < Runtime::kMarkers);
	// a marker that was never set does not hold anything back
	return wait_unless_reached(rt().stream, rt().upload_marker[marker]);
}

int cnet_compute_wait_upload(void) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // would pull the upload stream into the recording
	CNET_HIP(hipEventRecord(rt().upload_done, rt().upload_stream));
	CNET_HIP(hipStreamWaitEvent(rt().stream, rt().upload_done, 0));
	return CNET_OK;
}

int cnet_copy_ticket(int upload_stream, int64_t *ticket) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_CHECK_ARG(ticket != nullptr);
	Runtime &r = rt();
	const int which = upload_stream ? 1 : 0;
	const int64_t n = r.tickets_issued[which];
	CNET_HIP(hipEventRecord(r.ticket_event[which][n % Runtime::kTickets], which ? r.upload_stream : r.stream));
	r.tickets_issued[which] = n + 1;
	*ticket = 2 * n + which;
	return CNET_OK;
}

int cnet_copy_wait(int64_t ticket) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	Runtime &r = rt();
	const int which = (int) (ticket & 1);
	const int64_t n = ticket >> 1;
	CNET_CHECK_ARG(ticket >= 0 && n < r.tickets_issued[which]);
	CNET_HIP(hipEventSynchronize(r.ticket_event[which][n % Runtime::kTickets]));
	return CNET_OK;
}

int cnet_compute_wait_ticket(int64_t ticket) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // would pull the upload stream into the recording
	Runtime &r = rt();
	const int which = (int) (ticket & 1);
	const int64_t n = ticket >> 1;
	CNET_CHECK_ARG(ticket >= 0 && which == 1 && n < r.tickets_issued[which]);
	// a ticket whose event has been handed out again since stands for a later point of the same stream: the wait still covers it
	return wait_unless_reached(r.stream, r.ticket_event[which][n % Runtime::kTickets]);
}

int cnet_upload_sync(void) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_HIP(hipStreamSynchronize(rt().upload_stream));
	return CNET_OK;
}

int cnet_memcpy_d2h(void *host_dst, const void *src, size_t bytes) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	if (!bytes) return CNET_OK;
	CNET_CHECK_ARG(host_dst && src);
	CNET_HIP(hipMemcpyAsync(host_dst, src, bytes, hipMemcpyDeviceToHost, rt().stream));
	CNET_HIP(hipStreamSynchronize(rt().stream));
	return CNET_OK;
}

// ---- graphs: record the launches of a repeated sequence once, replay them with one call
int cnet_graph_begin(void) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	// no first-use set-up call of a kernel may fall inside the recording
	const int primed = cgemm_prime_attributes();
	if (primed != CNET_OK) return primed;
	CNET_HIP(hipStreamBeginCapture(rt().stream, hipStreamCaptureModeThreadLocal));
	rt().capturing = true;
	return CNET_OK;
}

int cnet_graph_end(void **graph_exec) {
	CNET_REQUIRE_INIT();
	Runtime &r = rt();
	if (!r.capturing) return fail(CNET_ERR_INVALID_ARGUMENT, "cnet_graph_end without cnet_graph_begin");
	r.capturing = false;
	hipGraph_t graph = nullptr;
	hipError_t e = hipStreamEndCapture(r.stream, &graph);
	if (e != hipSuccess || !graph) {
		(void) hipGetLastError();
		if (graph_exec) *graph_exec = nullptr;
		return hip_fail(e != hipSuccess ? e : hipErrorUnknown, "hipStreamEndCapture (a call inside the recording failed)");
	}
	if (!graph_exec) {  // the caller abandons the recording
		(void) hipGraphDestroy(graph);
		return CNET_OK;
	}
	*graph_exec = nullptr;
	int slot = 0;
	while (slot < Runtime::kGraphs && r.graph_exec[slot]) ++slot;
	if (slot == Runtime::kGraphs) {
		(void) hipGraphDestroy(graph);
		return fail(CNET_ERR_UNSUPPORTED, "cnet_graph_end: %d recordings exist already: destroy some first", Runtime::kGraphs);
	}
	hipGraphExec_t exec = nullptr;
	e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
	if (e != hipSuccess) {
		(void) hipGraphDestroy(graph);
		return hip_fail(e, "hipGraphInstantiate");
	}
	// the graph the executable was made from is kept until cnet_graph_destroy
	r.graph_exec[slot] = exec;
	r.graph_template[slot] = graph;
	*graph_exec = exec;
	r.graphs_alive++;
	return CNET_OK;
}

// slot of a live recording, -1 for a handle this library did not hand out (or has destroyed already)
static int graph_slot(void *graph_exec) {
	Runtime &r = rt();
	for (int k = 0; k < Runtime::kGraphs; ++k)
		if (r.graph_exec[k] && (void *) r.graph_exec[k] == graph_exec) return k;
	return -1;
}

int cnet_graph_launch(void *graph_exec) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();
	CNET_CHECK_ARG(graph_exec != nullptr);
	if (graph_slot(graph_exec) < 0) return fail(CNET_ERR_INVALID_ARGUMENT, "cnet_graph_launch: not a live recording of this library");
	CNET_HIP(hipGraphLaunch((hipGraphExec_t) graph_exec, rt().stream));
	return CNET_OK;
}

int cnet_graph_destroy(void *graph_exec) {
	CNET_REQUIRE_INIT();
	CNET_NOT_IN_CAPTURE();  // waits for the stream, which would break the recording
	if (!graph_exec) return CNET_OK;
	Runtime &r = rt();
	const int slot = graph_slot(graph_exec);
	if (slot < 0) return fail(CNET_ERR_INVALID_ARGUMENT, "cnet_graph_destroy: not a live recording of this library");
	CNET_HIP(hipStreamSynchronize(r.stream));
	const hipError_t e1 = hipGraphExecDestroy(r.graph_exec[slot]);
	const hipError_t e2 = hipGraphDestroy(r.graph_template[slot]);
	r.graph_exec[slot] = nullptr;
	r.graph_template[slot] = nullptr;
	if (r.graphs_alive > 0) r.graphs_alive--;
	if (e1 != hipSuccess) return hip_fail(e1, "hipGraphExecDestroy");
	if (e2 != hipSuccess) return hip_fail(e2, "hipGraphDestroy");
	return CNET_OK;
}

int cnet_memcpy_d2d(void *dst, const void *src, size_t bytes) {
	CNET_REQUIRE_INIT();
	if (!bytes) return CNET_OK;
	CNET_CHECK_ARG(dst && src);
	CNET_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, rt().stream));
	return CNET_OK;
}

}  // extern "C"
