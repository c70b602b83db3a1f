// Split-plane complex GEMM on gfx950 fp32 MFMA, and the Linear entry points built on it.
//
//   C[M x N] (+)= A[M x K] * B[K x N]      (complex; optionally conj(B))
//   Cr += Ar*Br - Ai*Bi ,  Ci += Ar*Bi + Ai*Br      -> four v_mfma_f32_32x32x2_f32 per (A tile, B tile, k pair)
//
// Work decomposition
//   workgroup = 256 threads = 4 wavefronts (one per SIMD) computing a BM x BN block of C;
//   wavefront = WM x WN sub-block = (WM/32) x (WN/32) MFMA tiles, with a real and an imaginary accumulator
//   (16 VGPR each) per tile kept in registers for the whole K loop.
// Data movement (cgemm_kernel, any shape; the fast path further down moves tiles from global memory straight into LDS)
//   K is walked in chunks of KC = 16.  Each chunk of the four operand planes is fetched from global memory into
//   registers (float4, coalesced along the contiguous dimension of the source), then written to LDS in
//   [k][row] order, whatever the source layout: an MFMA operand fragment (lane l -> row l%32, k = l/32) is
//   then 32 consecutive floats per half-wave, free of bank conflicts.  Sources that are contiguous along k are
//   transposed by the LDS write; the row pitch (rows + 4) spreads those writes over all banks.
//   LDS is double buffered: the global loads of chunk c+1 are issued before the MFMAs of chunk c and are written
//   to the other buffer late in that chunk, so there is one barrier per chunk and it is covered by MFMA work.
//   conj(B) costs nothing: the sign goes onto B's imaginary plane on its way into LDS.  The minus sign of
//   Ai*Bi is one v_xor on the Ai fragment per k pair.
// Launch
//   one workgroup per C block and per problem (blockIdx.y: the dz and the dzs product of a backward pass are
//   one launch).  Workgroup ids are dealt round-robin to the 8 XCDs by the hardware; the id is remapped so that
//   each XCD works on a contiguous strip of C blocks and re-uses operand tiles through its own L2.
// Three kernels share this file: cgemm_kernel (above; any shape and alignment), cgemm_fast_kernel (16-byte aligned
// operands and K a multiple of 16: tiles go from global memory straight into LDS; the one the large products run on),
// and cgemm_skinny_kernel (a C of few 16 x 16 tiles: one tile per workgroup, K shared among its wavefronts).
// cgemm_dispatch picks among them and pick_tile picks the block shape.
#include "common.hpp"
#include "gate.hpp"
#include "rows.hpp"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int KC = 16;         // k extent of one LDS stage
constexpr int NTHREADS = 256;  // 4 wavefronts
constexpr int NUM_XCD = 8;

struct CgemmProblem {
	const float *a_re, *a_im, *b_re, *b_im;
	float *c_re, *c_im;
	float a_im_sign;  // -1: multiply by conj(A)
	float b_im_sign;  // -1: multiply by conj(B)
};

struct CgemmArgs {
	CgemmProblem p[2];
	int M, N, K;
	long lda, ldb, ldc;
	int accumulate;
	int tiles_m, tiles_n;
	long stride_a, stride_b, stride_c;  // element strides between the matrices of a strided batch (blockIdx.z)
	// Triangular B (square, zeros stored outside the triangle): 1 = B[k][n] is zero for k > n, 2 = zero for k < n.
	// A block of columns [n0, n0 + BN) then only walks the K chunks that can hold non-zeros.
	int tri;
	// Split K: short grids (a small batch against a long reduction) run `splits` workgroups per block of C, each over
	// `chunks_per_split` chunks of K, writing partial blocks to `partial`; splitk_reduce_kernel adds them in split order.
	// blockIdx.z = batch index * splits + split.
	int splits, chunks_per_split;
	float *partial;  // [split][problem][batch][re, im][M][N]
	// Tail: when the blocks of C do not fill a whole number of rounds over the compute units, the blocks of the last,
	// partly filled round ("tail blocks": the last tail_tiles of the nprob x tiles_m x tiles_n blocks) are cut into
	// tail_splits pieces along K, tail_chunks chunks each.  The launch has one workgroup per block of the full rounds
	// (problems share blockIdx.x); workgroup i < tail_tiles x tail_splits computes piece i as well, after its block, so
	// every compute unit gets the same share of the tail wherever the hardware places the workgroups.  A piece writes its
	// whole block to partial[tail block][piece][re, im][BM][BN]; tail_reduce_kernel adds the pieces in order.
	int tail_tiles, tail_splits, tail_chunks, nprob;
	// Mirror: one problem is computed and its result also written, conjugated, to the C planes of p[1] (honouring
	// `accumulate` there as well).  The backward passes use it when the incoming dz* gradient is the conjugate of the dz
	// gradient, as it is under every real-valued loss: the dz* product is then the conjugate of the dz product (the same
	// sums with signs applied exactly) and need not be computed.  Not combined with a strided batch.
	// mirror == 2 (MIRROR_GELU): the C planes of p[1] receive the CGelu of the final value of C instead (a Linear followed by
	// a CGelu in one launch: the pre-activation and the activation are both written, neither is read back); always assigned.
	int mirror;
	// The imaginary plane of A holds nothing but +0 (the caller vouches: real samples in front of a transform) and is not read:
	// two real products per complex one, re = Ar Br, im = +-Ar Bi, the bits of the four products on such an A.  Honoured by the
	// block kernels for a row-major A against a k-major B (the layout of the transform); ignored elsewhere.
	// a_real == 2: the two planes of A are two real operands of their own and C = (Ar Br) + i (Ai Bi): the transform of
	// real samples folded about n/2 (cos is even and sin odd under k -> n - k: Ar holds x[k] + x[n - k], Ai holds
	// x[k] - x[n - k], and K is half as long).  Block kernels of that layout only; the caller sees to it that they take it.
	int a_real = 0;
	// mirror == 3 (MIRROR_HERM): element (row, col) with herm_lo <= col <= herm_hi also goes, conjugated, to column herm_n - col
	// of the same row of C (honouring `accumulate`): the transform of real samples computes columns 0 .. n/2 and fills the others
	// as it stores those.  One problem; the columns written this way must lie outside the product's own.
	int herm_n = 0, herm_lo = 1, herm_hi = 0;
	// mirror == 4 (MIRROR_HGELU): the value y of C at (row, col) is multiplied by the shared row hv[col], h = y hv goes to the C
	// planes of p[1] and its CGelu to (g_re, g_im), all with leading dimension ldc: a transform followed by a Hadamard gate with
	// shared weights and a CGelu in one launch, with the arithmetic of hadamard_gelu_fwd_kernel on the stored y.  Honoured by the
	// small-C kernel without slices of K only (the caller checks); always assigned.
	const float *hv_re = nullptr, *hv_im = nullptr;
	float *g_re = nullptr, *g_im = nullptr;
	// mirror == 5 (MIRROR_CE): C is a block of logits whose columns all lie in one tile (N <= 16).  The workgroup that has formed
	// 16 rows of it also runs the forward pass of CrossEntropy and the gradient of the loss over them (crossent_fwd_row_at on the
	// tile in LDS, the routine and the instantiation the separate launch would run: the same bits): a narrow Linear head and its
	// loss in one launch.  Small-C kernel without slices of K (the caller checks); C is assigned.
	const int *ce_labels = nullptr;
	float *ce_out_re = nullptr, *ce_out_im = nullptr, *ce_s = nullptr, *ce_loss = nullptr;
	int *ce_argmax = nullptr;
	float *ce_dz_re = nullptr, *ce_dz_im = nullptr, *ce_dzs_re = nullptr, *ce_dzs_im = nullptr;
	long ce_ldo = 0, ce_lddz = 0;
	int ce_vec = 0;  // the 128-bit instantiation of the row routine (what the separate launch would pick for these operands)
};
constexpr int MIRROR_CONJ = 1, MIRROR_GELU = 2, MIRROR_HERM = 3, MIRROR_HGELU = 4, MIRROR_CE = 5;

// the conjugate of (vr, vi) into element `off` of the mirror planes
__device__ __forceinline__ void mirror_store(const CgemmArgs &args, long off, float vr, float vi) {
	if (args.mirror != MIRROR_CONJ) return;
	float mr = vr, mi = -vi;
	if (args.accumulate) {
		mr += args.p[1].c_re[off];
		mi += args.p[1].c_im[off];
	}
	args.p[1].c_re[off] = mr;
	args.p[1].c_im[off] = mi;
}

// one plane (part 0: real, 1: imaginary) of the product's value at (row, col) to the Hermitian partner of that element
__device__ __forceinline__ void herm_store_part(const CgemmArgs &args, int part, int row, int col, float v) {
	if (args.mirror != MIRROR_HERM || col < args.herm_lo || col > args.herm_hi) return;
	float *m = (part ? args.p[0].c_im : args.p[0].c_re) + (long) row * args.ldc + (args.herm_n - col);
	const float mv = part ? -v : v;
	*m = args.accumulate ? *m + mv : mv;
}
__device__ __forceinline__ void herm_store(const CgemmArgs &args, int row, int col, float vr, float vi) {
	herm_store_part(args, 0, row, col, vr);
	herm_store_part(args, 1, row, col, vi);
}

// the CGelu of the final value (vr, vi) of element `off` into the planes of p[1]
__device__ __forceinline__ void gelu_store(const CgemmArgs &args, long off, float vr, float vi) {
	if (args.mirror != MIRROR_GELU) return;
	args.p[1].c_re[off] = cnet::gelu_value(vr);
	args.p[1].c_im[off] = cnet::gelu_value(vi);
}

// Which block of C (per problem) a linear block number stands for: walks groups of 8 block rows column by column, after
// spreading consecutive workgroup numbers (which the hardware deals round-robin to the XCDs) over contiguous strips.
__device__ __forceinline__ void map_block(const CgemmArgs &args, int pid, int grid_n, int &tile_m, int &tile_n) {
	const int total = args.tiles_m * grid_n;
	if (total % NUM_XCD == 0) pid = (pid % NUM_XCD) * (total / NUM_XCD) + pid / NUM_XCD;
	constexpr int GROUP = 8;
	const int width = GROUP * grid_n;
	const int first_m = (pid / width) * GROUP;
	const int gsize = min(args.tiles_m - first_m, GROUP);
	tile_m = first_m + (pid % width) % gsize;
	tile_n = (pid % width) / gsize;
}

// column blocks per grid row: with a triangular operand each workgroup handles a block and its mirror image
__device__ __host__ __forceinline__ int grid_tiles_n(const CgemmArgs &args) { return args.tri ? (args.tiles_n + 1) / 2 : args.tiles_n; }

// first chunk and one-past-last chunk of K for the block of columns starting at n0
template <int BN>
__device__ __forceinline__ void chunk_range(const CgemmArgs &args, int n0, int &c_lo, int &c_hi) {
	c_lo = 0;
	c_hi = (args.K + KC - 1) / KC;
	if (args.tri == 1) c_hi = min(c_hi, (n0 + BN + KC - 1) / KC);
	if (args.tri == 2) c_lo = n0 / KC;
	if (args.splits > 1) {
		c_lo = (blockIdx.z % args.splits) * args.chunks_per_split;
		c_hi = min(c_hi, c_lo + args.chunks_per_split);
	}
}

// where this workgroup writes its block: C itself, or its slice of the partial planes when K is split
__device__ __forceinline__ void output_planes(const CgemmArgs &args, CgemmProblem &pb, long &ldc, int &accumulate) {
	ldc = args.ldc;
	accumulate = args.accumulate;
	if (args.splits > 1) {
		const long plane = (long) args.M * args.N;
		const long nbatch = gridDim.z / args.splits, split = blockIdx.z % args.splits, b = blockIdx.z / args.splits;
		pb.c_re = args.partial + (((split * gridDim.y + blockIdx.y) * nbatch + b) * 2) * plane;
		pb.c_im = pb.c_re + plane;
		ldc = args.N;
		accumulate = 0;
	}
}

__device__ __forceinline__ void batch_offset(CgemmProblem &pb, const CgemmArgs &args) {
	const long z = blockIdx.z / args.splits;
	pb.a_re += z * args.stride_a;
	pb.a_im += z * args.stride_a;
	pb.b_re += z * args.stride_b;
	pb.b_im += z * args.stride_b;
	pb.c_re += z * args.stride_c;
	pb.c_im += z * args.stride_c;
}

__device__ __forceinline__ float keep(float v, unsigned mask) { return __uint_as_float(__float_as_uint(v) & mask); }

// One operand (both planes) of one K chunk: ROWS rows of the block by KC values of k.
// MCONTIG: the source is stored [k][row] (row contiguous); otherwise [row][k] (k contiguous).
template <int ROWS, bool MCONTIG, int VEC>
struct Stage;

template <int ROWS, bool MCONTIG>
struct Stage<ROWS, MCONTIG, 4> {
	static constexpr int UNITS = ROWS * KC / 4 / NTHREADS;  // float4 per thread and plane
	float4 re[UNITS], im[UNITS];
	bool ok[UNITS];

	__device__ __forceinline__ void load(const float *__restrict__ pre, const float *__restrict__ pim, int row0, int k0,
			int rows_total, int K, long ld) {
#pragma unroll
		for (int u = 0; u < UNITS; ++u) {
			int unit = threadIdx.x + u * NTHREADS;
			int row, k;
			if (MCONTIG) {
				k = unit / (ROWS / 4);
				row = (unit % (ROWS / 4)) * 4;
			} else {
				row = unit / (KC / 4);
				k = (unit % (KC / 4)) * 4;
			}
			// branch-free edge handling: an out-of-range unit reads element 0 and is replaced by zeros when it is
			// written to LDS, so nothing consumes the loaded registers before the MFMAs of the current chunk
			ok[u] = (row0 + row < rows_total) && (k0 + k < K);
			long off = MCONTIG ? (long) (k0 + k) * ld + row0 + row : (long) (row0 + row) * ld + k0 + k;
			off = ok[u] ? off : 0;
			re[u] = *reinterpret_cast<const float4 *>(pre + off);
			im[u] = *reinterpret_cast<const float4 *>(pim + off);
		}
	}

	template <int LDS_PITCH>
	__device__ __forceinline__ void store(float *sre, float *sim, float im_sign) const {
#pragma unroll
		for (int u = 0; u < UNITS; ++u) {
			int unit = threadIdx.x + u * NTHREADS;
			const unsigned m = ok[u] ? 0xffffffffu : 0u;  // bitwise zeroing: no branch, no NaN * 0
			float4 a = make_float4(keep(re[u].x, m), keep(re[u].y, m), keep(re[u].z, m), keep(re[u].w, m));
			float4 b = make_float4(keep(im[u].x * im_sign, m), keep(im[u].y * im_sign, m), keep(im[u].z * im_sign, m),
					keep(im[u].w * im_sign, m));
			if (MCONTIG) {
				int k = unit / (ROWS / 4);
				int row = (unit % (ROWS / 4)) * 4;
				*reinterpret_cast<float4 *>(sre + k * LDS_PITCH + row) = a;
				*reinterpret_cast<float4 *>(sim + k * LDS_PITCH + row) = b;
			} else {
				int row = unit / (KC / 4);
				int k = (unit % (KC / 4)) * 4;
				sre[(k + 0) * LDS_PITCH + row] = a.x;
				sre[(k + 1) * LDS_PITCH + row] = a.y;
				sre[(k + 2) * LDS_PITCH + row] = a.z;
				sre[(k + 3) * LDS_PITCH + row] = a.w;
				sim[(k + 0) * LDS_PITCH + row] = b.x;
				sim[(k + 1) * LDS_PITCH + row] = b.y;
				sim[(k + 2) * LDS_PITCH + row] = b.z;
				sim[(k + 3) * LDS_PITCH + row] = b.w;
			}
		}
	}
};

// Scalar variant for shapes whose contiguous extent or leading dimension is not a multiple of 4.
template <int ROWS, bool MCONTIG>
struct Stage<ROWS, MCONTIG, 1> {
	static constexpr int UNITS = ROWS * KC / NTHREADS;
	float re[UNITS], im[UNITS];
	bool ok[UNITS];

	__device__ __forceinline__ void load(const float *__restrict__ pre, const float *__restrict__ pim, int row0, int k0,
			int rows_total, int K, long ld) {
#pragma unroll
		for (int u = 0; u < UNITS; ++u) {
			int unit = threadIdx.x + u * NTHREADS;
			int row = MCONTIG ? unit % ROWS : unit / KC;
			int k = MCONTIG ? unit / ROWS : unit % KC;
			ok[u] = (row0 + row < rows_total) && (k0 + k < K);
			long off = MCONTIG ? (long) (k0 + k) * ld + row0 + row : (long) (row0 + row) * ld + k0 + k;
			off = ok[u] ? off : 0;
			re[u] = pre[off];
			im[u] = pim[off];
		}
	}

	template <int LDS_PITCH>
	__device__ __forceinline__ void store(float *sre, float *sim, float im_sign) const {
#pragma unroll
		for (int u = 0; u < UNITS; ++u) {
			int unit = threadIdx.x + u * NTHREADS;
			int row = MCONTIG ? unit % ROWS : unit / KC;
			int k = MCONTIG ? unit / ROWS : unit % KC;
			const unsigned m = ok[u] ? 0xffffffffu : 0u;
			sre[k * LDS_PITCH + row] = keep(re[u], m);
			sim[k * LDS_PITCH + row] = keep(im[u] * im_sign, m);
		}
	}
};

template <int BM, int BN, int WM, int WN, bool A_MCONTIG, bool B_NCONTIG, int VEC>
__global__ __launch_bounds__(NTHREADS, 2) void cgemm_kernel(const CgemmArgs args) {
	static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per workgroup");
	constexpr int TM = WM / 32, TN = WN / 32;
	constexpr int PA = BM + 4, PB = BN + 4;  // LDS row pitch in floats
	constexpr int A_PLANE = KC * PA, B_PLANE = KC * PB;
	constexpr int STAGE_FLOATS = 2 * A_PLANE + 2 * B_PLANE;
	extern __shared__ float smem[];

	CgemmProblem pb = args.p[blockIdx.y];
	batch_offset(pb, args);
	long ldc;
	int accumulate;
	output_planes(args, pb, ldc, accumulate);
	const int M = args.M, N = args.N, K = args.K;

	// ---- which block of C
	const int grid_n = grid_tiles_n(args);
	int tile_m, tile_n_first;
	map_block(args, blockIdx.x, grid_n, tile_m, tile_n_first);
	const int m0 = tile_m * BM;
	// a triangular operand: this workgroup takes column block j and then its mirror tiles_n - 1 - j, so that every
	// workgroup walks the same number of K chunks in total
	const int npass = (args.tri && tile_n_first != args.tiles_n - 1 - tile_n_first) ? 2 : 1;

	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int wm0 = (wave / (BN / WN)) * WM;
	const int wn0 = (wave % (BN / WN)) * WN;
	const int r = lane & 31, h = lane >> 5;

	floatx16 acc_re[TM][TN], acc_im[TM][TN];
	for (int pass = 0; pass < npass; ++pass) {
	const int tile_n = pass ? args.tiles_n - 1 - tile_n_first : tile_n_first;
	const int n0 = tile_n * BN;
	if (pass) __syncthreads();  // every wave has finished reading the last stage of the previous block
#pragma unroll
	for (int i = 0; i < TM; ++i)
#pragma unroll
		for (int j = 0; j < TN; ++j)
#pragma unroll
			for (int e = 0; e < 16; ++e) {
				acc_re[i][j][e] = 0.f;
				acc_im[i][j][e] = 0.f;
			}

	Stage<BM, A_MCONTIG, VEC> sa;
	Stage<BN, B_NCONTIG, VEC> sb;

	int c_lo, c_hi;
	chunk_range<BN>(args, n0, c_lo, c_hi);
	sa.load(pb.a_re, pb.a_im, m0, c_lo * KC, M, K, args.lda);
	sb.load(pb.b_re, pb.b_im, n0, c_lo * KC, N, K, args.ldb);
	sa.template store<PA>(smem, smem + A_PLANE, pb.a_im_sign);
	sb.template store<PB>(smem + 2 * A_PLANE, smem + 2 * A_PLANE + B_PLANE, pb.b_im_sign);
	__syncthreads();

	// Operand fragments are double buffered in registers: those of k pair ks+1 are read from LDS while the MFMAs
	// of k pair ks run.  Per chunk there is ONE barrier, placed two k pairs before the end: by then every wave has
	// issued its last read of the current stage and has written the next stage, so the 32 MFMAs that follow cover
	// the barrier skew and the LDS latency of the first fragment of the next chunk.
	float are[2][TM], aim[2][TM], anim[2][TM], bre[2][TN], bim[2][TN];
	auto fetch = [&](const float *stage, int ks, int slot) {
		const int k = ks * 2 + h;
		const float *s_are = stage + wm0 + r, *s_aim = stage + A_PLANE + wm0 + r;
		const float *s_bre = stage + 2 * A_PLANE + wn0 + r, *s_bim = stage + 2 * A_PLANE + B_PLANE + wn0 + r;
#pragma unroll
		for (int i = 0; i < TM; ++i) {
			are[slot][i] = s_are[k * PA + i * 32];
			aim[slot][i] = s_aim[k * PA + i * 32];
		}
#pragma unroll
		for (int j = 0; j < TN; ++j) {
			bre[slot][j] = s_bre[k * PB + j * 32];
			bim[slot][j] = s_bim[k * PB + j * 32];
		}
	};
	fetch(smem, 0, 0);

	for (int c = c_lo; c < c_hi; ++c) {
		const float *cur = smem + ((c - c_lo) & 1) * STAGE_FLOATS;
		float *nxt = smem + ((c - c_lo + 1) & 1) * STAGE_FLOATS;
		const bool more = (c + 1 < c_hi);
		if (more) {
			sa.load(pb.a_re, pb.a_im, m0, (c + 1) * KC, M, K, args.lda);
			sb.load(pb.b_re, pb.b_im, n0, (c + 1) * KC, N, K, args.ldb);
		}
#pragma unroll
		for (int ks = 0; ks < KC / 2; ++ks) {
			const int cs = ks & 1;
			if (ks + 1 < KC / 2) fetch(cur, ks + 1, cs ^ 1);
			if (ks == KC / 2 - 2) {
				if (more) {
					sa.template store<PA>(nxt, nxt + A_PLANE, pb.a_im_sign);
					sb.template store<PB>(nxt + 2 * A_PLANE, nxt + 2 * A_PLANE + B_PLANE, pb.b_im_sign);
				}
				__syncthreads();
			}
			if (ks == KC / 2 - 1 && more) fetch(nxt, 0, cs ^ 1);
#pragma unroll
			for (int i = 0; i < TM; ++i) anim[cs][i] = -aim[cs][i];
			__builtin_amdgcn_sched_barrier(0);
#pragma unroll
			for (int i = 0; i < TM; ++i)
#pragma unroll
				for (int j = 0; j < TN; ++j) {
					acc_re[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[cs][i], bre[cs][j], acc_re[i][j], 0, 0, 0);
					acc_im[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[cs][i], bim[cs][j], acc_im[i][j], 0, 0, 0);
				}
#pragma unroll
			for (int i = 0; i < TM; ++i)
#pragma unroll
				for (int j = 0; j < TN; ++j) {
					acc_re[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(anim[cs][i], bim[cs][j], acc_re[i][j], 0, 0, 0);
					acc_im[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(aim[cs][i], bre[cs][j], acc_im[i][j], 0, 0, 0);
				}
			__builtin_amdgcn_sched_barrier(0);
		}
	}

	// ---- epilogue: accumulator element e of lane (r, h) is C[(e/4)*8 + h*4 + e%4][r] of its 32x32 tile.  The empty
	// asm keeps the address arithmetic below the loop (hoisted above it, it is spilled).
	int r_st = r, h_st = h;
	asm volatile("" : "+v"(r_st), "+v"(h_st));
#pragma unroll
	for (int i = 0; i < TM; ++i)
#pragma unroll
		for (int j = 0; j < TN; ++j) {
			const int col = n0 + wn0 + j * 32 + r_st;
			if (col >= N) continue;
#pragma unroll
			for (int e = 0; e < 16; ++e) {
				const int row = m0 + wm0 + i * 32 + (e >> 2) * 8 + h_st * 4 + (e & 3);
				if (row < M) {
					const long off = (long) row * ldc + col;
					float vr = acc_re[i][j][e], vi = acc_im[i][j][e];
					if (args.mirror && args.splits == 1) {
						mirror_store(args, (long) row * args.ldc + col, vr, vi);
						herm_store(args, row, col, vr, vi);
					}
					if (accumulate) {
						vr += pb.c_re[off];
						vi += pb.c_im[off];
					}
					pb.c_re[off] = vr;
					pb.c_im[off] = vi;
					if (args.mirror && args.splits == 1) gelu_store(args, (long) row * args.ldc + col, vr, vi);
				}
			}
		}
	}  // pass
}


// ---------------------------------------------------------------------------------------------------------------
// Fast path: K % KC == 0, 128-bit aligned operands whose contiguous extents and leading dimensions are multiples of 4 (any
// M and N).  Same decomposition as cgemm_kernel,
// with the per-chunk overhead taken out of the vector ALU, the registers and the LDS write port:
//   * operand tiles go from global memory straight into LDS (global_load_lds_dwordx4), 1 KiB per wave-wide
//     instruction, so a chunk needs no staging registers and no LDS write instructions; global addresses are
//     "uniform tile base (advanced with scalar adds) + per-lane 32-bit offset that never changes";
//   * LDS layouts follow from that (a transfer fills consecutive LDS bytes in lane order):
//       - a source contiguous along its rows lands as [k][row] (pitch = rows) and is read one float per k pair;
//       - a source contiguous along k lands as [row][16 k values]; the four 16-byte groups of a row are XOR-swizzled
//         with bits 2..3 of the row (applied to the global address each lane fetches), and the fragments come back with
//         128-bit reads: lane (row r, half h) takes k group h for k steps 0..3 and k group h + 2 for k steps 4..7;
//         16 consecutive rows cover all 64 banks.
//     The k order inside a chunk is therefore permuted: MFMA step s of half h multiplies k = 4h + s (s < 4) or
//     k = 8 + 4h + (s - 4); the [k][row] operands are addressed with the same map, so the products pair up correctly.
//   * LDS holds two (128 x 128) or three (smaller blocks) stages; the transfers of chunk c + stages - 1 are issued
//     before the MFMAs of chunk c, one vmcnt wait and one barrier per chunk publish the next stage;
//   * the scheduler is told to interleave (one MFMA, then a few DS / memory instructions) so everything else
//     issues in the shadow of the matrix pipe;
//   * the K loop holds (almost) no vector-ALU instruction, because each one costs the matrix pipe a few cycles (shared
//     issue port): signs are applied to the accumulators when they are stored (or compiled into the choice of the
//     negated operand, for the 128 x 128 block), and the chunk loop is unrolled over the LDS stages so that addresses
//     are "lane base + immediate".
// Operand fragments of one wavefront: T tiles of 32 rows, both planes.
//   MCONTIG ([k][row] in LDS): one float per tile, plane and k step, double buffered per step.
//   otherwise ([row][k] swizzled): one float4 per tile, plane and half chunk (set 0: steps 0..3, set 1: steps 4..7).
template <int T, bool MCONTIG, int PITCH, int PLANE, bool REAL = false>
struct Frag {
	float s_re[2][T], s_im[2][T];
	float4 q_re[2][T], q_im[2][T];
	const float *base0, *base1;  // per-lane LDS addresses inside stage 0, plane re
	const float *row_base[T];    // [k][row] operands: base0 of each tile; everything else in an address is a multiple of 256 bytes

	// w0: first row of the wavefront's sub-block; r = lane % 32, h = lane / 32
	__device__ __forceinline__ void init(const float *plane_re, int w0, int r, int h) {
		if (MCONTIG) {
			base0 = plane_re + w0 + r + h * 4 * PITCH;
			base1 = base0;
#pragma unroll
			for (int i = 0; i < T; ++i) row_base[i] = base0 + i * 32;
		} else {
			const int row = w0 + r;
			const int sw = (row >> 2) & 3;
			base0 = plane_re + row * KC + ((h ^ sw) * 4);
			base1 = plane_re + row * KC + (((h + 2) ^ sw) * 4);
		}
	}
	// [k][row] operands: values of k step s into slot s & 1
	__device__ __forceinline__ void fetch_step(int stage_off, int s) {
		if (MCONTIG) {
			const int line = (s < 4 ? s : s + 4) * PITCH;
#pragma unroll
			for (int i = 0; i < T; ++i) {
				s_re[s & 1][i] = row_base[i][stage_off + line];
				if (!REAL) s_im[s & 1][i] = row_base[i][stage_off + PLANE + line];
			}
		}
	}
	// [row][k] operands: the four k values of half chunk `set`
	__device__ __forceinline__ void fetch_set(int stage_off, int set) {
		if (!MCONTIG) {
			const float *b = (set ? base1 : base0) + stage_off;
#pragma unroll
			for (int i = 0; i < T; ++i) {
				q_re[set][i] = *reinterpret_cast<const float4 *>(b + i * 32 * KC);
				if (!REAL) q_im[set][i] = *reinterpret_cast<const float4 *>(b + PLANE + i * 32 * KC);
			}
		}
	}
	static __device__ __forceinline__ float comp(const float4 &v, int c) { return c == 0 ? v.x : (c == 1 ? v.y : (c == 2 ? v.z : v.w)); }
	__device__ __forceinline__ float re(int s, int i) const { return MCONTIG ? s_re[s & 1][i] : comp(q_re[s >> 2][i], s & 3); }
	__device__ __forceinline__ float im(int s, int i) const { return REAL ? 0.f : (MCONTIG ? s_im[s & 1][i] : comp(q_im[s >> 2][i], s & 3)); }
};

// One operand (both planes) of one K chunk, loaded straight into LDS.  A unit is one wave-wide instruction: lane l
// delivers 16 bytes to LDS float offset (unit * 64 + l) * 4 of the plane, unit = u * 4 + wavefront.
//   MCONTIG: the plane is [k][ROWS] (pitch ROWS): the unit covers 256 / ROWS lines of k.
//   otherwise: the plane is [row][KC] with the 16-byte groups of a row XOR-swizzled by bits 2..3 of the row; LDS
//   position (row, q) receives global group q ^ swizzle(row).
template <int ROWS, bool MCONTIG>
struct DlStage {
	static constexpr int UNITS = ROWS * KC / 256 / 4;
	static constexpr int PITCH = MCONTIG ? ROWS : KC;
	static constexpr int PLANE = ROWS * KC;
	unsigned goff[UNITS];  // byte offset of this lane's 16 bytes inside the operand tile of a chunk
	int wave_s;            // wavefront number, held in a scalar register

	// rows_valid: rows of the operand that exist from the first row of this block on (>= ROWS inside the matrix).  Rows
	// past the end are fetched from the last valid ones instead: what they produce lies outside C and is never stored.
	// When MCONTIG a line of k is fetched in groups of four rows, so the last group may reach up to three floats past the
	// rows that exist: they lie inside the line (the leading dimension is a multiple of four) and feed only rows of C that
	// do not exist either.
	__device__ __forceinline__ void init(long ld, int rows_valid) {
		const int wave = threadIdx.x >> 6;
		wave_s = __builtin_amdgcn_readfirstlane(wave);
		const int lane = threadIdx.x & 63;
#pragma unroll
		for (int u = 0; u < UNITS; ++u) {
			const int pos = ((u * 4 + wave) * 64 + lane) * 4;  // float offset inside the LDS plane
			if (MCONTIG) {
				const int k = pos / ROWS, row = min(pos % ROWS, ((rows_valid + 3) & ~3) - 4);
				goff[u] = (unsigned) (((long) k * ld + row) * 4);
			} else {
				const int row = pos / KC, q = (pos % KC) / 4;
				goff[u] = (unsigned) (((long) min(row, rows_valid - 1) * ld + ((q ^ ((row >> 2) & 3)) * 4)) * 4);
			}
		}
	}
	__device__ __forceinline__ void issue(int u, const float *tile_re, const float *tile_im, float *sre, float *sim) const {
#if defined(__HIP_DEVICE_COMPILE__)
		// Written as assembly on purpose: for the builtin the compiler cannot tell which LDS reads the transfer may
		// alias and puts a vmcnt(0) wait in front of the first fragment read of the current chunk, which exposes the
		// whole memory latency once per chunk.  The wait that is needed (before the barrier that publishes the stage)
		// is in the kernel.  m0 = LDS byte address of the KiB this wavefront fills; one wait state before its use.
		const unsigned dst = (unsigned) ((u * 4 + wave_s) * 1024);  // scalar arithmetic: nothing for the vector ALU
		const unsigned lre = (unsigned) (size_t) sre + dst;
		const unsigned lim = (unsigned) (size_t) sim + dst;
		asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(goff[u]), "s"(tile_re), "s"(lre) : "memory", "m0");
		asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(goff[u]), "s"(tile_im), "s"(lim) : "memory", "m0");
#endif
	}
	// the real plane only (an operand whose imaginary plane is not read)
	__device__ __forceinline__ void issue_re(int u, const float *tile_re, float *sre) const {
#if defined(__HIP_DEVICE_COMPILE__)
		const unsigned dst = (unsigned) ((u * 4 + wave_s) * 1024);
		const unsigned lre = (unsigned) (size_t) sre + dst;
		asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(goff[u]), "s"(tile_re), "s"(lre) : "memory", "m0");
#endif
	}
};

// Signs (conj) are applied to the fragments.  NST stages of LDS: chunk c + NST - 1 is requested while chunk c is
// multiplied, so with three stages a transfer has two chunks of MFMA time to arrive (the small blocks, whose chunk is
// shorter than a memory round trip, use three; 128 x 128 has room for two).
// waves_per_eu(2, 4): LDS allows at most four workgroups per compute unit anyway, so the register allocator need not
// squeeze the small blocks for an occupancy that cannot materialise.
// GAUSS: three real products per complex one instead of four (P = Ar Br, Q = Ai Bi, T = (Ar + sa Ai)(Br + sb Bi) with
// sa, sb the signs of the imaginary parts: re = P - sa sb Q, im = T - P - sa sb Q).  A quarter of the matrix work less,
// for one addition per operand fragment and k pair; the imaginary part then carries the rounding of all three products
// (normwise as accurate as four products, not componentwise).
// The last two template arguments name the form of the complex product:
//   THREE, REAL_A = false, false  four real products (or two sets of accumulators with signs, see below)
//   true, false                   three real products (Gauss; CgemmArgs via cnet_cgemm_set_products)
//   false, true                   the imaginary plane of A is all +0 and is neither fetched nor multiplied
//                                 (CgemmArgs::a_real == 1): two real products, re = Ar Br, im = Ar Bi
//   true, true                    the planes of A are two real operands of their own, C = (Ar Br) + i (Ai Bi)
//                                 (CgemmArgs::a_real == 2, the folded samples of a transform): two real products
template <int BM, int BN, int WM, int WN, bool A_MCONTIG, bool B_NCONTIG, int NST, bool THREE = false, bool REAL_A = false>
__global__ __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 4))) void cgemm_fast_kernel(const CgemmArgs args) {
	static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per workgroup");
	constexpr bool A_FOLD = THREE && REAL_A, GAUSS = THREE && !REAL_A, A_REAL = REAL_A && !THREE;
	constexpr int TM = WM / 32, TN = WN / 32;
	typedef DlStage<BM, A_MCONTIG> StageA;
	typedef DlStage<BN, B_NCONTIG> StageB;
	constexpr int A_PLANE = StageA::PLANE, B_PLANE = StageB::PLANE;
	constexpr int STAGE_FLOATS = 2 * A_PLANE + 2 * B_PLANE;
	constexpr int KS = KC / 2;  // k pairs (MFMA k extent = 2) per chunk
#ifndef CNET_SCHED_RECIPE
#define CNET_SCHED_RECIPE 1
#endif
	constexpr bool SCHED_RECIPE = CNET_SCHED_RECIPE;
	extern __shared__ float smem[];

	const int grid_n = grid_tiles_n(args);
	const int total = args.tiles_m * grid_n;  // blocks of C per problem
	const int K = args.K;
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int wm0 = (wave / (BN / WN)) * WM;
	const int wn0 = (wave % (BN / WN)) * WN;
	const int r = lane & 31, h = lane >> 5;

	// Work of this workgroup: one block of C; with a triangular operand the mirrored column block j -> tiles_n - 1 - j
	// as a second pass (every workgroup then walks the same number of K chunks in total); with tail blocks (see
	// CgemmArgs) the first tail_tiles x tail_splits workgroups also compute one K piece of a tail block as a second
	// pass: every workgroup of the launch has the same amount of work, wherever the hardware places it.
	int tile_m_first = 0, tile_n_first = 0;
	if (!args.tail_tiles) map_block(args, blockIdx.x, grid_n, tile_m_first, tile_n_first);
	int npass = 1;
	if (args.tri && tile_n_first != args.tiles_n - 1 - tile_n_first) npass = 2;
	if (args.tail_tiles && (int) blockIdx.x < args.tail_tiles * args.tail_splits) npass = 2;

	// Accumulators.  A wavefront with one or two tiles keeps the four real products apart (P = Ar Br, R = Ar Bi, Q = Ai Bi,
	// S = Ai Br) and combines them with their signs when it stores, so its K loop has no vector-ALU instruction for signs at
	// all; with four tiles there are only registers for two sets, re = P -+ Q and im = +-R +- S, and one operand of the
	// second product is negated per k pair (see the modes below).
	constexpr bool ACC4 = TM * TN <= 2 && !A_REAL && !A_FOLD;
	constexpr bool ACC_Q = ACC4 || GAUSS, ACC_S = ACC4 && !GAUSS;
	floatx16 acc_re[TM][TN], acc_im[TM][TN], acc_q[ACC_Q ? TM : 1][ACC_Q ? TN : 1], acc_s[ACC_S ? TM : 1][ACC_S ? TN : 1];
	for (int pass = 0; pass < npass; ++pass) {
	int prob = blockIdx.y, tile_m = tile_m_first, tile_n = pass ? args.tiles_n - 1 - tile_n_first : tile_n_first;
	int piece = -1, tail_block = 0;  // piece >= 0: this pass computes one K piece of a tail block
	if (args.tail_tiles) {
		int w = blockIdx.x;
		if (pass) {
			tail_block = blockIdx.x / args.tail_splits;
			piece = blockIdx.x - tail_block * args.tail_splits;
			w = total * args.nprob - args.tail_tiles + tail_block;
		}
		prob = w / total;
		map_block(args, w - prob * total, grid_n, tile_m, tile_n);
	}
	CgemmProblem pb = args.p[prob];
	batch_offset(pb, args);
	long ldc;
	int accumulate;
	output_planes(args, pb, ldc, accumulate);
	const int m0 = tile_m * BM, n0 = tile_n * BN;
	if (pass) __syncthreads();  // every wave has finished reading the last stage of the previous block
#pragma unroll
	for (int i = 0; i < TM; ++i)
#pragma unroll
		for (int j = 0; j < TN; ++j)
#pragma unroll
			for (int e = 0; e < 16; ++e) {
				acc_re[i][j][e] = 0.f;
				acc_im[i][j][e] = 0.f;
				if (ACC_Q) acc_q[i][j][e] = 0.f;
				if (ACC_S) acc_s[i][j][e] = 0.f;
			}

	StageA sa;
	StageB sb;
	sa.init(args.lda, args.M - m0);
	sb.init(args.ldb, args.N - n0);
	constexpr int UA = StageA::UNITS, UB = StageB::UNITS;

	// uniform tile bases of chunk 0 and the per-chunk advance (elements)
	const long a_tile0 = A_MCONTIG ? (long) m0 : (long) m0 * args.lda;
	const long b_tile0 = B_NCONTIG ? (long) n0 : (long) n0 * args.ldb;
	const long a_step = A_MCONTIG ? (long) KC * args.lda : (long) KC;
	const long b_step = B_NCONTIG ? (long) KC * args.ldb : (long) KC;
	int c_lo, c_hi;
	chunk_range<BN>(args, n0, c_lo, c_hi);
	int row_org = 0, col_org = 0;  // what the stores subtract from (row, col): a piece writes block-local coordinates
	if (piece >= 0) {
		c_lo = piece * args.tail_chunks;
		c_hi = min(c_hi, c_lo + args.tail_chunks);
		pb.c_re = args.partial + ((long) (tail_block * args.tail_splits + piece) * 2) * (BM * BN);
		pb.c_im = pb.c_re + BM * BN;
		ldc = BN;
		accumulate = 0;
		row_org = m0;
		col_org = n0;
	}

	// all units of one chunk of both operands into the stage at `stage`
	auto issue_chunk = [&](int chunk, float *stage) {
#pragma unroll
		for (int u = 0; u < UA; ++u) {
			if (A_REAL)
				sa.issue_re(u, pb.a_re + a_tile0 + chunk * a_step, stage);
			else
				sa.issue(u, pb.a_re + a_tile0 + chunk * a_step, pb.a_im + a_tile0 + chunk * a_step, stage, stage + A_PLANE);
		}
#pragma unroll
		for (int u = 0; u < UB; ++u)
			sb.issue(u, pb.b_re + b_tile0 + chunk * b_step, pb.b_im + b_tile0 + chunk * b_step, stage + 2 * A_PLANE,
					stage + 2 * A_PLANE + B_PLANE);
	};
	// Signs of the imaginary parts (conj): (Ar + i sa Ai)(Br + i sb Bi) = (Ar Br - sa sb Ai Bi) + i (sb Ar Bi + sa Ai Br).
	// Which operand is negated is a compile-time property of the loop below, so the only vector-ALU work per k pair is one
	// negation per A fragment (every VALU instruction costs the matrix pipe a few cycles: it shares its issue port):
	//   mode 0 (no conj):  re += Ar Br + (-Ai) Bi   im += Ar Bi + Ai Br
	//   mode 1 (conj B):   re += Ar Br + Ai Bi      im += (-Ar) Bi + Ai Br
	//   mode 2 (conj A):   re += Ar Br + Ai Bi      im += Ar Bi + (-Ai) Br
	//   mode 3 (both):     re += Ar Br + (-Ai) Bi   im += Ar Bi + Ai Br, negated when it is stored
	const int mode = (pb.a_im_sign < 0.f ? 2 : 0) | (pb.b_im_sign < 0.f ? 1 : 0);
	const float sign_a = pb.a_im_sign < 0.f ? -1.f : 1.f, sign_b = pb.b_im_sign < 0.f ? -1.f : 1.f;  // uniform: scalar registers

	constexpr int LOADS_PER_CHUNK = (A_REAL ? 1 : 2) * UA + 2 * UB;  // transfers one wavefront issues per chunk
	static_assert(NST == 2 || NST == 3, "two or three stages");
	static_assert(LOADS_PER_CHUNK < 16, "fits the low bits of the vmcnt field");
#pragma unroll
	for (int d = 0; d < NST - 1; ++d)
		if (c_lo + d < c_hi) issue_chunk(c_lo + d, smem + d * STAGE_FLOATS);
	__builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the tiles have landed in LDS
	__syncthreads();

	Frag<TM, A_MCONTIG, StageA::PITCH, A_PLANE, A_REAL> fa;
	Frag<TN, B_NCONTIG, StageB::PITCH, B_PLANE> fb;
	fa.init(smem, wm0, r, h);
	fb.init(smem + 2 * A_PLANE, wn0, r, h);
	fa.fetch_step(0, 0);
	fb.fetch_step(0, 0);
	fa.fetch_set(0, 0);
	fb.fetch_set(0, 0);

	// One chunk, held in stage `cur`.
	auto chunk = [&](int cur, auto mode_c, int c) __attribute__((always_inline)) {
		constexpr int MODE = decltype(mode_c)::value;
		const int nxt = cur + 1 == NST ? 0 : cur + 1, far = cur == 0 ? NST - 1 : cur - 1;
		const int CUR = cur * STAGE_FLOATS, NXT = nxt * STAGE_FLOATS, FAR = far * STAGE_FLOATS;
		const bool ahead = (c + NST - 1 < c_hi);
		if (ahead) issue_chunk(c + NST - 1, smem + FAR);
#pragma unroll
		for (int ks = 0; ks < KS; ++ks) {
			if (ks + 1 < KS) {
				fa.fetch_step(CUR, ks + 1);
				fb.fetch_step(CUR, ks + 1);
			}
			if (ks == 0) {  // second half of this chunk for the [row][k] operands
				fa.fetch_set(CUR, 1);
				fb.fetch_set(CUR, 1);
			}
			if (ks == KS - 1) {
				// this wavefront's part of the next chunk is in LDS (transfers complete in order: with three stages the
				// ones just issued for the chunk after it may still be in flight)
				if (NST == 3 && ahead)
					__builtin_amdgcn_s_waitcnt(0x0F70 | LOADS_PER_CHUNK);
				else
					__builtin_amdgcn_s_waitcnt(0x0F70);
				__syncthreads();
				fa.fetch_step(NXT, 0);
				fb.fetch_step(NXT, 0);
				fa.fetch_set(NXT, 0);
				fb.fetch_set(NXT, 0);
			}
			float are[TM], aim[TM], neg[TM], bre[TN], bim[TN];
#pragma unroll
			for (int i = 0; i < TM; ++i) {
				are[i] = fa.re(ks, i);
				aim[i] = fa.im(ks, i);
				if (!ACC4 && !GAUSS && !A_REAL && !A_FOLD) neg[i] = MODE == 1 ? -are[i] : -aim[i];
			}
#pragma unroll
			for (int j = 0; j < TN; ++j) {
				bre[j] = fb.re(ks, j);
				bim[j] = fb.im(ks, j);
			}
			if constexpr (A_FOLD) {
#pragma unroll
				for (int i = 0; i < TM; ++i)
#pragma unroll
					for (int j = 0; j < TN; ++j) {
						acc_re[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[i], bre[j], acc_re[i][j], 0, 0, 0);
						acc_im[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(aim[i], bim[j], acc_im[i][j], 0, 0, 0);
					}
			} else if constexpr (A_REAL) {
#pragma unroll
				for (int i = 0; i < TM; ++i)
#pragma unroll
					for (int j = 0; j < TN; ++j) {
						acc_re[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[i], bre[j], acc_re[i][j], 0, 0, 0);
						acc_im[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[i], bim[j], acc_im[i][j], 0, 0, 0);
					}
			} else if constexpr (GAUSS) {
				float asum[TM], bsum[TN];
#pragma unroll
				for (int i = 0; i < TM; ++i) asum[i] = fmaf(sign_a, aim[i], are[i]);
#pragma unroll
				for (int j = 0; j < TN; ++j) bsum[j] = fmaf(sign_b, bim[j], bre[j]);
#pragma unroll
				for (int i = 0; i < TM; ++i)
#pragma unroll
					for (int j = 0; j < TN; ++j) {
						acc_re[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[i], bre[j], acc_re[i][j], 0, 0, 0);    // P
						acc_q[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(aim[i], bim[j], acc_q[i][j], 0, 0, 0);      // Q
						acc_im[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(asum[i], bsum[j], acc_im[i][j], 0, 0, 0);  // T
					}
			} else if constexpr (ACC4) {
#pragma unroll
				for (int i = 0; i < TM; ++i)
#pragma unroll
					for (int j = 0; j < TN; ++j) {
						acc_re[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[i], bre[j], acc_re[i][j], 0, 0, 0);  // P
						acc_im[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[i], bim[j], acc_im[i][j], 0, 0, 0);  // R
					}
#pragma unroll
				for (int i = 0; i < TM; ++i)
#pragma unroll
					for (int j = 0; j < TN; ++j) {
						acc_q[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(aim[i], bim[j], acc_q[i][j], 0, 0, 0);  // Q
						acc_s[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(aim[i], bre[j], acc_s[i][j], 0, 0, 0);  // S
					}
			} else {
#pragma unroll
				for (int i = 0; i < TM; ++i)
#pragma unroll
					for (int j = 0; j < TN; ++j) {
						acc_re[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(are[i], bre[j], acc_re[i][j], 0, 0, 0);
						acc_im[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(MODE == 1 ? neg[i] : are[i], bim[j], acc_im[i][j], 0, 0, 0);
					}
#pragma unroll
				for (int i = 0; i < TM; ++i)
#pragma unroll
					for (int j = 0; j < TN; ++j) {
						acc_re[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32((MODE == 0 || MODE == 3) ? neg[i] : aim[i], bim[j], acc_re[i][j], 0, 0, 0);
						acc_im[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(MODE == 2 ? neg[i] : aim[i], bre[j], acc_im[i][j], 0, 0, 0);
					}
			}
			if (SCHED_RECIPE && ks < KS - 1) {
				// scheduling recipe for this k pair: after each MFMA let a few of the pending VALU / LDS / global
				// instructions issue, so they run in the shadow of the matrix pipe
#pragma unroll
				for (int q = 0; q < ((A_REAL || A_FOLD) ? 2 : GAUSS ? 3 : 4) * TM * TN; ++q) {
					__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
					__builtin_amdgcn_sched_group_barrier(0x002, 2, 0);  // <= 2 VALU
					__builtin_amdgcn_sched_group_barrier(0x080, 1, 0);  // <= 1 LDS
					__builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // <= 1 global load
				}
			}
			__builtin_amdgcn_sched_barrier(0);
		}
	};
	// the chunks of this block: chunk c_lo + n sits in stage n % NST.  The loop body is one round over the stages, so the
	// stage part of every LDS address is an immediate (no address additions in the loop); what is left over after the
	// last full round follows the loop.
	auto kloop = [&](auto mode_c) __attribute__((always_inline)) {
		int c = c_lo;
		if constexpr (NST == 2) {
			for (; c + 1 < c_hi; c += 2) {
				chunk(0, mode_c, c);
				chunk(1, mode_c, c + 1);
			}
			if (c < c_hi) chunk(0, mode_c, c);
		} else {
			for (; c + 2 < c_hi; c += 3) {
				chunk(0, mode_c, c);
				chunk(1, mode_c, c + 1);
				chunk(2, mode_c, c + 2);
			}
			if (c < c_hi) chunk(0, mode_c, c);
			if (c + 1 < c_hi) chunk(1, mode_c, c + 1);
		}
	};
	if constexpr (ACC4 || GAUSS || A_REAL || A_FOLD) {
		kloop(std::integral_constant<int, 0>());  // the signs wait for the store
	} else {
		switch (mode) {
		case 0: kloop(std::integral_constant<int, 0>()); break;
		case 1: kloop(std::integral_constant<int, 1>()); break;
		case 2: kloop(std::integral_constant<int, 2>()); break;
		default: kloop(std::integral_constant<int, 3>()); break;
		}
	}
	const bool q_minus = mode == 0 || mode == 3, r_minus = (mode & 1) != 0, s_minus = (mode & 2) != 0;
	// The addresses of the stores are formed here, after the loop: left to itself the compiler computes them before the
	// loop, where the registers are full, and spills them.
	int r_st = r, h_st = h;
	asm volatile("" : "+v"(r_st), "+v"(h_st));
	const bool mirror_now = args.mirror && piece < 0 && args.splits == 1;  // partial blocks are mirrored when they are added up

#pragma unroll
	for (int i = 0; i < TM; ++i)
#pragma unroll
		for (int j = 0; j < TN; ++j) {
			const int col = n0 + wn0 + j * 32 + r_st;
			if (col >= args.N) continue;  // blocks on the right and bottom edge of C are partly outside
#pragma unroll
			for (int e = 0; e < 16; ++e) {
				const int row = m0 + wm0 + i * 32 + (e >> 2) * 8 + h_st * 4 + (e & 3);
				if (row < args.M) {
					const long off = (long) (row - row_org) * ldc + (col - col_org);
					float vr, vi;
					if constexpr (A_FOLD) {
						vr = acc_re[i][j][e];
						vi = acc_im[i][j][e];
					} else if constexpr (A_REAL) {
						vr = acc_re[i][j][e];
						vi = r_minus ? -acc_im[i][j][e] : acc_im[i][j][e];
					} else if constexpr (GAUSS) {
						const float p = acc_re[i][j][e], q = q_minus ? acc_q[i][j][e] : -acc_q[i][j][e];  // q_minus: sa sb = +1
						vr = p - q;
						vi = (acc_im[i][j][e] - p) - q;
					} else if constexpr (ACC4) {
						const float q = acc_q[i][j][e], rr = acc_im[i][j][e], ss = acc_s[i][j][e];
						vr = q_minus ? acc_re[i][j][e] - q : acc_re[i][j][e] + q;
						vi = (r_minus ? -rr : rr) + (s_minus ? -ss : ss);
					} else {
						vr = acc_re[i][j][e];
						vi = mode == 3 ? -acc_im[i][j][e] : acc_im[i][j][e];
					}
					if (mirror_now) {
						mirror_store(args, (long) row * args.ldc + col, vr, vi);
						herm_store(args, row, col, vr, vi);
					}
					if (accumulate) {
						vr += pb.c_re[off];
						vi += pb.c_im[off];
					}
					pb.c_re[off] = vr;
					pb.c_im[off] = vi;
					if (mirror_now) gelu_store(args, (long) row * args.ldc + col, vr, vi);
				}
			}
		}
	}  // pass
}

// C (+)= sum over splits of the partial blocks, added in split order (deterministic).  One thread per element of one plane.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(CgemmArgs args, int nprob, int nbatch) {
	const long plane = (long) args.M * args.N;
	const long idx = (long) blockIdx.x * 256 + threadIdx.x;
	if (idx >= 2 * plane) return;
	const int prob = blockIdx.y, b = blockIdx.z;
	const int part = idx >= plane;  // 0: re, 1: im
	const long e = idx - part * plane;
	const long row = e / args.N, col = e - row * args.N;
	const float *first = args.partial + (((long) prob * nbatch + b) * 2 + part) * plane + e;
	float v = cnet::ordered_sum(first, (long) nprob * nbatch * 2 * plane, args.splits);
	float *c = (part ? args.p[prob].c_im : args.p[prob].c_re) + (long) b * args.stride_c + row * args.ldc + col;
	const float fin = args.accumulate ? *c + v : v;
	*c = fin;
	herm_store_part(args, part, (int) row, (int) col, v);
	if (args.mirror == MIRROR_CONJ) {
		float *m = (part ? args.p[1].c_im : args.p[1].c_re) + row * args.ldc + col;
		const float mv = part ? -v : v;
		*m = args.accumulate ? *m + mv : mv;
	} else if (args.mirror == MIRROR_GELU) {
		(part ? args.p[1].c_im : args.p[1].c_re)[row * args.ldc + col] = cnet::gelu_value(fin);
	}
}

// C (+)= sum over the K pieces of each tail block, added in piece order.  blockIdx.x = tail block, blockIdx.y = a slice
// of its two planes.
template <int BM, int BN>
__global__ __launch_bounds__(256) void tail_reduce_kernel(CgemmArgs args) {
	const int grid_n = grid_tiles_n(args);
	const int total = args.tiles_m * grid_n;
	const int w = total * args.nprob - args.tail_tiles + blockIdx.x;
	const int prob = w / total;
	int tile_m, tile_n;
	map_block(args, w - prob * total, grid_n, tile_m, tile_n);
	const int m0 = tile_m * BM, n0 = tile_n * BN;
	const float *first = args.partial + ((long) blockIdx.x * args.tail_splits * 2) * (BM * BN);
	// blockIdx.y = which 1024 of the 2 x BM x BN values of the block
	for (int idx = blockIdx.y * 1024 + threadIdx.x; idx < (int) (blockIdx.y + 1) * 1024; idx += 256) {
		const int part = idx / (BM * BN), e = idx - part * (BM * BN);
		const int row = m0 + e / BN, col = n0 + e % BN;
		if (row >= args.M || col >= args.N) continue;
		const float v = cnet::ordered_sum(first + idx, 2L * BM * BN, args.tail_splits);
		float *c = (part ? args.p[prob].c_im : args.p[prob].c_re) + (long) row * args.ldc + col;
		const float fin = args.accumulate ? *c + v : v;
		*c = fin;
		herm_store_part(args, part, row, col, v);
		if (args.mirror == MIRROR_CONJ) {
			float *m = (part ? args.p[1].c_im : args.p[1].c_re) + (long) row * args.ldc + col;
			const float mv = part ? -v : v;
			*m = args.accumulate ? *m + mv : mv;
		} else if (args.mirror == MIRROR_GELU) {
			(part ? args.p[1].c_im : args.p[1].c_re)[(long) row * args.ldc + col] = cnet::gelu_value(fin);
		}
	}
}

// ---- small C: one 16 x 16 tile per workgroup, K shared out among its wavefronts ---------------------------------------
//
// A product with a small C (a batch of 64 rows against a 784-long reduction) has too few blocks for the kernels above
// and is bound by latency, not by arithmetic.  Here a workgroup of W wavefronts owns one 16 x 16 tile of C (small, so
// that even a 64 x 784 result spreads over 196 compute units); wavefront w walks the w-th part of K with its operands
// loaded straight from global memory into the MFMA operand registers (no LDS staging: nothing is shared between
// wavefronts but the tile of C), three groups of 16 k values in flight.  The W partial tiles meet in LDS and are added
// in wavefront order, so the result does not depend on timing, and C is written once: no second kernel.  Lane (r, q) of
// a wavefront, r = lane % 16, feeds row / column r of the tile; step s of a group (v_mfma_f32_16x16x4_f32) takes k =
// 16 g + 4 q + s from lane quarter q, which lets an operand that is contiguous along K arrive as one float4 per plane.
// What makes the loop run at the pace of its 16 MFMAs per group: the loop body has no branch (otherwise the compiler
// waits for every load in flight at the top of each round), the ring slots are refilled after use, in place (no register
// copies), the wavefront number is a scalar, and addresses are 32-bit offsets into buffer descriptors.
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Four k values of one plane for this lane, through a buffer descriptor of the plane: the lane's part of the address
// is a 32-bit byte offset shared by the re and im planes (one integer add per load instead of 64-bit address
// arithmetic, which would cost this kernel more issue cycles than its MFMAs), every load is unconditional, so the loads
// of several groups stay in flight together, and a load past the end of the plane returns zero instead of faulting.
template <bool V4>
__device__ __forceinline__ void load_k4(__amdgpu_buffer_rsrc_t plane, unsigned lane_bytes, unsigned kstride_bytes, int k, float v[4]) {
	if constexpr (V4) {
		const floatx4 t = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(plane, lane_bytes + 4u * k, 0, 0));
		v[0] = t[0];
		v[1] = t[1];
		v[2] = t[2];
		v[3] = t[3];
	} else {
#pragma unroll
		for (int s = 0; s < 4; ++s)
			v[s] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(plane, lane_bytes + (unsigned) (k + s) * kstride_bytes, 0, 0));
	}
}

// descriptor of `bytes` bytes at p: raw 32-bit data, no swizzle, loads checked against `bytes`
__device__ __forceinline__ __amdgpu_buffer_rsrc_t plane_rsrc(const float *p, unsigned bytes) {
	return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p), 0, bytes, 0x00020000);
}

// how the lanes of cgemm_skinny_kernel step through the two operands (elements), and the length of each plane (bytes)
struct SkinnyStrides {
	unsigned a_kstride, a_mstride, b_kstride, b_nstride, a_bytes, b_bytes;
};

// the tile (tile_m, tile_n) of the product `args`; red = W x 2 x 4 x 64 floats of LDS ([W][re, im][4][64]).  KEEP: the finished
// values (what the planes of C hold afterwards) also go to keep[re, im][row of C][16] in LDS, for a workgroup that goes on
// with them.  SOLO: the calling wavefront forms the tile alone, for a K of one group (K <= 16), where the other wavefronts
// of a workgroup would only add zeros: no LDS, no barrier, the same bits; the wavefronts of a workgroup can then take
// different tiles at the same time.
template <int W, bool A_V4, bool B_V4, bool CE = false, bool KEEP = false, bool SOLO = false>
__device__ __forceinline__ void skinny_tile_at(const CgemmArgs &args, const SkinnyStrides &st, const int tile_m, const int tile_n, float *red,
		float *keep = nullptr) {
	constexpr int WS = SOLO ? 1 : W;  // wavefronts that share K
	const unsigned a_kstride = st.a_kstride, a_mstride = st.a_mstride, b_kstride = st.b_kstride, b_nstride = st.b_nstride;
	const unsigned a_bytes = st.a_bytes, b_bytes = st.b_bytes;
	constexpr int DEPTH = 3;  // (5 and 8 groups in flight measured 4 to 20 % slower: the loop is not waiting for memory)
	// the wavefront number as a scalar: the K range, the loop over it and its branches then run on the scalar unit
	const int wave = SOLO ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const int lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
	CgemmProblem pb = args.p[blockIdx.y];
	batch_offset(pb, args);
	const int m0 = tile_m * 16, n0 = tile_n * 16;
	// lanes beyond the edge of C read the last valid row / column again; their results are not stored
	const unsigned a_off = 4u * min(m0 + r, args.M - 1) * a_mstride, b_off = 4u * min(n0 + r, args.N - 1) * b_nstride;  // bytes
	const __amdgpu_buffer_rsrc_t a_re = plane_rsrc(pb.a_re, a_bytes), a_im = plane_rsrc(pb.a_im, a_bytes);
	const __amdgpu_buffer_rsrc_t b_re = plane_rsrc(pb.b_re, b_bytes), b_im = plane_rsrc(pb.b_im, b_bytes);
	// this workgroup's groups of K (all of them, or one slice when a long K is cut across workgroups), then this wavefront's
	const int all_groups = (args.K + 15) / 16;
	int first = 0, last = all_groups;
	if (args.splits > 1) {
		first = (blockIdx.z % args.splits) * args.chunks_per_split;
		last = min(last, first + args.chunks_per_split);
	}
	const int per = (last - first + WS - 1) / WS;
	const int g_lo = first + wave * per, g_hi = min(last, g_lo + per);
	long ldc;
	int accumulate;
	output_planes(args, pb, ldc, accumulate);  // C, or the slice of the partial planes that splitk_reduce_kernel adds up

	struct Group {
		float ar[4], ai[4], br[4], bi[4];
	};
	auto fetch = [&](Group &t, int g) __attribute__((always_inline)) {
		const int k = g * 16 + 4 * q;
		load_k4<A_V4>(a_re, a_off, 4u * a_kstride, k, t.ar);
		load_k4<A_V4>(a_im, a_off, 4u * a_kstride, k, t.ai);
		load_k4<B_V4>(b_re, b_off, 4u * b_kstride, k, t.br);
		load_k4<B_V4>(b_im, b_off, 4u * b_kstride, k, t.bi);
	};
	// four independent accumulator chains, P = Ar Br, R = Ar Bi, Q = Ai Bi, S = Ai Br: no MFMA waits for the one before
	// it, and the conjugation signs wait until the sums are complete
	const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
	floatx4 acc_p = zero, acc_r = zero, acc_q = zero, acc_s = zero;
	Group buf[DEPTH];
	if constexpr (SOLO) {
		fetch(buf[0], g_lo);  // the one group there is
	} else {
#pragma unroll
		for (int d = 0; d < DEPTH; ++d) fetch(buf[d], g_lo + d);
	}
	// One group: what lies past the end of K is zeroed first (an operand stored along K has its next row or padding
	// there; four selects per plane, nothing next to 16 MFMAs), then P, R, Q, S advance by four k values per step.
	auto use = [&](Group &t, int g) __attribute__((always_inline)) {
		const int left = args.K - (g * 16 + 4 * q);
#pragma unroll
		for (int s = 0; s < 4; ++s) {
			const bool in = s < left;
			t.ar[s] = in ? t.ar[s] : 0.f;
			t.ai[s] = in ? t.ai[s] : 0.f;
			t.br[s] = in ? t.br[s] : 0.f;
			t.bi[s] = in ? t.bi[s] : 0.f;
		}
#pragma unroll
		for (int s = 0; s < 4; ++s) {
			acc_p = __builtin_amdgcn_mfma_f32_16x16x4f32(t.ar[s], t.br[s], acc_p, 0, 0, 0);
			acc_r = __builtin_amdgcn_mfma_f32_16x16x4f32(t.ar[s], t.bi[s], acc_r, 0, 0, 0);
			acc_q = __builtin_amdgcn_mfma_f32_16x16x4f32(t.ai[s], t.bi[s], acc_q, 0, 0, 0);
			acc_s = __builtin_amdgcn_mfma_f32_16x16x4f32(t.ai[s], t.br[s], acc_s, 0, 0, 0);
		}
	};
	// Slot d of the ring is used, then refilled with the group DEPTH further on (in this order, so that the loaded values
	// stay in the registers they arrived in).  The loop body is one round over the slots without a branch, which lets
	// the compiler count the loads in flight instead of waiting for all of them; the refill is unconditional (beyond
	// this wavefront's range it is not used), and what is left after the last full round follows the loop.
	if constexpr (SOLO) {
		if (g_lo < g_hi) use(buf[0], g_lo);
	} else {
		int g = g_lo;
		for (; g + DEPTH <= g_hi; g += DEPTH) {
#pragma unroll
			for (int d = 0; d < DEPTH; ++d) {
				use(buf[d], g + d);
				fetch(buf[d], g + d + DEPTH);
			}
		}
#pragma unroll
		for (int d = 0; d < DEPTH - 1; ++d)
			if (g + d < g_hi) use(buf[d], g + d);
	}
	// re = Ar Br - (sa Ai)(sb Bi), im = Ar (sb Bi) + (sa Ai) Br
	const float sa = pb.a_im_sign, sb = pb.b_im_sign, sq = -sa * sb;
	float solo[2][4];
#pragma unroll
	for (int e = 0; e < 4; ++e) {
		const float fr = acc_p[e] + sq * acc_q[e], fi = sb * acc_r[e] + sa * acc_s[e];
		if (SOLO) {
			solo[0][e] = fr;
			solo[1][e] = fi;
		} else {
			red[((wave * 2 + 0) * 4 + e) * 64 + lane] = fr;
			red[((wave * 2 + 1) * 4 + e) * 64 + lane] = fi;
		}
	}
	if (!SOLO) __syncthreads();
	const int col = n0 + r;
	if (!SOLO && args.mirror == MIRROR_HGELU) {
		// both planes of an element by one lane (the gate needs the complex value): the 4 accumulator registers go to the first
		// four wavefronts; each plane is added in wavefront order, as below
		for (int e = wave; e < 4; e += W) {
			float vr = 0.f, vi = 0.f;
#pragma unroll
			for (int w = 0; w < W; ++w) {
				vr += red[((w * 2 + 0) * 4 + e) * 64 + lane];
				vi += red[((w * 2 + 1) * 4 + e) * 64 + lane];
			}
			const int row = m0 + 4 * q + e;
			if (row < args.M && col < args.N) {
				const long off = (long) row * ldc + col;
				pb.c_re[off] = vr;
				pb.c_im[off] = vi;
				const float wr = args.hv_re[col], wi = args.hv_im[col];
				const float hr = vr * wr - vi * wi, hi = vr * wi + vi * wr;
				args.p[1].c_re[off] = hr;
				args.p[1].c_im[off] = hi;
				args.g_re[off] = cnet::gelu_value(hr);
				args.g_im[off] = cnet::gelu_value(hi);
			}
		}
		return;
	}
	// the 8 (plane, accumulator register) pairs are added and stored by the first wavefronts, one or two pairs each
	__shared__ float logits[CE ? 2 * 16 * 16 : 1];  // CE: the finished tile, [re, im][row][col]
	auto finish = [&](const int part, const int e, const float v) __attribute__((always_inline)) {
		const int row = m0 + 4 * q + e;
		if (CE) logits[(part * 16 + 4 * q + e) * 16 + r] = v;
		if (row < args.M && col < args.N) {
			float *dst = (part ? pb.c_im : pb.c_re) + (long) row * ldc + col;
			const float fin = accumulate ? *dst + v : v;
			*dst = fin;
			if (KEEP) keep[(part * cnet::GATE_MAX_ROWS + row) * 16 + r] = fin;
			if (args.splits == 1) herm_store_part(args, part, row, col, v);
			if (args.mirror == MIRROR_CONJ && args.splits == 1) {
				float *m = (part ? args.p[1].c_im : args.p[1].c_re) + (long) row * args.ldc + col;
				const float mv = part ? -v : v;
				*m = args.accumulate ? *m + mv : mv;
			} else if (args.mirror == MIRROR_GELU && args.splits == 1) {
				(part ? args.p[1].c_im : args.p[1].c_re)[(long) row * args.ldc + col] = cnet::gelu_value(fin);
			}
		}
	};
	if constexpr (SOLO) {
		// (0 + x, as the sum over the wavefronts starts: a zero result is +0 either way)
#pragma unroll
		for (int c = 0; c < 8; ++c) finish(c >> 2, c & 3, 0.f + solo[c >> 2][c & 3]);
	} else {
		for (int c = wave; c < 8; c += W) {
			const int part = c >> 2, e = c & 3;
			float v = 0.f;
#pragma unroll
			for (int w = 0; w < W; ++w) v += red[((w * 2 + part) * 4 + e) * 64 + lane];
			finish(part, e, v);
		}
	}
	if constexpr (CE) {
		// the 16 rows of logits of this tile, one wavefront per row at a time: loss, argmax, normalised row and gradient
		__syncthreads();
		const cnet::rows::GradPlanes grad = {args.ce_dz_re, args.ce_dz_im, args.ce_dzs_re, args.ce_dzs_im, args.ce_lddz};
		for (int rr = wave; rr < 16 && m0 + rr < args.M; rr += W) {
			const float *pr = logits + rr * 16, *pi = logits + (16 + rr) * 16;
			if (args.ce_vec)
				cnet::rows::crossent_fwd_row_at<4, 1, true>(pr, pi, m0 + rr, true, lane, lane, 0, 0, nullptr, nullptr, nullptr, args.ce_labels,
						args.ce_out_re, args.ce_out_im, args.ce_ldo, args.ce_s, args.ce_loss, args.ce_argmax, args.N, grad, 0);
			else
				cnet::rows::crossent_fwd_row_at<1, 1, true>(pr, pi, m0 + rr, true, lane, lane, 0, 0, nullptr, nullptr, nullptr, args.ce_labels,
						args.ce_out_re, args.ce_out_im, args.ce_ldo, args.ce_s, args.ce_loss, args.ce_argmax, args.N, grad, 0);
		}
	}
}

// the tile that workgroup number `bx` of a launch over all tiles of `args` takes
template <int W, bool A_V4, bool B_V4, bool CE = false>
__device__ __forceinline__ void skinny_tile(const CgemmArgs &args, const SkinnyStrides &st, const int bx, float *red) {
	// Consecutive workgroup numbers go round-robin to the XCDs: give each XCD a contiguous run of tiles, row tiles
	// fastest, so that the tiles sharing columns of B meet in one L2 and each XCD reads its own part of B only.
	const int total = args.tiles_m * args.tiles_n, xcd = bx % NUM_XCD, share = total / NUM_XCD, extra = total % NUM_XCD;
	const int tile = xcd * share + min(xcd, extra) + bx / NUM_XCD;
	const int tile_n = tile / args.tiles_m;
	skinny_tile_at<W, A_V4, B_V4, CE>(args, st, tile - tile_n * args.tiles_m, tile_n, red);
}

template <int W, bool A_V4, bool B_V4, bool CE = false>
__global__ __launch_bounds__(64 * W) void cgemm_skinny_kernel(const CgemmArgs args, const SkinnyStrides st) {
	__shared__ float red[W * 2 * 4 * 64];
	skinny_tile<W, A_V4, B_V4, CE>(args, st, blockIdx.x, red);
}

// Two unrelated small products in one launch (the input gradient and the weight gradient of a narrow Linear layer, each
// a few microseconds of work behind a launch that costs as much): workgroups [0, tiles0) take the tiles of the first,
// the others those of the second.  Neither is cut along K or batched (blockIdx.z = 0); blockIdx.y is the problem of
// a pair, as in the plain kernel.
template <int W, bool A_V4, bool B_V4>
__global__ __launch_bounds__(64 * W) void cgemm_skinny_two_kernel(const CgemmArgs args0, const SkinnyStrides st0, const int tiles0,
		const CgemmArgs args1, const SkinnyStrides st1) {
	__shared__ float red[W * 2 * 4 * 64];
	if ((int) blockIdx.x < tiles0) skinny_tile<W, A_V4, B_V4>(args0, st0, blockIdx.x, red);
	else skinny_tile<W, A_V4, B_V4>(args1, st1, blockIdx.x - tiles0, red);
}

// The two backward products of a narrow Linear (args0: dx = g w, all rows of the batch, K <= 16; args1: dw = g^T x) and, behind
// them, the backward pass of the Hadamard gate with a shared row of weights whose CGelu produced x.  Workgroup n < tiles_n of
// dx forms columns 16 n .. 16 n + 15 of dx (a row tile per wavefront), keeps them in LDS, takes them through the CGelu and
// the gate (the arithmetic of hadamard_bwd_shared_sym_kernel, operation for operation) and adds the rows of the batch into
// dv in the order of that kernel and of slab_sum_sym_kernel<4, 64>; the workgroups after those take the tiles of dw, which
// the gate does not read.  The bits of the three launches it replaces, without their partial planes.  The gate's operands
// are fetched before the product starts.
template <int W, bool A_V4, bool B_V4>
__global__ __launch_bounds__(64 * W) void cgemm_skinny_gate_bwd_kernel(const CgemmArgs args0, const SkinnyStrides st0, const CgemmArgs args1,
		const SkinnyStrides st1, const cnet::GateBwd ga) {
	__shared__ float red[W * 2 * 4 * 64];  // the sums over the wavefronts of a tile of dw, or the slab sums of dv, [slab][re, im][16]
	__shared__ float keep[2 * cnet::GATE_MAX_ROWS * 16];  // [re, im][row][column of the tile]: dx, then the terms of dv
	if ((int) blockIdx.x >= args0.tiles_n) {
		skinny_tile<W, A_V4, B_V4>(args1, st1, blockIdx.x - args0.tiles_n, red);
		return;
	}
	constexpr int PER = cnet::GATE_MAX_ROWS * 16 / (64 * W);  // elements of the column block per thread, at most
	const int tn = blockIdx.x, n0 = tn * 16, rows = args0.M, cols = args0.N;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const int c = threadIdx.x & 15, col = n0 + c;
	const bool live = col < cols;
	float ua[PER], ub[PER], vc = 0.f, vd = 0.f;
	if (live) {
		vc = ga.v_re[col];
		vd = ga.v_im[col];
	}
#pragma unroll
	for (int j = 0; j < PER; ++j) {
		const int row = (threadIdx.x >> 4) + j * (4 * W);
		ua[j] = ub[j] = 0.f;
		if (live && row < rows) {
			ua[j] = ga.u_re[(long) row * ga.ldu + col];
			ub[j] = ga.u_im[(long) row * ga.ldu + col];
		}
	}
	for (int tm = wave; tm < args0.tiles_m; tm += W) skinny_tile_at<W, A_V4, B_V4, false, true, true>(args0, st0, tm, tn, red, keep);
	__syncthreads();  // keep holds the column block of dx
#pragma unroll
	for (int j = 0; j < PER; ++j) {
		const int row = (threadIdx.x >> 4) + j * (4 * W);
		if (!live || row >= rows) continue;
		const float a = ua[j], b = ub[j];
		float gr = keep[row * 16 + c], gi = keep[(cnet::GATE_MAX_ROWS + row) * 16 + c];
		{  // through the CGelu at h = u v, recomputed with the bits of the forward pass
			const float hr = a * vc - b * vd, hi = a * vd + b * vc;
			const float px = 0.5f * cnet::gelu_slope(hr), py = 0.5f * cnet::gelu_slope(hi);
			const float sm = px + py, df = px - py;
			const float o_r = gr * sm + gr * df, o_i = gi * sm + (-gi) * df;
			gr = o_r;
			gi = o_i;
		}
		if (ga.dh.dz_re) {
			const long off = (long) row * ga.lddh + col;
			ga.dh.dz_re[off] = gr;
			ga.dh.dz_im[off] = gi;
			if (ga.dh.dzs_re) {
				ga.dh.dzs_re[off] = gr;
				ga.dh.dzs_im[off] = -gi;
			}
		}
		{
			const float o_r = gr * vc - gi * vd, o_i = gr * vd + gi * vc;
			const long off = (long) row * ga.lddu + col;
			if (ga.accumulate) {
				ga.du.dz_re[off] = ga.du.dz_re[off] + o_r;
				ga.du.dz_im[off] = ga.du.dz_im[off] + o_i;
				if (ga.du.dzs_re) {
					ga.du.dzs_re[off] = ga.du.dzs_re[off] + o_r;
					ga.du.dzs_im[off] = ga.du.dzs_im[off] + (-o_i);
				}
			} else {
				ga.du.dz_re[off] = o_r;
				ga.du.dz_im[off] = o_i;
				if (ga.du.dzs_re) {
					ga.du.dzs_re[off] = o_r;
					ga.du.dzs_im[off] = -o_i;
				}
			}
		}
		keep[row * 16 + c] = gr * a - gi * b;
		keep[(cnet::GATE_MAX_ROWS + row) * 16 + c] = gr * b + gi * a;
	}
	__syncthreads();
	// dv: the sum of each slab of rows (at most 32 slabs: the host checks), then the slabs
	const int nslabs = ga.nslabs;
	for (int idx = threadIdx.x; idx < 32 * nslabs; idx += 64 * W) {
		const int k = idx >> 5, part = (idx >> 4) & 1;
		const float *term = keep + part * cnet::GATE_MAX_ROWS * 16 + c;
		const int r0 = k * ga.rows_per_slab, r1 = min(rows, r0 + ga.rows_per_slab);
		float acc[cnet::GATE_CS_Y];
#pragma unroll
		for (int ty = 0; ty < cnet::GATE_CS_Y; ++ty) {
			acc[ty] = 0.f;
			for (int row = r0 + ty; row < r1; row += cnet::GATE_CS_Y) acc[ty] += term[row * 16];
		}
		red[idx] = ((acc[0] + acc[1]) + acc[2]) + acc[3];
	}
	__syncthreads();
	if (threadIdx.x < 32 && live) {
		const int part = threadIdx.x >> 4;
		const int per = (nslabs + 3) / 4;
		float s = 0.f;
#pragma unroll
		for (int l = 0; l < 4; ++l) {
			const int k0 = min(nslabs, l * per), k1 = min(nslabs, k0 + per);
			float run = 0.f;  // the slabs of lane l, in order
			for (int k = k0; k < k1; ++k) run += red[k * 32 + threadIdx.x];
			s = l == 0 ? run : s + run;
		}
		float *out = part == 0 ? ga.dv.dz_re : ga.dv.dz_im;
		out[col] = ga.accumulate ? out[col] + s : s;
		if (ga.dv.dzs_re) {
			float *m = part == 0 ? ga.dv.dzs_re : ga.dv.dzs_im;
			const float mv = part == 0 ? s : -s;
			m[col] = ga.accumulate ? m[col] + mv : mv;
		}
	}
}

SkinnyStrides skinny_strides(const CgemmArgs &args, bool a_mcontig, bool b_ncontig) {
	// elements from the first to one past the last of an operand plane
	const long span_a = a_mcontig ? (args.K - 1) * args.lda + args.M : (args.M - 1) * args.lda + args.K;
	const long span_b = b_ncontig ? (args.K - 1) * args.ldb + args.N : (args.N - 1) * args.ldb + args.K;
	return SkinnyStrides{a_mcontig ? (unsigned) args.lda : 1u, a_mcontig ? 1u : (unsigned) args.lda, b_ncontig ? (unsigned) args.ldb : 1u,
			b_ncontig ? 1u : (unsigned) args.ldb, (unsigned) (4 * span_a), (unsigned) (4 * span_b)};
}

template <int W, bool A_V4, bool B_V4>
int launch_skinny(const CgemmArgs &args, bool a_mcontig, bool b_ncontig, int nprob, int batch) {
	auto kern = cgemm_skinny_kernel<W, A_V4, B_V4>;
	hipLaunchKernelGGL(kern, dim3(args.tiles_m * args.tiles_n, nprob, batch * args.splits), dim3(64 * W), 0, cnet::rt().stream, args,
			skinny_strides(args, a_mcontig, b_ncontig));
	CNET_LAUNCH_CHECK();
	if (args.splits > 1) {
		dim3 rgrid((unsigned) ((2L * args.M * args.N + 255) / 256), nprob, batch);
		hipLaunchKernelGGL(splitk_reduce_kernel, rgrid, dim3(256), 0, cnet::rt().stream, args, nprob, batch);
		CNET_LAUNCH_CHECK();
	}
	return CNET_OK;
}

// the launch whose workgroups go on to the CrossEntropy of their rows of logits (CgemmArgs::ce_*; one column of tiles, no slices)
template <int W, bool A_V4, bool B_V4>
int launch_skinny_ce(const CgemmArgs &args, bool a_mcontig, bool b_ncontig) {
	auto kern = cgemm_skinny_kernel<W, A_V4, B_V4, true>;
	hipLaunchKernelGGL(kern, dim3(args.tiles_m * args.tiles_n, 1, 1), dim3(64 * W), 0, cnet::rt().stream, args, skinny_strides(args, a_mcontig, b_ncontig));
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

// Whether the product is small enough for cgemm_skinny_kernel; if so, `args` gets the tile counts and, for a long K,
// the number and length of the slices of K (the partial planes are allocated by try_skinny).
bool plan_skinny(bool a_mcontig, bool b_ncontig, const CgemmArgs &proto, int nprob, int batch, CgemmArgs &args) {
	static const bool enabled = [] {
		const char *e = getenv("CNET_CGEMM_SKINNY");  // tuning override: 0 sends every product to the block kernels
		return !e || atoi(e) != 0;
	}();
	if (!enabled || proto.tri || batch > 65535) return false;
	args = proto;
	args.tiles_m = (args.M + 15) / 16;
	args.tiles_n = (args.N + 15) / 16;
	const long tiles = (long) args.tiles_m * args.tiles_n * nprob * batch;
	// Measured against the block kernels with K cut (64 x 784 x 784: 9 against 15 us; 64 x 10 x 784: 8 against 12 us;
	// 10 x 784 x 64: 4 against 9 us; 256 x 784 x 784, 784 tiles: 19.5 against 23 us); with more than four tiles per
	// compute unit the block kernels have enough blocks of their own.
	static const long tile_limit = [] {
		const char *e = getenv("CNET_CGEMM_SKINNY_TILES");  // tuning override of the largest number of tiles
		return e ? atol(e) : 0L;
	}();
	const long cus = cnet::rt().prop.multiProcessorCount;
	const long most = tile_limit ? tile_limit : 4 * cus;
	if (tiles > most) return false;
	// the kernel addresses each operand plane with 32-bit byte offsets
	const long span_a = a_mcontig ? (args.K - 1) * args.lda + args.M : (args.M - 1) * args.lda + args.K;
	const long span_b = b_ncontig ? (args.K - 1) * args.ldb + args.N : (args.N - 1) * args.ldb + args.K;
	if (span_a >= (1L << 30) || span_b >= (1L << 30)) return false;
	args.splits = 1;
	args.chunks_per_split = 0;
	args.partial = nullptr;
	args.nprob = nprob;
	args.tail_tiles = args.tail_splits = args.tail_chunks = 0;
	if (args.K > 1024) {
		// A long K against a C of few tiles (the weight gradient of a narrow layer over a large batch): slices of K go to
		// workgroups of their own, at least 256 long and no more slices than give two workgroups to every compute unit;
		// the slices are added in order by splitk_reduce_kernel.
		const int groups = (args.K + 15) / 16;
		const long splits = std::min<long>(2 * cus / tiles, groups / 16);
		if (splits < 2 || (long) batch * splits > 65535) return false;
		args.chunks_per_split = (int) ((groups + splits - 1) / splits);
		if (args.chunks_per_split > 64) {
			// still longer than 1024 per slice: the block kernels do better, unless C is so small (the weight gradient of a
			// 784 -> 10 layer over a batch of 16384: 49 tiles) that they would run a handful of blocks; then slices of 1024,
			// several workgroups to a compute unit (16384 x 784 x 10: 90 -> 25 us)
			const long more = (groups + 63) / 64;
			if (2 * tiles > cus || more > 128 || (long) batch * more > 65535) return false;
			args.chunks_per_split = (int) ((groups + more - 1) / more);
		}
		args.splits = (groups + args.chunks_per_split - 1) / args.chunks_per_split;  // no empty slice
	}
	return true;
}

// expected duration in us of the launch planned by plan_skinny: about 3 us plus 7.5 ns per k of a slice (measured at up
// to two tiles per compute unit), plus the kernel that adds the slices
double skinny_us(const CgemmArgs &args, int nprob, int batch) {
	const long cus = cnet::rt().prop.multiProcessorCount;
	const long wgs = (long) args.tiles_m * args.tiles_n * nprob * batch * args.splits;
	const int k_slice = args.splits > 1 ? args.chunks_per_split * 16 : args.K;
	return (3.0 + 0.0075 * k_slice) * std::max(1.0, wgs / (2.0 * cus)) + (args.splits > 1 ? 6.0 : 0.0);
}

// which instantiation of cgemm_skinny_kernel a planned product takes: float4 loads along K per operand, wavefronts per tile
struct SkinnyVariant {
	bool a_v4, b_v4;
	int w;
	bool operator==(const SkinnyVariant &o) const { return a_v4 == o.a_v4 && b_v4 == o.b_v4 && w == o.w; }
};

SkinnyVariant skinny_variant(bool a_mcontig, bool b_ncontig, const CgemmArgs &args, int nprob, int batch) {
	SkinnyVariant v;
	v.a_v4 = !a_mcontig && args.lda % 4 == 0 && args.stride_a % 4 == 0 && args.K % 4 == 0;
	v.b_v4 = !b_ncontig && args.ldb % 4 == 0 && args.stride_b % 4 == 0 && args.K % 4 == 0;
	for (int q = 0; q < nprob; ++q) {
		v.a_v4 = v.a_v4 && cnet::aligned16(args.p[q].a_re) && cnet::aligned16(args.p[q].a_im);
		v.b_v4 = v.b_v4 && cnet::aligned16(args.p[q].b_re) && cnet::aligned16(args.p[q].b_im);
	}
	// Four wavefronts per tile, which leaves room for several tiles on a compute unit; eight (two per SIMD, each other's
	// latency cover) when there are so few tiles that most units hold one at most (64 x 784 x 784: 9.0 -> 8.5 us; with
	// three tiles per unit, 256 x 784 x 784: 19.8 -> 21.6 us, so not there).
	static const int forced_w = [] {
		const char *e = getenv("CNET_CGEMM_SKINNY_W");  // tuning override: 4, 8 or 16 wavefronts per tile
		return e ? atoi(e) : 0;
	}();
	const long wgs = (long) args.tiles_m * args.tiles_n * nprob * batch * args.splits;
	v.w = forced_w == 4 || forced_w == 8 || forced_w == 16 ? forced_w
			: (args.splits == 1 && 2 * wgs <= 3 * cnet::rt().prop.multiProcessorCount && args.K >= 256) ? 8 : 4;
	return v;
}

// expands to CALL<W, A_V4, B_V4> ARGS for the variant v
#define CNET_SKINNY_PICK(v, CALL, ARGS)                                                                                          \
	((v).w == 16 ? CNET_SKINNY_PICK_W(v, 16, CALL, ARGS) : (v).w == 8 ? CNET_SKINNY_PICK_W(v, 8, CALL, ARGS) : CNET_SKINNY_PICK_W(v, 4, CALL, ARGS))
#define CNET_SKINNY_PICK_W(v, W, CALL, ARGS)                                                                                     \
	((v).a_v4 ? ((v).b_v4 ? CALL<W, true, true> ARGS : CALL<W, true, false> ARGS)                                                \
			  : ((v).b_v4 ? CALL<W, false, true> ARGS : CALL<W, false, false> ARGS))

// true and *rc set when the product was small enough for cgemm_skinny_kernel
bool try_skinny(bool a_mcontig, bool b_ncontig, const CgemmArgs &proto, int nprob, int batch, int *rc) {
	CgemmArgs args;
	if (!plan_skinny(a_mcontig, b_ncontig, proto, nprob, batch, args)) return false;
	if (args.splits > 1) {
		args.partial = (float *) cnet::workspace((size_t) args.splits * nprob * batch * 2 * args.M * args.N * sizeof(float));
		if (!args.partial) {
			*rc = CNET_ERR_OUT_OF_MEMORY;
			return true;
		}
	}
	const SkinnyVariant v = skinny_variant(a_mcontig, b_ncontig, args, nprob, batch);
	*rc = CNET_SKINNY_PICK(v, launch_skinny, (args, a_mcontig, b_ncontig, nprob, batch));
	return true;
}

template <int W, bool A_V4, bool B_V4>
int launch_skinny_two(const CgemmArgs &args0, const SkinnyStrides &st0, const CgemmArgs &args1, const SkinnyStrides &st1, int nprob) {
	const int tiles0 = args0.tiles_m * args0.tiles_n, tiles1 = args1.tiles_m * args1.tiles_n;
	auto kern = cgemm_skinny_two_kernel<W, A_V4, B_V4>;
	hipLaunchKernelGGL(kern, dim3(tiles0 + tiles1, nprob, 1), dim3(64 * W), 0, cnet::rt().stream, args0, st0, tiles0, args1, st1);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

// Whether two products are both small enough for cgemm_skinny_kernel, neither cut along K, and take the same
// instantiation `v` of it, so that they can go out as one launch.
bool plan_skinny_two(bool a_mcontig0, bool b_ncontig0, const CgemmArgs &proto0, bool a_mcontig1, bool b_ncontig1, const CgemmArgs &proto1,
		int nprob, CgemmArgs &args0, CgemmArgs &args1, SkinnyVariant &v) {
	static const bool enabled = [] {
		const char *e = getenv("CNET_CGEMM_SKINNY_TWO");  // tuning override: 0 launches the two products one after the other
		return !e || atoi(e) != 0;
	}();
	if (!enabled || proto0.M <= 0 || proto0.N <= 0 || proto0.K <= 0 || proto1.M <= 0 || proto1.N <= 0 || proto1.K <= 0) return false;
	if (!plan_skinny(a_mcontig0, b_ncontig0, proto0, nprob, 1, args0) || !plan_skinny(a_mcontig1, b_ncontig1, proto1, nprob, 1, args1))
		return false;
	if (args0.splits != 1 || args1.splits != 1) return false;
	// together they must still be a small launch
	if (((long) args0.tiles_m * args0.tiles_n + (long) args1.tiles_m * args1.tiles_n) * nprob > 4L * cnet::rt().prop.multiProcessorCount)
		return false;
	v = skinny_variant(a_mcontig0, b_ncontig0, args0, nprob, 1);
	return v == skinny_variant(a_mcontig1, b_ncontig1, args1, nprob, 1);
}

// Two such products as one launch: true and *rc set.  Otherwise nothing is launched.
bool try_skinny_two(bool a_mcontig0, bool b_ncontig0, const CgemmArgs &proto0, bool a_mcontig1, bool b_ncontig1, const CgemmArgs &proto1,
		int nprob, int *rc) {
	CgemmArgs args0, args1;
	SkinnyVariant v0;
	if (!plan_skinny_two(a_mcontig0, b_ncontig0, proto0, a_mcontig1, b_ncontig1, proto1, nprob, args0, args1, v0)) return false;
	const SkinnyStrides st0 = skinny_strides(args0, a_mcontig0, b_ncontig0), st1 = skinny_strides(args1, a_mcontig1, b_ncontig1);
	*rc = CNET_SKINNY_PICK(v0, launch_skinny_two, (args0, st0, args1, st1, nprob));
	return true;
}

template <int W, bool A_V4, bool B_V4>
int launch_skinny_gate_bwd(const CgemmArgs &args0, const SkinnyStrides &st0, const CgemmArgs &args1, const SkinnyStrides &st1,
		const cnet::GateBwd &gate) {
	auto kern = cgemm_skinny_gate_bwd_kernel<W, A_V4, B_V4>;
	hipLaunchKernelGGL(kern, dim3(args0.tiles_n + args1.tiles_m * args1.tiles_n, 1, 1), dim3(64 * W), 0, cnet::rt().stream, args0, st0, args1, st1,
			gate);
	CNET_LAUNCH_CHECK();
	return CNET_OK;
}

// tail_splits >= 2: cut the blocks of the last, partly filled round into that many pieces along K (see CgemmArgs)
// Whether the block kernels of one or two tiles per wavefront form a complex product from three real ones
// (cgemm_fast_kernel<.., GAUSS>); the cost model then prices those shapes at three quarters of their matrix work.
int g_three_products = -1;
inline bool three_products() {
	if (g_three_products < 0) {
		const char *e = getenv("CNET_CGEMM_3M");
		g_three_products = e ? (atoi(e) != 0) : 0;
	}
	return g_three_products != 0;
}

// The block kernels ask for more dynamic LDS than the default limit, which takes one hipFuncSetAttribute per instantiation.
// launch() makes that call at the first launch of each; a first launch inside a stream capture would make it while the capture
// is open, so cnet_graph_begin has all of them made beforehand (cgemm_prime_attributes) and launch() skips its own.
bool g_attrs_primed = false;

// STAGES: LDS stages of the fast kernel; 0 = three, two for the 128 x 128 block (whose two stages fill the LDS of two
// workgroups per compute unit).  The 64 x 64 block also runs with two: four workgroups to a unit instead of three.
template <int BM, int BN, int STAGES>
constexpr int fast_stages() {
	return STAGES ? STAGES : (BM == 128 && BN == 128) ? 2 : 3;
}

template <int BM, int BN, int WM, int WN, bool A_MCONTIG, bool B_NCONTIG, int VEC, int STAGES = 0>
hipError_t prime_attributes() {
	constexpr size_t smem = 2 * (size_t) (2 * KC * (BM + 4) + 2 * KC * (BN + 4)) * sizeof(float);
	hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, VEC>),
			hipFuncAttributeMaxDynamicSharedMemorySize, (int) smem);
	if constexpr (VEC == 4) {
		constexpr int NST = fast_stages<BM, BN, STAGES>();
		constexpr size_t fast_smem = (size_t) NST * 2 * KC * (BM + BN) * sizeof(float);
		if (e == hipSuccess)
			e = hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST>),
					hipFuncAttributeMaxDynamicSharedMemorySize, (int) fast_smem);
		if constexpr (!A_MCONTIG && B_NCONTIG) {
			if (e == hipSuccess)
				e = hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, false, true>),
						hipFuncAttributeMaxDynamicSharedMemorySize, (int) fast_smem);
			if (e == hipSuccess)
				e = hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, true, true>),
						hipFuncAttributeMaxDynamicSharedMemorySize, (int) fast_smem);
		}
		if constexpr ((WM / 32) * (WN / 32) <= 2 || A_MCONTIG || B_NCONTIG) {
			if (e == hipSuccess)
				e = hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, true>),
						hipFuncAttributeMaxDynamicSharedMemorySize, (int) fast_smem);
		}
	}
	return e;
}

// (the shapes pick_tile can choose: the scalar-load fallback keeps to the small block)
template <bool A_MCONTIG, bool B_NCONTIG, int VEC>
hipError_t prime_shapes() {
	hipError_t e = prime_attributes<64, 64, 32, 32, A_MCONTIG, B_NCONTIG, VEC>();
	if constexpr (VEC == 4) {
		if (e == hipSuccess) e = prime_attributes<128, 128, 64, 64, A_MCONTIG, B_NCONTIG, VEC>();
		if (e == hipSuccess) e = prime_attributes<64, 128, 32, 64, A_MCONTIG, B_NCONTIG, VEC>();
		if (e == hipSuccess) e = prime_attributes<128, 64, 64, 32, A_MCONTIG, B_NCONTIG, VEC>();
		if (e == hipSuccess) e = prime_attributes<64, 64, 32, 32, A_MCONTIG, B_NCONTIG, VEC, 2>();
	}
	return e;
}

template <int BM, int BN, int WM, int WN, bool A_MCONTIG, bool B_NCONTIG, int VEC, int STAGES = 0>
int launch(const CgemmArgs &proto, int nprob, int batch, int tail_splits = 0, int k_cuts = -1) {
	CgemmArgs args = proto;
	args.tiles_m = (args.M + BM - 1) / BM;
	args.tiles_n = (args.N + BN - 1) / BN;
	args.nprob = nprob;
	args.tail_tiles = args.tail_splits = args.tail_chunks = 0;
	constexpr size_t smem = 2 * (size_t) (2 * KC * (BM + 4) + 2 * KC * (BN + 4)) * sizeof(float);
	// A grid that leaves most compute units idle while each workgroup walks a long K (a small batch against a long
	// reduction: every chunk then waits a full memory latency) is cut along K.
	args.splits = 1;
	args.chunks_per_split = 0;
	args.partial = nullptr;
	{
		const long blocks = (long) args.tiles_m * args.tiles_n * nprob * batch;
		const long cus = cnet::rt().prop.multiProcessorCount;
		const int nchunks = (args.K + KC - 1) / KC;
		int splits = k_cuts;  // from the cost model; -1: the rule for the kernels it does not cover
		if (k_cuts < 0) {
			splits = 1;
			if (!args.tri && blocks * 2 <= cus && nchunks >= 8 && (long) batch * (cus / blocks) <= 65535)
				splits = (int) std::min<long>(cus / blocks, nchunks / 4);
		}
		if (splits >= 2) {
			args.chunks_per_split = (nchunks + splits - 1) / splits;
			args.splits = (nchunks + args.chunks_per_split - 1) / args.chunks_per_split;  // no empty split
			const size_t bytes = (size_t) args.splits * nprob * batch * 2 * args.M * args.N * sizeof(float);
			args.partial = (float *) cnet::workspace(bytes);
			if (!args.partial) return CNET_ERR_OUT_OF_MEMORY;
		}
	}
	dim3 grid(args.tiles_m * grid_tiles_n(args), nprob, batch * args.splits);
	// The fast kernel addresses a lane's 16 bytes inside the operand tile of a chunk with an unsigned 32-bit byte offset:
	// (row * ld + k) * 4 for rows < min(block edge, rows of the operand), or (k * ld + row) * 4 for k < KC.  A leading
	// dimension beyond that (8.4 M floats for a K-contiguous operand under a 128-row block) goes to cgemm_kernel, whose
	// offsets are 64-bit.
	auto offsets_fit = [](long ld, bool rows_contig, int block_rows, int rows) {
		const long last = rows_contig ? (long) (KC - 1) * ld + block_rows : (long) (std::min(block_rows, rows) - 1) * ld + KC;
		return last * 4 < (1L << 32);
	};
	const bool fast_ok = VEC == 4 && args.K % KC == 0 && offsets_fit(args.lda, A_MCONTIG, BM, args.M) &&
			offsets_fit(args.ldb, B_NCONTIG, BN, args.N);
	if (tail_splits >= 2 && fast_ok && !args.tri && batch == 1 && args.splits == 1) {
		const long cus = cnet::rt().prop.multiProcessorCount;
		const long all = (long) args.tiles_m * args.tiles_n * nprob;
		const int nchunks = args.K / KC;
		const int r = (int) (all % cus);
		if (all > cus && r > 0 && (long) r * tail_splits <= all - r) {
			args.tail_chunks = (nchunks + tail_splits - 1) / tail_splits;
			args.tail_splits = (nchunks + args.tail_chunks - 1) / args.tail_chunks;  // no empty piece
			args.tail_tiles = r;
			args.partial = (float *) cnet::workspace((size_t) r * args.tail_splits * 2 * BM * BN * sizeof(float));
			if (!args.partial) return CNET_ERR_OUT_OF_MEMORY;
			grid = dim3((unsigned) (all - r), 1, 1);  // one workgroup per full block; the first r x s also do a piece
		}
	}
	auto finish = [&]() -> int {
		if (args.tail_tiles) {
			hipLaunchKernelGGL((tail_reduce_kernel<BM, BN>), dim3(args.tail_tiles, 2 * BM * BN / 1024), dim3(256), 0, cnet::rt().stream, args);
			CNET_LAUNCH_CHECK();
		}
		if (args.splits > 1) {
			dim3 rgrid((unsigned) ((2L * args.M * args.N + 255) / 256), nprob, batch);
			hipLaunchKernelGGL(splitk_reduce_kernel, rgrid, dim3(256), 0, cnet::rt().stream, args, nprob, batch);
			CNET_LAUNCH_CHECK();
		}
		return CNET_OK;
	};
	if constexpr (VEC == 4) {
		if (fast_ok) {  // any M and N: edge blocks re-read the last valid rows and store only what is inside C
			constexpr int NST = fast_stages<BM, BN, STAGES>();
			constexpr size_t fast_smem = (size_t) NST * 2 * KC * (BM + BN) * sizeof(float);
			if constexpr (!A_MCONTIG && B_NCONTIG) {
				if (args.a_real == 2) {
					static bool fold_attr_set = false;
					if (!fold_attr_set && !g_attrs_primed) {
						CNET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, true, true>),
								hipFuncAttributeMaxDynamicSharedMemorySize, (int) fast_smem));
						fold_attr_set = true;
					}
					hipLaunchKernelGGL((cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, true, true>), grid, dim3(NTHREADS), fast_smem,
							cnet::rt().stream, args);
					CNET_LAUNCH_CHECK();
					return finish();
				}
				if (args.a_real) {
					static bool real_attr_set = false;
					if (!real_attr_set && !g_attrs_primed) {
						CNET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, false, true>),
								hipFuncAttributeMaxDynamicSharedMemorySize, (int) fast_smem));
						real_attr_set = true;
					}
					hipLaunchKernelGGL((cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, false, true>), grid, dim3(NTHREADS), fast_smem,
							cnet::rt().stream, args);
					CNET_LAUNCH_CHECK();
					return finish();
				}
			}
			// Three accumulator sets of four tiles (192 registers) leave too few for the fragments of two k-contiguous
			// operands (float4 each): that one layout of the 128 x 128 block spills and keeps four products.
			if constexpr ((WM / 32) * (WN / 32) <= 2 || A_MCONTIG || B_NCONTIG) {
				if (three_products()) {
					static bool gauss_attr_set = false;
					if (!gauss_attr_set && !g_attrs_primed) {
						CNET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, true>),
								hipFuncAttributeMaxDynamicSharedMemorySize, (int) fast_smem));
						gauss_attr_set = true;
					}
					hipLaunchKernelGGL((cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST, true>), grid, dim3(NTHREADS), fast_smem,
							cnet::rt().stream, args);
					CNET_LAUNCH_CHECK();
					return finish();
				}
			}
			static bool fast_attr_set = false;
			if (!fast_attr_set && !g_attrs_primed) {
				CNET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST>),
						hipFuncAttributeMaxDynamicSharedMemorySize, (int) fast_smem));
				fast_attr_set = true;
			}
			hipLaunchKernelGGL((cgemm_fast_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, NST>), grid, dim3(NTHREADS), fast_smem,
					cnet::rt().stream, args);
			CNET_LAUNCH_CHECK();
			return finish();
		}
	}
	if (args.a_real == 2) return cnet::fail(CNET_ERR_UNSUPPORTED, "cgemm: the folded form of a real operand has block kernels for aligned operands only");
	auto kern = cgemm_kernel<BM, BN, WM, WN, A_MCONTIG, B_NCONTIG, VEC>;
	static bool attr_set = false;  // per instantiation
	if (!attr_set && !g_attrs_primed) {
		CNET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
				(int) smem));
		attr_set = true;
	}
	hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), smem, cnet::rt().stream, args);
	CNET_LAUNCH_CHECK();
	return finish();
}

// Block shape for the fast kernel (0: 128 x 128, 1: 64 x 128, 2: 128 x 64, 3: 64 x 64, 4: 64 x 64 with two LDS stages), whether the blocks of a partly
// filled last round are cut along K (*tail = number of pieces, 0 = no), and the expected duration of the launch in us.
// layout (block_layout): 0 = A row-major and B k-major, 1 = both operands with k contiguous (the one layout whose
// 128 x 128 kernel has no three-product form), 2 = both with their rows contiguous (and the fourth combination).
inline int block_layout(bool a_mcontig, bool b_ncontig) {
	return (!a_mcontig && b_ncontig) ? 0 : (!a_mcontig && !b_ncontig) ? 1 : 2;
}
double plan_blocks(const CgemmArgs &a, int nprob, int batch, int layout, int *shape, int *tail_pieces, int *k_cuts) {
	const long cus = cnet::rt().prop.multiProcessorCount;
	auto blocks = [&](int bm, int bn) {
		long tn = (a.N + bn - 1) / bn;
		if (a.tri) tn = (tn + 1) / 2;  // one workgroup per mirrored pair of column blocks
		return (long) ((a.M + bm - 1) / bm) * tn * nprob * batch;
	};
	// tuning override: CNET_CGEMM_TILE = 0 (128x128), 1 (64x128), 2 (128x64), 3 (64x64), 4 (64x64, two LDS stages)
	static const int forced = [] {
		const char *e = getenv("CNET_CGEMM_TILE");
		return e ? atoi(e) : -1;
	}();
	// CNET_CGEMM_TAIL = 0 / 1: never / whenever possible cut the blocks of a partly filled last round along K
	static const int forced_tail = [] {
		const char *e = getenv("CNET_CGEMM_TAIL");
		return e ? atoi(e) : -1;
	}();
	// Expected duration of the launch with each block shape.  The busiest compute unit works through p = ceil(blocks /
	// units) blocks, so the launch takes p block-times, whether or not all units have that many and whether or not a
	// block on the edge of C is full, divided by the efficiency measured for the shape at p blocks per unit on full
	// blocks (fraction of the fp32 MFMA peak on operands of random values, a set of tables per operand layout), at K = 512,
	// 1024 and 2048; in between and below, 1 / efficiency follows a broken line in 1 / K (a
	// loop part and a fixed part per block: first loads and the write-out of C weigh more on a short K, and more on the
	// small shapes).  The tables carry what a formula would miss: a unit holds two workgroups of the larger shapes, three
	// of 64 x 64 and four of 64 x 64 with two LDS stages, a lone workgroup cannot keep the matrix pipe busy, and with 3 or 5
	// blocks of 128 x 128 per unit, 4 of 64 x 64 or 5 of its two-stage form, the hardware dispatcher leaves some units with
	// one block more than the others.
	// Alternative for a partly filled last round (q full rounds, r blocks left over): cut those r blocks into s pieces
	// along K, one piece for each workgroup of the full rounds.  Then the launch takes q block-times plus 1/s of one,
	// plus the fixed cost of a short piece and of the kernel that adds the pieces.
	struct Shape {
		int bm, bn;
		// [layout: 0 A row-major and B k-major, 1 both K-contiguous, 2 both with their rows contiguous][K = 512, 1024, 2048]
		// [p = 1 .. 8 (8 stands for everything above)], operands of random values
		float eff[3][3][8];
	};
	static const Shape shapes[5] = {
			{128, 128,
					{{{0.808f, 0.897f, 0.686f, 0.903f, 0.760f, 0.902f, 0.796f, 0.905f},
							{0.848f, 0.922f, 0.702f, 0.925f, 0.778f, 0.923f, 0.814f, 0.924f},
							{0.873f, 0.936f, 0.707f, 0.934f, 0.782f, 0.937f, 0.822f, 0.936f}},
					{{0.821f, 0.899f, 0.689f, 0.907f, 0.763f, 0.908f, 0.806f, 0.909f},
							{0.864f, 0.928f, 0.912f, 0.932f, 0.921f, 0.931f, 0.901f, 0.930f},
							{0.892f, 0.943f, 0.933f, 0.946f, 0.939f, 0.947f, 0.944f, 0.947f}},
					{{0.815f, 0.897f, 0.686f, 0.906f, 0.763f, 0.907f, 0.799f, 0.908f},
							{0.856f, 0.927f, 0.702f, 0.929f, 0.783f, 0.929f, 0.819f, 0.931f},
							{0.881f, 0.943f, 0.710f, 0.944f, 0.791f, 0.945f, 0.828f, 0.946f}}}},
			{64, 128,
					{{{0.775f, 0.864f, 0.857f, 0.879f, 0.873f, 0.883f, 0.881f, 0.887f},
							{0.842f, 0.904f, 0.897f, 0.912f, 0.909f, 0.915f, 0.913f, 0.917f},
							{0.875f, 0.924f, 0.917f, 0.929f, 0.927f, 0.931f, 0.930f, 0.933f}},
					{{0.794f, 0.858f, 0.867f, 0.879f, 0.879f, 0.886f, 0.887f, 0.891f},
							{0.865f, 0.903f, 0.910f, 0.915f, 0.918f, 0.920f, 0.921f, 0.922f},
							{0.903f, 0.930f, 0.936f, 0.940f, 0.942f, 0.943f, 0.944f, 0.945f}},
					{{0.780f, 0.870f, 0.865f, 0.884f, 0.879f, 0.888f, 0.887f, 0.891f},
							{0.846f, 0.907f, 0.904f, 0.917f, 0.915f, 0.920f, 0.920f, 0.922f},
							{0.879f, 0.931f, 0.927f, 0.936f, 0.936f, 0.938f, 0.939f, 0.940f}}}},
			{128, 64,
					{{{0.792f, 0.862f, 0.866f, 0.881f, 0.879f, 0.885f, 0.884f, 0.888f},
							{0.857f, 0.906f, 0.913f, 0.918f, 0.921f, 0.921f, 0.921f, 0.921f},
							{0.894f, 0.932f, 0.937f, 0.939f, 0.939f, 0.942f, 0.941f, 0.943f}},
					{{0.795f, 0.859f, 0.863f, 0.878f, 0.876f, 0.883f, 0.882f, 0.887f},
							{0.862f, 0.903f, 0.911f, 0.916f, 0.918f, 0.918f, 0.918f, 0.919f},
							{0.898f, 0.928f, 0.935f, 0.939f, 0.941f, 0.943f, 0.942f, 0.942f}},
					{{0.781f, 0.865f, 0.861f, 0.880f, 0.877f, 0.883f, 0.882f, 0.885f},
							{0.846f, 0.906f, 0.902f, 0.917f, 0.913f, 0.917f, 0.917f, 0.918f},
							{0.881f, 0.927f, 0.923f, 0.932f, 0.932f, 0.936f, 0.936f, 0.936f}}}},
			{64, 64,
					{{{0.756f, 0.833f, 0.868f, 0.713f, 0.880f, 0.887f, 0.888f, 0.894f},
							{0.835f, 0.891f, 0.914f, 0.743f, 0.923f, 0.925f, 0.925f, 0.926f},
							{0.880f, 0.919f, 0.936f, 0.758f, 0.942f, 0.942f, 0.946f, 0.949f}},
					{{0.764f, 0.831f, 0.867f, 0.711f, 0.880f, 0.884f, 0.886f, 0.888f},
							{0.850f, 0.894f, 0.913f, 0.744f, 0.923f, 0.921f, 0.924f, 0.923f},
							{0.899f, 0.929f, 0.941f, 0.761f, 0.945f, 0.946f, 0.947f, 0.950f}},
					{{0.752f, 0.829f, 0.866f, 0.712f, 0.880f, 0.886f, 0.888f, 0.891f},
							{0.834f, 0.886f, 0.912f, 0.744f, 0.921f, 0.921f, 0.925f, 0.928f},
							{0.878f, 0.921f, 0.934f, 0.761f, 0.943f, 0.945f, 0.949f, 0.948f}}}},
			{64, 64,
					{{{0.767f, 0.843f, 0.873f, 0.889f, 0.756f, 0.902f, 0.905f, 0.909f},
							{0.846f, 0.899f, 0.917f, 0.924f, 0.785f, 0.933f, 0.935f, 0.934f},
							{0.890f, 0.926f, 0.939f, 0.944f, 0.798f, 0.950f, 0.951f, 0.948f}},
					{{0.770f, 0.845f, 0.866f, 0.888f, 0.754f, 0.894f, 0.896f, 0.873f},
							{0.852f, 0.900f, 0.915f, 0.924f, 0.784f, 0.928f, 0.934f, 0.875f},
							{0.901f, 0.929f, 0.939f, 0.948f, 0.798f, 0.939f, 0.951f, 0.888f}},
					{{0.754f, 0.839f, 0.870f, 0.886f, 0.754f, 0.900f, 0.904f, 0.904f},
							{0.834f, 0.894f, 0.914f, 0.923f, 0.784f, 0.930f, 0.933f, 0.932f},
							{0.878f, 0.921f, 0.934f, 0.944f, 0.797f, 0.951f, 0.951f, 0.950f}}}}};
	// what a very long K adds to the K = 2048 figures (8192 x 1024 of C, K up to 32768: 1 / efficiency stays linear in 1 / K)
	static const float long_k_gain[5][3] = {{0.007f, 0.016f, 0.019f}, {0.018f, 0.032f, 0.027f}, {0.030f, 0.027f, 0.032f},
			{0.021f, 0.025f, 0.024f}, {0.021f, 0.025f, 0.024f}};
	static const bool k_dependent = [] {
		const char *e = getenv("CNET_CGEMM_KMODEL");  // tuning override: 0 uses the K = 2048 table for every K
		return !e || atoi(e) != 0;
	}();
	auto eff = [&](int k, long p, int K) {
		const int i = p < 8 ? (int) p - 1 : 7;
		const float(*t)[8] = shapes[k].eff[layout];
		if (!k_dependent) return (double) t[2][i];
		// 1 / efficiency as a broken line in 1 / K through the three tables; the piece between 512 and 1024 also serves below
		// 512; beyond K = 2048 the line runs on to the figure for an endless K (long_k_gain)
		const double inv512 = 1.0 / t[0][i], inv1024 = 1.0 / t[1][i], inv2048 = 1.0 / t[2][i], x = 1.0 / K;
		double e;
		if (x <= 1.0 / 2048)
			e = (1.0 + long_k_gain[k][layout] * (1.0 - 2048.0 * x)) / inv2048;
		else if (x <= 1.0 / 1024)
			e = 1.0 / (inv2048 + (inv1024 - inv2048) * (x - 1.0 / 2048) / (1.0 / 1024 - 1.0 / 2048));
		else
			e = 1.0 / (inv1024 + (inv512 - inv1024) * (x - 1.0 / 1024) / (1.0 / 512 - 1.0 / 1024));
		// A row-major A against a k-major B with rows of A beyond 4096 values: the 64 x 64 blocks lose 1.9 % per doubling of K
		// (8192 x 1024 of C: .960 at K = 4096, .941, .925, .904 at 32768, where the larger shapes hold .95 - .97)
		if (layout == 0 && shapes[k].bm == 64 && shapes[k].bn == 64 && K > 4096) e *= 1.0 - 0.019 * std::log2(K / 4096.0);
		return e;
	};
	// 256 flop per clock and compute unit at the device's engine clock (kHz -> cycles per microsecond), as cnet_get_device_info
	// reports it; 2.4 GHz when the driver gives none
	const int khz = cnet::rt().prop.clockRate;
	const double flop_per_us_per_unit = 256.0 * (khz > 0 ? khz * 1e-3 : 2.4e3);
	const int nchunks = (a.K + KC - 1) / KC;
	const bool tail_possible = forced_tail != 0 && a.K % KC == 0 && !a.tri && batch == 1;
	int best = 3, best_tail = 0, best_cuts = 1;
	double best_us = 1e30;
	for (int k = 0; k < 5; ++k) {
		if (forced >= 0 && forced != k) continue;
		if (k == 4 && (forced != 4 && a.K % KC != 0)) continue;  // only the fast kernel has the two-stage form: shape 3 there
		// beyond seven blocks per unit the two-stage form is erratic on a long K (8192 x 1024 of C: .95 at K = 2048, .83 - .97
		// from 4096 on, layout by layout)
		if (k == 4 && forced != 4 && a.K > 2048 && blocks(64, 64) > 7 * cus) continue;
		const long nb = blocks(shapes[k].bm, shapes[k].bn);
		const long per_unit = (nb + cus - 1) / cus;
		// three real products per complex one in the shapes that have the registers for it (fast kernel only: K in whole chunks)
		// an A without imaginary parts: two real products (fast kernel only: K in whole chunks)
		const double work = (a.a_real && a.K % KC == 0) ? 4.0 : (three_products() && a.K % KC == 0 && !(k == 0 && layout == 1)) ? 6.0 : 8.0;
		const double block_us = work * shapes[k].bm * shapes[k].bn * a.K / flop_per_us_per_unit;
		// between shapes that are equally fast the larger block wins: it moves half as many operand bytes through L2
		const double bonus = 1.0 - 0.00000025 * shapes[k].bm * shapes[k].bn;
		double us = per_unit * block_us / eff(k, per_unit, a.K) * bonus;
		int tail = 0, cuts = 1;
		const long q = nb / cus, r = nb % cus;
		if (tail_possible && q >= 1 && r > 0) {
			// as many pieces as there are workgroups in the full rounds, so that each of them gets one; a piece is at
			// least three chunks long
			const int s = (int) std::min<long>(q * cus / r, nchunks / 3);
			if (s >= 2) {
				const double tail_us = (q * block_us / eff(k, q, a.K) + block_us / s / 0.8 + 20.0) * bonus;
				if (tail_us < us || forced_tail == 1) {
					us = tail_us;
					tail = s;
				}
			}
		}
		// A short grid (fewer than two blocks per unit: idle units, or lone workgroups that cannot fill the matrix pipe)
		// against a long K: every block is cut into s slices along K that run as workgroups of their own and are added
		// in order by splitk_reduce_kernel.  Costs the shorter K per slice (lower efficiency) and the pass over the
		// partial planes (written and read once, C written, at about 4 TB/s).
		static const bool plan_cuts = [] {
			const char *e = getenv("CNET_CGEMM_KCUT");  // tuning override: 0 cuts K only when half of the units would idle
			return !e || atoi(e) != 0;
		}();
		if (!a.tri && nb < 2 * cus && nchunks >= 8 && (plan_cuts || nb * 2 <= cus)) {
			const long few = nb * 2 <= cus ? std::min<long>(cus / nb, nchunks / 4) : 0;  // one slice-workgroup per unit
			for (long s : {2L, 3L, 4L, 6L, 8L, few}) {
				if (s < 2 || nchunks / s < 4 || (long) batch * s > 65535) continue;
				const int k_slice = (int) ((nchunks + s - 1) / s) * KC;
				const long p = (nb * s + cus - 1) / cus;
				const double slice_us = work * shapes[k].bm * shapes[k].bn * k_slice / flop_per_us_per_unit;
				const double pass_us = 6.0 + (s + 1.0 + (a.accumulate ? 1.0 : 0.0)) * 8.0 * a.M * a.N * nprob * batch / 4.0e6;
				const double cut_us = p * slice_us / eff(k, p, k_slice) * bonus + pass_us;
				if (cut_us < us) {
					us = cut_us;
					cuts = (int) s;
					tail = 0;
				}
			}
		}
		if (us < best_us) {
			best_us = us;
			best = k;
			best_tail = tail;
			best_cuts = cuts;
		}
	}
	*shape = best;
	*tail_pieces = best_tail;
	*k_cuts = best_cuts;
	return best_us + 12.0;  // launch, first loads and the write-out of C
}

template <bool A_MCONTIG, bool B_NCONTIG, int VEC>
int pick_tile(const CgemmArgs &a, int nprob, int batch) {
	// the scalar-load fallback (odd shapes) keeps to the small block: its address arithmetic would spill otherwise
	if constexpr (VEC == 1) {
		return launch<64, 64, 32, 32, A_MCONTIG, B_NCONTIG, VEC>(a, nprob, batch);
	} else {
		int best, best_tail, cuts;
		plan_blocks(a, nprob, batch, block_layout(A_MCONTIG, B_NCONTIG), &best, &best_tail, &cuts);
		if (best == 0) return launch<128, 128, 64, 64, A_MCONTIG, B_NCONTIG, VEC>(a, nprob, batch, best_tail, cuts);
		if (best == 1) return launch<64, 128, 32, 64, A_MCONTIG, B_NCONTIG, VEC>(a, nprob, batch, best_tail, cuts);
		if (best == 2) return launch<128, 64, 64, 32, A_MCONTIG, B_NCONTIG, VEC>(a, nprob, batch, best_tail, cuts);
		if (best == 4) return launch<64, 64, 32, 32, A_MCONTIG, B_NCONTIG, VEC, 2>(a, nprob, batch, best_tail, cuts);
		return launch<64, 64, 32, 32, A_MCONTIG, B_NCONTIG, VEC>(a, nprob, batch, best_tail, cuts);
	}
}

}  // namespace

namespace {

// dst[plane][r][c] = src_plane[r][c] inside rows x cols and zero outside, for the two planes (blockIdx.y) of an operand;
// dst has rows_d rows of ldd floats per plane, ldd a multiple of four.  One thread per four columns of dst.
__global__ __launch_bounds__(256) void pack_planes_kernel(const float *__restrict__ s_re, const float *__restrict__ s_im, long lds, int rows,
		int cols, float *__restrict__ dst, int rows_d, int ldd) {
	const int groups = ldd / 4;
	const long idx = (long) blockIdx.x * 256 + threadIdx.x;
	if (idx >= (long) rows_d * groups) return;
	const int r = (int) (idx / groups), c0 = (int) (idx - (long) r * groups) * 4;
	const float *s = (blockIdx.y ? s_im : s_re) + (long) r * lds;
	float v[4] = {0.f, 0.f, 0.f, 0.f};
	if (r < rows) {
#pragma unroll
		for (int k = 0; k < 4; ++k)
			if (c0 + k < cols) v[k] = s[c0 + k];
	}
	*reinterpret_cast<float4 *>(dst + ((long) blockIdx.y * rows_d + r) * ldd + c0) = make_float4(v[0], v[1], v[2], v[3]);
}

}  // namespace

namespace cnet {

static int cgemm_dispatch(bool a_mcontig, bool b_ncontig, CgemmArgs &a, int nprob, int batch);

// Operands that the 128-bit transfers of the fast kernel cannot take (a leading dimension that is no multiple of four, a
// plane that does not start on 16 bytes): a large product first copies them into aligned planes of the library's operand
// buffer, K padded with zeros to whole chunks, and runs on those (2048^3 with every plane one float off its alignment:
// 0.67 -> 0.49 ms; the register-staged kernel that takes such operands directly runs at 102-106 TFLOP/s).  True when the
// product has been handed on that way (*rc set); false when it is not such a product or the buffer cannot be had.
static bool cgemm_packed(bool a_mcontig, bool b_ncontig, const CgemmArgs &a, int nprob, int batch, int *rc) {
	static const bool enabled = [] {
		const char *e = getenv("CNET_CGEMM_PACK");  // tuning override: 0 leaves misaligned operands to the register-staged kernel
		return !e || atoi(e) != 0;
	}();
	if (!enabled || batch != 1 || a.tri || a.a_real == 2) return false;
	auto misaligned = [&](const float *re, const float *im, long ld) { return ld % 4 != 0 || !aligned16(re) || !aligned16(im); };
	bool any = false;
	for (int q = 0; q < nprob; ++q)
		any = any || misaligned(a.p[q].a_re, a.p[q].a_im, a.lda) || misaligned(a.p[q].b_re, a.p[q].b_im, a.ldb);
	if (!any) return false;
	if ((double) a.M * a.N * a.K < (double) (1L << 27) || (long) a.M * a.N < 256L * 256) return false;
	const int kp = (a.K + KC - 1) / KC * KC;
	// (a run along M or N is padded to a multiple of four floats; the product itself keeps its M and N)
	const int a_rows = a_mcontig ? kp : a.M, a_ld = a_mcontig ? (a.M + 3) / 4 * 4 : kp;
	const int b_rows = b_ncontig ? kp : a.N, b_ld = b_ncontig ? (a.N + 3) / 4 * 4 : kp;
	const size_t a_floats = 2 * (size_t) a_rows * a_ld, b_floats = 2 * (size_t) b_rows * b_ld;
	// the distinct operands of the one or two problems (a pair of gradients shares one of them)
	const bool same_a = nprob == 2 && a.p[0].a_re == a.p[1].a_re && a.p[0].a_im == a.p[1].a_im;
	const bool same_b = nprob == 2 && a.p[0].b_re == a.p[1].b_re && a.p[0].b_im == a.p[1].b_im;
	const int na = (nprob == 2 && !same_a) ? 2 : 1, nb = (nprob == 2 && !same_b) ? 2 : 1;
	const size_t bytes = (na * a_floats + nb * b_floats) * sizeof(float);
	if (bytes > ((size_t) 2 << 30)) return false;
	if (rt().capturing && bytes > rt().operand_workspace_bytes) return false;  // the buffer cannot grow inside a recording
	float *buf = (float *) operand_workspace(bytes);
	if (!buf) {
		*rc = CNET_ERR_OUT_OF_MEMORY;
		return true;
	}
	CgemmArgs pk = a;
	pk.K = kp;
	pk.lda = a_ld;
	pk.ldb = b_ld;
	auto pack = [&](const float *re, const float *im, long ld, int rows, int cols, float *dst, int rows_d, int ldd) {
		const long threads = (long) rows_d * (ldd / 4);
		hipLaunchKernelGGL(pack_planes_kernel, dim3((unsigned) ((threads + 255) / 256), 2), dim3(256), 0, rt().stream, re, im, ld, rows, cols, dst,
				rows_d, ldd);
	};
	for (int q = 0; q < nprob; ++q) {
		float *pa = buf + (size_t) ((q == 1 && !same_a) ? 1 : 0) * a_floats;
		float *pb = buf + na * a_floats + (size_t) ((q == 1 && !same_b) ? 1 : 0) * b_floats;
		if (q == 0 || !same_a) pack(a.p[q].a_re, a.p[q].a_im, a.lda, a_mcontig ? a.K : a.M, a_mcontig ? a.M : a.K, pa, a_rows, a_ld);
		if (q == 0 || !same_b) pack(a.p[q].b_re, a.p[q].b_im, a.ldb, b_ncontig ? a.K : a.N, b_ncontig ? a.N : a.K, pb, b_rows, b_ld);
		pk.p[q].a_re = pa;
		pk.p[q].a_im = pa + (size_t) a_rows * a_ld;
		pk.p[q].b_re = pb;
		pk.p[q].b_im = pb + (size_t) b_rows * b_ld;
	}
	if (hipGetLastError() != hipSuccess) {
		*rc = fail(CNET_ERR_HIP, "cgemm: launch of the pass that aligns the operands failed");
		return true;
	}
	*rc = cgemm_dispatch(a_mcontig, b_ncontig, pk, nprob, batch);
	return true;
}

// nprob = 1 or 2 problems of identical shape.
static int cgemm_dispatch(bool a_mcontig, bool b_ncontig, CgemmArgs &a, int nprob, int batch) {
	if (a.M <= 0 || a.N <= 0) return CNET_OK;
	if (a.K <= 0) return fail(CNET_ERR_INVALID_ARGUMENT, "cgemm: K must be positive");
	if (a.a_real == 2) {  // (cgemm_folded has checked that the block kernels of this layout take it: nothing is split off)
		if (a_mcontig || !b_ncontig || nprob != 1 || batch != 1 || a.K % KC != 0)
			return fail(CNET_ERR_UNSUPPORTED, "cgemm: the folded form of a real operand is a row-major A against a k-major B, K in whole chunks");
		return pick_tile<false, true, 4>(a, nprob, batch);
	}
	if (a_mcontig || !b_ncontig) a.a_real = 0;  // only that layout has the kernels (the imaginary plane holds zeros: reading it is right too)
	int rc = CNET_OK;
	if (try_skinny(a_mcontig, b_ncontig, a, nprob, batch, &rc)) return rc;
	if (cgemm_packed(a_mcontig, b_ncontig, a, nprob, batch, &rc)) return rc;
	// A C that is a few columns wider than a multiple of the block width (784 = 12 x 64 + 16) costs a whole extra column
	// of blocks.  If the cost model says so, the product is done as two: the columns up to that multiple by the block
	// kernels, the narrow rest by the small-C kernel.  The two write disjoint columns of C.
	static const bool split_cols = [] {
		const char *e = getenv("CNET_CGEMM_COLSPLIT");  // tuning override: 0 never splits
		return !e || atoi(e) != 0;
	}();
	const int rest = a.N % 64;
	if (split_cols && !a.tri && batch == 1 && a.N > 64 && rest != 0 && rest <= 32 && a.K % KC == 0) {
		CgemmArgs left = a, right = a, planned;
		left.N = a.N - rest;
		right.N = rest;
		for (int q = 0; q < 2; ++q) {
			const long shift = b_ncontig ? left.N : (long) left.N * a.ldb;
			if (q < nprob) {
				right.p[q].b_re += shift;
				right.p[q].b_im += shift;
			}
			if (q < nprob || a.mirror) {  // the planes of p[1] are written by a mirrored product as well
				right.p[q].c_re += left.N;
				right.p[q].c_im += left.N;
			}
		}
		if (a.mirror == MIRROR_HERM) {  // columns of the right part count from its own first column
			right.herm_n = a.herm_n - 2 * left.N;
			right.herm_lo = a.herm_lo - left.N;
			right.herm_hi = a.herm_hi - left.N;
		}
		if (plan_skinny(a_mcontig, b_ncontig, right, nprob, batch, planned)) {
			int shape, tail, cuts;
			const double whole = plan_blocks(a, nprob, batch, block_layout(a_mcontig, b_ncontig), &shape, &tail, &cuts);
			const double parts = plan_blocks(left, nprob, batch, block_layout(a_mcontig, b_ncontig), &shape, &tail, &cuts) + skinny_us(planned, nprob, batch);
			if (parts < whole) {
				// one after the other on the compute stream: run side by side on two streams the narrow part's
				// workgroups took slots from the first round of the block kernel and the pair got slower (842 against
				// 773 us per step of the 784 -> 10 net at batch 4096)
				rc = cgemm_dispatch(a_mcontig, b_ncontig, left, nprob, batch);
				return rc != CNET_OK ? rc : cgemm_dispatch(a_mcontig, b_ncontig, right, nprob, batch);
			}
		}
	}
	// float4 path: every contiguous run starts 16-byte aligned and has a length that is a multiple of 4; a run along M or N
	// may also end inside its last group of four where the fast kernel takes the product (K in whole chunks, offsets that
	// fit): the leading dimension, a multiple of four, covers the group, and what the extra values feed is never stored
	auto vec_ok = [&](int K) {
		bool v = (a.lda % 4 == 0) && (a.ldb % 4 == 0) && (a.stride_a % 4 == 0) && (a.stride_b % 4 == 0);
		const bool ragged = K % KC == 0 && a.lda < (1L << 22) && a.ldb < (1L << 22);
		v = v && (a_mcontig ? (a.M % 4 == 0 || ragged) : K % 4 == 0) && (b_ncontig ? (a.N % 4 == 0 || ragged) : K % 4 == 0);
		for (int q = 0; q < nprob; ++q)
			v = v && aligned16(a.p[q].a_re) && aligned16(a.p[q].a_im) && aligned16(a.p[q].b_re) && aligned16(a.p[q].b_im);
		return v;
	};
	// A K that is not a whole number of chunks (a batch of 1000 in a weight gradient, a layer 1000 wide) would send the
	// whole product to the register-staged kernel (109-124 against 135-148 TFLOP/s on such shapes).  Instead the whole
	// chunks go to the fast kernel and the last 1..15 values of k are added by a second, short launch.
	static const bool split_k_rest = [] {
		const char *e = getenv("CNET_CGEMM_KREST");  // tuning override: 0 never splits off the rest of K
		return !e || atoi(e) != 0;
	}();
	const int k_rest = a.K % KC, k_whole = a.K - k_rest;
	if (split_k_rest && k_rest != 0 && k_whole >= 8 * KC && !a.tri && batch == 1 && vec_ok(k_whole) && (long) a.M * a.N >= 256 * 256) {
		CgemmArgs head = a, rest = a;
		head.K = k_whole;
		rest.K = k_rest;
		rest.accumulate = 1;  // onto what the first launch has written (its mirror planes too)
		for (int q = 0; q < nprob; ++q) {
			const long sa = a_mcontig ? (long) k_whole * a.lda : k_whole, sb = b_ncontig ? (long) k_whole * a.ldb : k_whole;
			rest.p[q].a_re += sa;
			rest.p[q].a_im += sa;
			rest.p[q].b_re += sb;
			rest.p[q].b_im += sb;
		}
		rc = cgemm_dispatch(a_mcontig, b_ncontig, head, nprob, batch);
		return rc != CNET_OK ? rc : cgemm_dispatch(a_mcontig, b_ncontig, rest, nprob, batch);
	}
	const bool vec = vec_ok(a.K);
	if (vec) {
		if (!a_mcontig && !b_ncontig) return pick_tile<false, false, 4>(a, nprob, batch);
		if (!a_mcontig && b_ncontig) return pick_tile<false, true, 4>(a, nprob, batch);
		if (a_mcontig && b_ncontig) return pick_tile<true, true, 4>(a, nprob, batch);
		return pick_tile<true, false, 4>(a, nprob, batch);
	}
	if (!a_mcontig && !b_ncontig) return pick_tile<false, false, 1>(a, nprob, batch);
	if (!a_mcontig && b_ncontig) return pick_tile<false, true, 1>(a, nprob, batch);
	if (a_mcontig && b_ncontig) return pick_tile<true, true, 1>(a, nprob, batch);
	return pick_tile<true, false, 1>(a, nprob, batch);
}

static CgemmArgs pair_args(int nprob, int M, int N, int K, const float *const a_re[2], const float *const a_im[2], long lda,
		const float *const b_re[2], const float *const b_im[2], long ldb, const bool conj_b[2], float *const c_re[2], float *const c_im[2],
		long ldc, int accumulate, int tri, int mirror);

// Called by cnet_graph_begin before the capture opens (see g_attrs_primed)
int cgemm_prime_attributes() {
	if (g_attrs_primed) return CNET_OK;
	hipError_t e = prime_shapes<false, false, 4>();
	if (e == hipSuccess) e = prime_shapes<false, true, 4>();
	if (e == hipSuccess) e = prime_shapes<true, true, 4>();
	if (e == hipSuccess) e = prime_shapes<true, false, 4>();
	if (e == hipSuccess) e = prime_shapes<false, false, 1>();
	if (e == hipSuccess) e = prime_shapes<false, true, 1>();
	if (e == hipSuccess) e = prime_shapes<true, true, 1>();
	if (e == hipSuccess) e = prime_shapes<true, false, 1>();
	if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute (dynamic LDS of the matrix kernels)");
	g_attrs_primed = true;
	return CNET_OK;
}

// Used by cdft.hip
int cgemm_pair(bool a_mcontig, bool b_ncontig, int nprob, int M, int N, int K, const float *const a_re[2],
		const float *const a_im[2], long lda, const float *const b_re[2], const float *const b_im[2], long ldb,
		const bool conj_b[2], float *const c_re[2], float *const c_im[2], long ldc, int accumulate, int tri, int mirror) {
	if (tri && N != K) return fail(CNET_ERR_INVALID_ARGUMENT, "cgemm: a triangular operand must be square");
	if (mirror && nprob != 1) return fail(CNET_ERR_INVALID_ARGUMENT, "cgemm: a mirrored product is one problem");
	CgemmArgs a = pair_args(nprob, M, N, K, a_re, a_im, lda, b_re, b_im, ldb, conj_b, c_re, c_im, ldc, accumulate, tri, mirror);
	return cgemm_dispatch(a_mcontig, b_ncontig, a, nprob, 1);
}

// y = x F, h = y .* hv (hv one shared row), g = gelu(h) in one launch of the small-C kernel, when the product is small enough
// for it and is not cut along K: *launched says whether it went out (used by cdft.hip; otherwise the caller runs the two passes)
int cgemm_dft_hgelu(int M, int n, const float *x_re, const float *x_im, long ldx, const float *f_re, const float *f_im, long ldf,
		const float *hv_re, const float *hv_im, float *y_re, float *y_im, float *h_re, float *h_im, float *g_re, float *g_im, long ld,
		bool *launched) {
	const float *ar[2] = {x_re, x_re}, *ai[2] = {x_im, x_im}, *br[2] = {f_re, f_re}, *bi[2] = {f_im, f_im};
	float *cr[2] = {y_re, h_re}, *ci[2] = {y_im, h_im};
	const bool cj[2] = {false, false};
	CgemmArgs a = pair_args(1, M, n, n, ar, ai, ldx, br, bi, ldf, cj, cr, ci, ld, 0, 0, MIRROR_HGELU);
	a.hv_re = hv_re;
	a.hv_im = hv_im;
	a.g_re = g_re;
	a.g_im = g_im;
	a.splits = 1;
	a.chunks_per_split = 0;
	a.partial = nullptr;
	a.tail_tiles = a.tail_splits = a.tail_chunks = 0;
	a.nprob = 1;
	*launched = false;
	CgemmArgs planned;
	if (!plan_skinny(false, true, a, 1, 1, planned) || planned.splits != 1) return CNET_OK;
	const SkinnyVariant v = skinny_variant(false, true, planned, 1, 1);
	*launched = true;
	return CNET_SKINNY_PICK(v, launch_skinny, (planned, false, true, 1, 1));
}

bool cgemm_linear_bwd_gate(const float *g_re, const float *g_im, long ldg, const float *x_re, const float *x_im, long ldx, const float *w_re,
		const float *w_im, long ldw, const Pair2 &dx, long lddx, int accumulate_dx, const Pair2 &dw, long lddw, int accumulate_dw, int B, int K,
		int N, const GateBwd &gate, int *rc) {
	if (B > GATE_MAX_ROWS) return false;
	// the two products as cnet_clinear_bwd_sym sets them up
	const float *gr[2] = {g_re, g_re}, *gi[2] = {g_im, g_im};
	const float *wr[2] = {w_re, w_re}, *wi[2] = {w_im, w_im}, *xr[2] = {x_re, x_re}, *xi[2] = {x_im, x_im};
	float *dxr[2] = {dx.dz_re, dx.dzs_re}, *dxi[2] = {dx.dz_im, dx.dzs_im}, *dwr[2] = {dw.dz_re, dw.dzs_re}, *dwi[2] = {dw.dz_im, dw.dzs_im};
	const bool cj[2] = {false, false};
	const CgemmArgs to_input = pair_args(1, B, K, N, gr, gi, ldg, wr, wi, ldw, cj, dxr, dxi, lddx, accumulate_dx, 0, dx.dzs_re ? MIRROR_CONJ : 0);
	const CgemmArgs to_weight = pair_args(1, N, K, B, gr, gi, ldg, xr, xi, ldx, cj, dwr, dwi, lddw, accumulate_dw, 0, dw.dzs_re ? MIRROR_CONJ : 0);
	CgemmArgs args0, args1;
	SkinnyVariant v;
	if (!plan_skinny_two(false, true, to_input, true, true, to_weight, 1, args0, args1, v)) return false;
	// one group of K per tile of dx (a wavefront forms it alone), the slab sums in LDS, one column block per workgroup
	if (args0.K > 16 || gate.nslabs > 32 || v.w * 64 * 2 * 4 < 32 * gate.nslabs) return false;
	const SkinnyStrides st0 = skinny_strides(args0, false, true), st1 = skinny_strides(args1, true, true);
	*rc = CNET_SKINNY_PICK(v, launch_skinny_gate_bwd, (args0, st0, args1, st1, gate));
	return true;
}

// Whether a product of this size would go to the block kernels (and not to the small-C kernel), as the folded form needs
bool cgemm_block_sized(int M, int N) {
	return ((long) (M + 15) / 16) * ((N + 15) / 16) > 4L * rt().prop.multiProcessorCount;
}

// C = (Ae B_re) + i (Ao B_im) for two real operands Ae, Ao [M][K] (K a multiple of 16, planes 16-byte aligned) against a
// k-major B, with the mirrored columns of cgemm_real_a (used by cdft.hip for the folded transform of real samples)
int cgemm_folded(int M, int N, int K, const float *ae, const float *ao, long lda, const float *b_re, const float *b_im, long ldb, float *c_re,
		float *c_im, long ldc, int herm_n) {
	const float *ar[2] = {ae, ae}, *ai[2] = {ao, ao}, *br[2] = {b_re, b_re}, *bi[2] = {b_im, b_im};
	float *cr[2] = {c_re, c_re}, *ci[2] = {c_im, c_im};
	const bool cj[2] = {false, false};
	CgemmArgs a = pair_args(1, M, N, K, ar, ai, lda, br, bi, ldb, cj, cr, ci, ldc, 0, 0, 0);
	a.a_real = 2;
	if (herm_n > N) {
		a.mirror = MIRROR_HERM;
		a.herm_n = herm_n;
		a.herm_lo = 1;
		a.herm_hi = herm_n - N;
	}
	return cgemm_dispatch(false, true, a, 1, 1);
}

// One product whose A (row-major) has an imaginary plane of nothing but +0, against a k-major B (used by cdft.hip)
// herm_n > 0: the conjugate of column c, 1 <= c <= herm_n - N, is also written to column herm_n - c (the columns from N on)
int cgemm_real_a(int M, int N, int K, const float *a_re, const float *a_im, long lda, const float *b_re, const float *b_im, long ldb, float *c_re,
		float *c_im, long ldc, int herm_n) {
	const float *ar[2] = {a_re, a_re}, *ai[2] = {a_im, a_im}, *br[2] = {b_re, b_re}, *bi[2] = {b_im, b_im};
	float *cr[2] = {c_re, c_re}, *ci[2] = {c_im, c_im};
	const bool cj[2] = {false, false};
	CgemmArgs a = pair_args(1, M, N, K, ar, ai, lda, br, bi, ldb, cj, cr, ci, ldc, 0, 0, 0);
	a.a_real = 1;
	if (herm_n > N) {
		a.mirror = MIRROR_HERM;
		a.herm_n = herm_n;
		a.herm_lo = 1;
		a.herm_hi = herm_n - N;
	}
	return cgemm_dispatch(false, true, a, 1, 1);
}

static CgemmArgs pair_args(int nprob, int M, int N, int K, const float *const a_re[2], const float *const a_im[2], long lda,
		const float *const b_re[2], const float *const b_im[2], long ldb, const bool conj_b[2], float *const c_re[2], float *const c_im[2],
		long ldc, int accumulate, int tri, int mirror) {
	CgemmArgs a;
	a.tri = tri;
	a.mirror = mirror;
	for (int q = 0; q < nprob; ++q) {
		a.p[q].a_re = a_re[q];
		a.p[q].a_im = a_im[q];
		a.p[q].b_re = b_re[q];
		a.p[q].b_im = b_im[q];
		a.p[q].c_re = c_re[q];
		a.p[q].c_im = c_im[q];
		a.p[q].a_im_sign = 1.0f;
		a.p[q].b_im_sign = conj_b[q] ? -1.0f : 1.0f;
	}
	if (nprob == 1) {
		a.p[1] = a.p[0];
		if (mirror) {  // the planes that receive the conjugate of the product, or its CGelu
			a.p[1].c_re = c_re[1];
			a.p[1].c_im = c_im[1];
		}
	}
	a.M = M;
	a.N = N;
	a.K = K;
	a.lda = lda;
	a.ldb = ldb;
	a.ldc = ldc;
	a.accumulate = accumulate;
	a.tiles_m = a.tiles_n = 0;
	a.stride_a = a.stride_b = a.stride_c = 0;
	return a;
}

}  // namespace cnet

using namespace cnet;

extern "C" {

int cnet_cgemm(int a_kmajor, int b_kmajor, int conj_b, int M, int N, int K, const float *a_re, const float *a_im,
		int64_t lda, const float *b_re, const float *b_im, int64_t ldb, float *c_re, float *c_im, int64_t ldc,
		int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(M >= 0 && N >= 0 && K > 0);
	if (M == 0 || N == 0) return CNET_OK;
	CNET_CHECK_ARG(a_re && a_im && b_re && b_im && c_re && c_im);
	CNET_CHECK_ARG(lda >= (a_kmajor ? M : K) && ldb >= (b_kmajor ? N : K) && ldc >= N);
	const float *ar[2] = {a_re, a_re}, *ai[2] = {a_im, a_im}, *br[2] = {b_re, b_re}, *bi[2] = {b_im, b_im};
	float *cr[2] = {c_re, c_re}, *ci[2] = {c_im, c_im};
	bool cj[2] = {conj_b != 0, conj_b != 0};
	return cgemm_pair(a_kmajor != 0, b_kmajor != 0, 1, M, N, K, ar, ai, lda, br, bi, ldb, cj, cr, ci, ldc, accumulate, 0, 0);
}

int cnet_cgemm_batched(int a_kmajor, int b_kmajor, int conj_a, int conj_b, int M, int N, int K, const float *a_re,
		const float *a_im, int64_t lda, int64_t stride_a, const float *b_re, const float *b_im, int64_t ldb, int64_t stride_b,
		float *c_re, float *c_im, int64_t ldc, int64_t stride_c, int batch, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(M >= 0 && N >= 0 && K > 0 && batch >= 0 && batch <= 65535);
	if (M == 0 || N == 0 || batch == 0) return CNET_OK;
	CNET_CHECK_ARG(a_re && a_im && b_re && b_im && c_re && c_im);
	CNET_CHECK_ARG(lda >= (a_kmajor ? M : K) && ldb >= (b_kmajor ? N : K) && ldc >= N);
	CNET_CHECK_ARG(stride_a >= 0 && stride_b >= 0 && (batch == 1 || stride_c >= (int64_t) M * ldc - (ldc - N)));
	CgemmArgs a;
	a.tri = 0;
	a.mirror = 0;
	a.p[0].a_re = a_re;
	a.p[0].a_im = a_im;
	a.p[0].b_re = b_re;
	a.p[0].b_im = b_im;
	a.p[0].c_re = c_re;
	a.p[0].c_im = c_im;
	a.p[0].a_im_sign = conj_a ? -1.0f : 1.0f;
	a.p[0].b_im_sign = conj_b ? -1.0f : 1.0f;
	a.p[1] = a.p[0];
	a.M = M;
	a.N = N;
	a.K = K;
	a.lda = lda;
	a.ldb = ldb;
	a.ldc = ldc;
	a.accumulate = accumulate;
	a.tiles_m = a.tiles_n = 0;
	a.stride_a = stride_a;
	a.stride_b = stride_b;
	a.stride_c = stride_c;
	return cgemm_dispatch(a_kmajor != 0, b_kmajor != 0, a, 1, batch);
}

int cnet_cgemm_set_products(int n) {
	CNET_CHECK_ARG(n == 3 || n == 4);
	if (cnet::rt().capturing && (n == 3) != three_products())
		return cnet::fail(CNET_ERR_UNSUPPORTED, "cnet_cgemm_set_products: not between cnet_graph_begin and cnet_graph_end");
	g_three_products = n == 3;
	return CNET_OK;
}

int cnet_cgemm_get_products(void) { return three_products() ? 3 : 4; }

int cnet_clinear_fwd(const float *x_re, const float *x_im, int64_t ldx, const float *w_re, const float *w_im,
		int64_t ldw, float *y_re, float *y_im, int64_t ldy, int B, int K, int N, int accumulate) {
	// y[B][N] = x[B][K] * w[N][K]^T : both operands contiguous along the reduction index
	return cnet_cgemm(0, 0, 0, B, N, K, x_re, x_im, ldx, w_re, w_im, ldw, y_re, y_im, ldy, accumulate);
}

int cnet_clinear_cgelu_fwd(const float *x_re, const float *x_im, int64_t ldx, const float *w_re, const float *w_im, int64_t ldw,
		float *h_re, float *h_im, float *y_re, float *y_im, int64_t ldy, int B, int K, int N, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && N >= 0 && K > 0);
	if (B == 0 || N == 0) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && w_re && w_im && h_re && h_im && y_re && y_im);
	CNET_CHECK_ARG(ldx >= K && ldw >= K && ldy >= N);
	const float *ar[2] = {x_re, x_re}, *ai[2] = {x_im, x_im}, *br[2] = {w_re, w_re}, *bi[2] = {w_im, w_im};
	float *cr[2] = {h_re, y_re}, *ci[2] = {h_im, y_im};
	bool cj[2] = {false, false};
	return cgemm_pair(false, false, 1, B, N, K, ar, ai, ldx, br, bi, ldw, cj, cr, ci, ldy, accumulate, 0, MIRROR_GELU);
}

int cnet_clinear_cross_entropy_fwd_bwd_sym(const float *x_re, const float *x_im, int64_t ldx, const float *w_re, const float *w_im, int64_t ldw,
		float *y_re, float *y_im, int64_t ldy, const int32_t *labels, float *out_re, float *out_im, int64_t ldo, float *s, float *loss,
		int32_t *argmax, float *dz_dz_re, float *dz_dz_im, float *dz_dzs_re, float *dz_dzs_im, int64_t lddz, int B, int K, int N) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && N > 0 && K > 0);
	if (B == 0) return CNET_OK;
	CNET_CHECK_ARG(x_re && x_im && w_re && w_im && y_re && y_im && labels && s && loss && argmax);
	CNET_CHECK_ARG(ldx >= K && ldw >= K && ldy >= N);
	CNET_CHECK_ARG((out_re == nullptr) == (out_im == nullptr) && (out_re == nullptr || ldo >= N));
	CNET_CHECK_ARG(dz_dz_re && dz_dz_im && ((dz_dzs_re == nullptr) == (dz_dzs_im == nullptr)) && lddz >= N);
	if (N <= 16) {
		const float *ar[2] = {x_re, x_re}, *ai[2] = {x_im, x_im}, *br[2] = {w_re, w_re}, *bi[2] = {w_im, w_im};
		float *cr[2] = {y_re, y_re}, *ci[2] = {y_im, y_im};
		const bool cj[2] = {false, false};
		CgemmArgs a = pair_args(1, B, N, K, ar, ai, ldx, br, bi, ldw, cj, cr, ci, ldy, 0, 0, MIRROR_CE), planned;
		if (plan_skinny(false, false, a, 1, 1, planned) && planned.splits == 1 && planned.tiles_n == 1) {
			planned.ce_labels = labels;
			planned.ce_out_re = out_re;
			planned.ce_out_im = out_im;
			planned.ce_ldo = ldo;
			planned.ce_s = s;
			planned.ce_loss = loss;
			planned.ce_argmax = argmax;
			planned.ce_dz_re = dz_dz_re;
			planned.ce_dz_im = dz_dz_im;
			planned.ce_dzs_re = dz_dzs_re;
			planned.ce_dzs_im = dz_dzs_im;
			planned.ce_lddz = lddz;
			// the instantiation cnet_cross_entropy_fwd_bwd_sym would run on these planes
			auto m4 = [](long v) { return v % 4 == 0; };
			planned.ce_vec = m4(N) && m4(ldy) && (!out_re || m4(ldo)) && m4(lddz) && aligned16(y_re) && aligned16(y_im) && aligned16(out_re) &&
					aligned16(out_im) && aligned16(dz_dz_re) && aligned16(dz_dz_im) && aligned16(dz_dzs_re) && aligned16(dz_dzs_im);
			const SkinnyVariant v = skinny_variant(false, false, planned, 1, 1);
			return CNET_SKINNY_PICK(v, launch_skinny_ce, (planned, false, false));
		}
	}
	// a head too wide or too tall for that kernel: the product, then the pass over its rows
	const int rc = cnet_clinear_fwd(x_re, x_im, ldx, w_re, w_im, ldw, y_re, y_im, ldy, B, K, N, 0);
	return rc ? rc : cnet_cross_entropy_fwd_bwd_sym(y_re, y_im, ldy, labels, out_re, out_im, ldo, s, loss, argmax, dz_dz_re, dz_dz_im, dz_dzs_re,
			dz_dzs_im, lddz, B, N);
}

int cnet_clinear_bwd_input(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im,
		int64_t ldg, const float *w_re, const float *w_im, int64_t ldw, float *dx_dz_re, float *dx_dz_im,
		float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int B, int K, int N, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && K >= 0 && N > 0);
	if (B == 0 || K == 0) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && g_dzs_re && g_dzs_im && w_re && w_im);
	CNET_CHECK_ARG(dx_dz_re && dx_dz_im && dx_dzs_re && dx_dzs_im);
	CNET_CHECK_ARG(ldg >= N && ldw >= K && lddx >= K);
	// dx[B][K] = g[B][N] * w[N][K] : reduction over N; w is stored [k=N][n=K]
	const float *ar[2] = {g_dz_re, g_dzs_re}, *ai[2] = {g_dz_im, g_dzs_im};
	const float *br[2] = {w_re, w_re}, *bi[2] = {w_im, w_im};
	float *cr[2] = {dx_dz_re, dx_dzs_re}, *ci[2] = {dx_dz_im, dx_dzs_im};
	bool cj[2] = {false, true};
	return cgemm_pair(false, true, 2, B, K, N, ar, ai, ldg, br, bi, ldw, cj, cr, ci, lddx, accumulate, 0, 0);
}

int cnet_clinear_bwd_weight(const float *g_dz_re, const float *g_dz_im, const float *g_dzs_re, const float *g_dzs_im,
		int64_t ldg, const float *x_re, const float *x_im, int64_t ldx, float *dw_dz_re, float *dw_dz_im,
		float *dw_dzs_re, float *dw_dzs_im, int64_t lddw, int B, int K, int N, int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B > 0 && K >= 0 && N >= 0);
	if (N == 0 || K == 0) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && g_dzs_re && g_dzs_im && x_re && x_im);
	CNET_CHECK_ARG(dw_dz_re && dw_dz_im && dw_dzs_re && dw_dzs_im);
	CNET_CHECK_ARG(ldg >= N && ldx >= K && lddw >= K);
	// dw[N][K] = g[B][N]^T * x[B][K] : reduction over the batch; both operands stored [k=B][row]
	const float *ar[2] = {g_dz_re, g_dzs_re}, *ai[2] = {g_dz_im, g_dzs_im};
	const float *br[2] = {x_re, x_re}, *bi[2] = {x_im, x_im};
	float *cr[2] = {dw_dz_re, dw_dzs_re}, *ci[2] = {dw_dz_im, dw_dzs_im};
	bool cj[2] = {false, true};
	return cgemm_pair(true, true, 2, N, K, B, ar, ai, ldg, br, bi, ldx, cj, cr, ci, lddw, accumulate, 0, 0);
}

int cnet_clinear_bwd_input_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, const float *w_re, const float *w_im,
		int64_t ldw, float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx, int B, int K, int N,
		int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B >= 0 && K >= 0 && N > 0);
	if (B == 0 || K == 0) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && w_re && w_im && dx_dz_re && dx_dz_im && ((dx_dzs_re == nullptr) == (dx_dzs_im == nullptr)));
	CNET_CHECK_ARG(ldg >= N && ldw >= K && lddx >= K);
	// dx = g * w as in cnet_clinear_bwd_input; dx* = conj(g) * conj(w) is its conjugate and is written, not computed
	const float *ar[2] = {g_dz_re, g_dz_re}, *ai[2] = {g_dz_im, g_dz_im};
	const float *br[2] = {w_re, w_re}, *bi[2] = {w_im, w_im};
	float *cr[2] = {dx_dz_re, dx_dzs_re}, *ci[2] = {dx_dz_im, dx_dzs_im};
	bool cj[2] = {false, false};
	return cgemm_pair(false, true, 1, B, K, N, ar, ai, ldg, br, bi, ldw, cj, cr, ci, lddx, accumulate, 0, dx_dzs_re != nullptr ? MIRROR_CONJ : 0);
}

int cnet_clinear_bwd_weight_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, const float *x_re, const float *x_im,
		int64_t ldx, float *dw_dz_re, float *dw_dz_im, float *dw_dzs_re, float *dw_dzs_im, int64_t lddw, int B, int K, int N,
		int accumulate) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B > 0 && K >= 0 && N >= 0);
	if (N == 0 || K == 0) return CNET_OK;
	CNET_CHECK_ARG(g_dz_re && g_dz_im && x_re && x_im && dw_dz_re && dw_dz_im && ((dw_dzs_re == nullptr) == (dw_dzs_im == nullptr)));
	CNET_CHECK_ARG(ldg >= N && ldx >= K && lddw >= K);
	const float *ar[2] = {g_dz_re, g_dz_re}, *ai[2] = {g_dz_im, g_dz_im};
	const float *br[2] = {x_re, x_re}, *bi[2] = {x_im, x_im};
	float *cr[2] = {dw_dz_re, dw_dzs_re}, *ci[2] = {dw_dz_im, dw_dzs_im};
	bool cj[2] = {false, false};
	return cgemm_pair(true, true, 1, N, K, B, ar, ai, ldg, br, bi, ldx, cj, cr, ci, lddw, accumulate, 0, dw_dzs_re != nullptr ? MIRROR_CONJ : 0);
}

int cnet_clinear_bwd_sym(const float *g_dz_re, const float *g_dz_im, int64_t ldg, const float *x_re, const float *x_im, int64_t ldx,
		const float *w_re, const float *w_im, int64_t ldw, float *dx_dz_re, float *dx_dz_im, float *dx_dzs_re, float *dx_dzs_im, int64_t lddx,
		int accumulate_dx, float *dw_dz_re, float *dw_dz_im, float *dw_dzs_re, float *dw_dzs_im, int64_t lddw, int accumulate_dw, int B,
		int K, int N) {
	CNET_REQUIRE_INIT();
	CNET_CHECK_ARG(B > 0 && K > 0 && N > 0);
	CNET_CHECK_ARG(g_dz_re && g_dz_im && x_re && x_im && w_re && w_im);
	CNET_CHECK_ARG(dx_dz_re && dx_dz_im && ((dx_dzs_re == nullptr) == (dx_dzs_im == nullptr)));
	CNET_CHECK_ARG(dw_dz_re && dw_dz_im && ((dw_dzs_re == nullptr) == (dw_dzs_im == nullptr)));
	CNET_CHECK_ARG(ldg >= N && ldx >= K && ldw >= K && lddx >= K && lddw >= K);
	// the two products as cnet_clinear_bwd_input_sym and cnet_clinear_bwd_weight_sym set them up
	const float *gr[2] = {g_dz_re, g_dz_re}, *gi[2] = {g_dz_im, g_dz_im};
	const float *wr[2] = {w_re, w_re}, *wi[2] = {w_im, w_im}, *xr[2] = {x_re, x_re}, *xi[2] = {x_im, x_im};
	float *dxr[2] = {dx_dz_re, dx_dzs_re}, *dxi[2] = {dx_dz_im, dx_dzs_im}, *dwr[2] = {dw_dz_re, dw_dzs_re}, *dwi[2] = {dw_dz_im, dw_dzs_im};
	const bool cj[2] = {false, false};
	CgemmArgs to_input = pair_args(1, B, K, N, gr, gi, ldg, wr, wi, ldw, cj, dxr, dxi, lddx, accumulate_dx, 0, dx_dzs_re ? MIRROR_CONJ : 0);
	CgemmArgs to_weight = pair_args(1, N, K, B, gr, gi, ldg, xr, xi, ldx, cj, dwr, dwi, lddw, accumulate_dw, 0, dw_dzs_re ? MIRROR_CONJ : 0);
	int rc = CNET_OK;
	if (try_skinny_two(false, true, to_input, true, true, to_weight, 1, &rc)) return rc;
	rc = cgemm_dispatch(false, true, to_input, 1, 1);
	return rc != CNET_OK ? rc : cgemm_dispatch(true, true, to_weight, 1, 1);
}

}  // extern "C"
