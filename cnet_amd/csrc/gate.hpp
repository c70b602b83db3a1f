// What elementwise.hip and cgemm.hip both name of the backward pass of a Hadamard gate under a real loss: the planes of a
// gradient pair, the order in which the rows of a batch are added into the gradient of a shared row of weights, and the
// launch that runs that backward pass behind the two backward products of a narrow Linear layer.
#ifndef CNET_CSRC_GATE_HPP_
#define CNET_CSRC_GATE_HPP_

#include <algorithm>

namespace cnet {

struct Pair2 {  // dz planes, and optionally the planes that receive the conjugate
	float *dz_re, *dz_im, *dzs_re, *dzs_im;
};

// Workgroup of the shared-row kernels: GATE_CS_X column groups x GATE_CS_Y row lanes.  The rows of the batch are cut into
// `nslabs` slabs of `rows_per_slab`; inside a slab row lane ty adds rows r0 + ty, r0 + ty + 4, ... and the four lanes are
// added as ((0 + 1) + 2) + 3; the slabs are added by 4 lanes (64 beyond 32 slabs) that each take a run of slabs in
// order, and those lanes in order.  Two workgroups per compute unit: against four, 129 instead of 138 us at 8192 x 4096 and
// 10.0 instead of 11.4 us at 1024 x 784 (half as many slabs to add); one per unit is slower everywhere.
constexpr int GATE_CS_X = 64, GATE_CS_Y = 4;
inline void gate_slabs(int rows, int cols, int vec_width, int compute_units, int *nslabs, int *rows_per_slab) {
	const long col_blocks = ((long) cols / vec_width + GATE_CS_X - 1) / GATE_CS_X;
	int n = (int) std::max(1L, std::min(256L, 2L * compute_units / col_blocks));
	n = std::min(n, (rows + GATE_CS_Y - 1) / GATE_CS_Y);
	*rows_per_slab = (rows + n - 1) / n;
	*nslabs = (rows + *rows_per_slab - 1) / *rows_per_slab;
}

// The gate h = u .* v (v one shared row) under a CGelu, backward, for the workgroup that has just formed 16 columns of the
// gradient at the CGelu's result (all rows): dh, du and the batch sum dv of those columns.
struct GateBwd {
	const float *u_re, *u_im;
	long ldu;
	const float *v_re, *v_im;
	Pair2 dh;  // gradient at the CGelu's operand (dz_re NULL: not kept)
	long lddh;
	Pair2 du;
	long lddu;
	Pair2 dv;  // one row
	int accumulate;  // of du and dv
	int nslabs, rows_per_slab;  // gate_slabs() of the shape: the order in which the separate launches add the rows
};
constexpr int GATE_MAX_ROWS = 128;  // rows of the batch one workgroup keeps in LDS

// dx = g w and dw = g^T x of a Linear (as cnet_clinear_bwd_sym) with the backward pass `gate` of the gate whose CGelu
// produced x, in one launch of the small-C kernel: false when the shape does not fit (nothing launched), else *rc set.
bool cgemm_linear_bwd_gate(const float *g_re, const float *g_im, long ldg, const float *x_re, const float *x_im, long ldx, const float *w_re,
		const float *w_im, long ldw, const Pair2 &dx, long lddx, int accumulate_dx, const Pair2 &dw, long lddw, int accumulate_dw, int B, int K,
		int N, const GateBwd &gate, int *rc);

}  // namespace cnet

#endif
