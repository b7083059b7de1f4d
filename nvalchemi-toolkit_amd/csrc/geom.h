// Pair geometry shared by the neighbor search and the pair kernel.
//
// The separation of atom j (image S) from atom i is defined on the float32 inputs as
//   d = (r_j - r_i) + (S0*a0 + S1*a1 + S2*a2),   a_k = rows of the cell,
// evaluated in double with one rounding per operation (no fused multiply-add), in exactly
// this association.  Both kernels decide "inside the cutoff" from this one expression, so a
// pair the list holds is a pair the potential sees.
// Convention: nvalchemi/models/_ops/neighbor_filter.py:98-119 (r_j - r_i + shift . cell,
// row-vector cell, strict <).
#pragma once

#include <hip/hip_runtime.h>

namespace nvamd {

struct Cell64 {
    double h[9];
};

// S . cell in the fixed association of the definition above (cell given as float32 rows)
__device__ __forceinline__ void shift_vector(const float* __restrict__ cell, int s0, int s1, int s2, double& tx,
                                             double& ty, double& tz) {
#pragma clang fp contract(off)
    const double a = (double)s0, b = (double)s1, c = (double)s2;
    tx = (a * (double)cell[0] + b * (double)cell[3]) + c * (double)cell[6];
    ty = (a * (double)cell[1] + b * (double)cell[4]) + c * (double)cell[7];
    tz = (a * (double)cell[2] + b * (double)cell[5]) + c * (double)cell[8];
}

// d = (r_j - r_i) + t and its square, t = S . cell already evaluated
__device__ __forceinline__ double pair_d2_shifted(float xi, float yi, float zi, float xj, float yj, float zj,
                                                  double tx, double ty, double tz, double& d0, double& d1,
                                                  double& d2) {
#pragma clang fp contract(off)
    d0 = ((double)xj - (double)xi) + tx;
    d1 = ((double)yj - (double)yi) + ty;
    d2 = ((double)zj - (double)zi) + tz;
    return (d0 * d0 + d1 * d1) + d2 * d2;
}

// The same d for a cell without off-diagonal terms when the wanted image is the nearest one:
// d_k = dd_k - rint(dd_k / h_kk) h_kk.  rint(.) is the negated shift, its product with h_kk is exact
// in double, so the fused multiply-add rounds once, exactly like dd_k + (S . cell)_k above.
__device__ __forceinline__ double pair_d2_nearest_diagonal(float xi, float yi, float zi, float xj, float yj,
                                                           float zj, const double* h, const double* h_inv,
                                                           double& d0, double& d1, double& d2) {
#pragma clang fp contract(off)
    const double e0 = (double)xj - (double)xi, e1 = (double)yj - (double)yi, e2 = (double)zj - (double)zi;
    d0 = __builtin_fma(-__builtin_rint(e0 * h_inv[0]), h[0], e0);
    d1 = __builtin_fma(-__builtin_rint(e1 * h_inv[1]), h[1], e1);
    d2 = __builtin_fma(-__builtin_rint(e2 * h_inv[2]), h[2], e2);
    return (d0 * d0 + d1 * d1) + d2 * d2;
}

// (the coordinates come as doubles: float32 inputs convert exactly, float64 inputs are used as they are)
__device__ __forceinline__ double pair_d2_exact(double xi, double yi, double zi, double xj, double yj,
                                                double zj, int s0, int s1, int s2,
                                                const double* __restrict__ h, double& d0,
                                                double& d1, double& d2) {
#pragma clang fp contract(off)
    double a = (double)s0, b = (double)s1, c = (double)s2;
    double tx = (a * h[0] + b * h[3]) + c * h[6];
    double ty = (a * h[1] + b * h[4]) + c * h[7];
    double tz = (a * h[2] + b * h[5]) + c * h[8];
    d0 = (xj - xi) + tx;
    d1 = (yj - yi) + ty;
    d2 = (zj - zi) + tz;
    return (d0 * d0 + d1 * d1) + d2 * d2;
}

// inverse of a 3x3 matrix given row-major (adjugate over determinant)
__device__ __forceinline__ void inv3(const double* m, double* inv) {
    double c00 = m[4] * m[8] - m[5] * m[7];
    double c01 = m[5] * m[6] - m[3] * m[8];
    double c02 = m[3] * m[7] - m[4] * m[6];
    double det = m[0] * c00 + m[1] * c01 + m[2] * c02;
    double id = 1.0 / det;
    inv[0] = c00 * id;
    inv[1] = (m[2] * m[7] - m[1] * m[8]) * id;
    inv[2] = (m[1] * m[5] - m[2] * m[4]) * id;
    inv[3] = c01 * id;
    inv[4] = (m[0] * m[8] - m[2] * m[6]) * id;
    inv[5] = (m[2] * m[3] - m[0] * m[5]) * id;
    inv[6] = c02 * id;
    inv[7] = (m[1] * m[6] - m[0] * m[7]) * id;
    inv[8] = (m[0] * m[4] - m[1] * m[3]) * id;
}

// blockIdx -> logical block so that each of the 8 XCDs (which receive consecutive
// workgroups round-robin) walks one contiguous eighth of the index space and keeps its
// own slice of the gathered data in its L2.
__device__ __forceinline__ unsigned xcd_contiguous_block(unsigned b, unsigned n_blocks) {
    constexpr unsigned kXcd = 8;
    unsigned per = (n_blocks + kXcd - 1) / kXcd;
    return (b % kXcd) * per + b / kXcd;  // may be >= n_blocks: caller skips
}

}  // namespace nvamd
