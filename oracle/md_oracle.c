/*
 * md_oracle.c -- CPU restatement of the batched-MD inner loop of nvalchemi-toolkit.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP path: it may be
 * loaded by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg, and by
 * nothing else.  The product library never links, imports or calls it.
 *
 * The arithmetic of this path lives in a third-party wheel that is absent from the
 * reference tree (nvalchemi-toolkit-ops==0.4.0, pinned in uv.lock:186-189,4168), so every
 * function below restates the published algorithm and anchors on the reference's own call
 * sites, docstrings and tests:
 *
 *   orc_nl_brute / orc_nl_cell   nvalchemi/neighbors.py:244-273 (output layout, overflow
 *                                protocol), nvalchemi/models/_ops/neighbor_filter.py:98-119
 *                                (pair geometry r_ij = r_j - r_i + S.cell, row-vector cell,
 *                                strict d2 < rc2), nvalchemi/hooks/neighbor_list.py:685-704
 *                                (bin -> histogram -> scan -> scatter -> stencil search)
 *   orc_lj_matrix                nvalchemi/models/_ops/lj.py:31-54,116-216,246-321 and
 *                                nvalchemi/models/lj.py:464-477 (fp64 per-system sum)
 *   orc_vv_pre / orc_vv_post     nvalchemi/dynamics/_ops/velocity_verlet.py:63-64,112
 *   orc_langevin_half_step       nvalchemi/dynamics/_ops/langevin.py:52-117,
 *                                nvalchemi/dynamics/integrators/nvt_langevin.py:103-196
 *   orc_nhc_chain_update         nvalchemi/dynamics/_ops/nose_hoover.py:143-246 (arguments, what is
 *                                updated in place), nvalchemi/dynamics/integrators/nvt_nose_hoover.py
 *                                :215-281 (chain - kick - drift | kick - chain)
 *   orc_fire_step                nvalchemi/dynamics/_ops/fire.py:245-362,
 *                                nvalchemi/dynamics/optimizers/fire.py:69-76,182-219,
 *                                nvalchemi/distributed/_dynamics_coordinator.py:296-322
 *   orc_fire2_step               nvalchemi/dynamics/_ops/fire.py:467-557 (arguments, defaults, what is
 *                                updated in place), nvalchemi/dynamics/optimizers/fire2.py:18-27,218-251
 *                                (the whole step before the forces, nothing after them)
 *   orc_fmax                     nvalchemi/dynamics/base.py:304-349
 *   orc_rebuild_check            nvalchemi/dynamics/_ops/neighbor_list_rebuild.py:37-139 (the
 *                                displacement kernel itself is in the absent wheel)
 *   orc_wrap_positions           nvalchemi/hooks/periodic.py:42-114
 *
 * Pinning status (what checks each function; see tests/test_oracle_*.py):
 *   orc_nl_brute   pinned: hand geometries restated from the reference tests
 *                  (test/hooks/test_neighbor_list_hook.py:65-105,630-719,
 *                  test/models/test_neighbor_filter.py:182-215), invariants (symmetry,
 *                  no self pair, no cross-system pair), lattice coordination numbers.
 *   orc_nl_cell    pinned against orc_nl_brute (set equality on random periodic,
 *                  triclinic, mixed-pbc, small-cell and non-periodic inputs).
 *   orc_lj_matrix  pinned: closed forms (u(sigma)=0, u(2^(1/6)sigma)=-eps with zero
 *                  force, literal dimer value), F = -dE/dr by fp64 finite differences,
 *                  W = -dE/d(strain) by finite differences, sum F = 0.
 *                  Still unpinned by anything the reference holds: whether the truncated
 *                  potential is energy-shifted at the cutoff (taken as NOT shifted), the
 *                  half-list energy attribution, and the C2 switching polynomial for
 *                  switch_width > 0: PARITY UNPINNED (the reference only says "C2-continuous ...
 *                  between cutoff - switch_width and cutoff"; the quintic of least degree is
 *                  taken and checked for what C2 continuity demands: S = 1 / 0 and zero slope
 *                  and curvature at the ends, S(1/2) = 1/2, F = -dE/dr by finite differences).
 *   orc_vv_*       pinned: harmonic-oscillator closed form, time reversibility.
 *   orc_fire_step  PARITY UNPINNED against the reference: the step is inside the absent wheel.
 *                  The order of its sub-steps follows the reference's own sentences (reductions
 *                  over what is passed in; MD integration with the stored dt, then mixing with
 *                  the stored alpha, then the parameter update; per-atom maxstep clamp; vanilla
 *                  branch only), each cited at the function.  Checked against those sentences
 *                  (tests that a mix-first order, post-kick reductions or an updated dt in the
 *                  integration would fail) and by invariants; what no sentence decides is
 *                  listed at the function.
 *   orc_langevin_half_step  PARITY UNPINNED against the reference: its random stream and the rounding
 *                  of its kernel are inside the absent library.  Pinned as mathematics: the generator
 *                  by the published Philox4x32-10 known answers, the deviates by their moments, the
 *                  step by its limits (no friction: the two half drifts of velocity Verlet; infinite
 *                  friction: velocities redrawn at kT/m) and by the invariance of the Maxwell-Boltzmann
 *                  variance under the O step.
 *   orc_fire2_step  PARITY UNPINNED against the reference: the step is inside the absent library.  The
 *                  parameter names (delaystep, dtgrow, dtshrink, alphashrink, alpha0, tmax, tmin) are those of
 *                  FIRE 2.0 as published with its LAMMPS implementation (Guenole et al., Comput. Mater. Sci.
 *                  175, 109584 (2020)); the restatement follows that algorithm with the semi-implicit Euler
 *                  integrator, the half step back on a reset, unit masses (the reference's op takes none) and
 *                  no initial delay (its state holds no step count).  Taken without evidence: mixing factors
 *                  from the alpha and |v| of the entry, applied after the kick; the half step back with the
 *                  time step before its reduction; maxstep as a limit on the largest atomic displacement of
 *                  a system, by scaling the whole system's step.  Checked by what the algorithm fixes (the
 *                  Euler limit, the reset, the bounds on dt and on the displacement, the counter) and by
 *                  reaching the minimum.
 *   orc_nhc_chain_update  PARITY UNPINNED against the reference: the kernel is inside the absent
 *                  library (the reference only names it: Martyna-Tobias-Klein equations, Yoshida-Suzuki
 *                  factorisation, chain masses Q_1 = N_f kT tau^2, Q_k = kT tau^2).  The restatement is
 *                  the published half-step propagator of Martyna, Tuckerman, Tobias and Klein (Mol. Phys.
 *                  87, 1117 (1996)) with one pass of the 3- or 5-weight Suzuki-Yoshida scheme.  Pinned as
 *                  mathematics: second-order convergence of the whole step to an adaptive integration of
 *                  the Nose-Hoover chain equations of motion, the conserved extended energy, time
 *                  reversal, weights summing to one.
 *   orc_fmax       pinned: in-tree Torch definition is complete; literal cases.
 *   orc_rebuild_check  pinned by the reference's own cases (flags cleared on every call, 1.0 over a
 *                  threshold of 0.5 flags, 0.1 does not, per-system selectivity, reference refreshed
 *                  only when flagged: test/hooks/test_neighbor_list_hook.py:166-246).  PARITY UNPINNED:
 *                  strict versus non-strict comparison at the threshold, the minimum-image form of the
 *                  displacement, and whether the refresh covers the flagged system's unmoved atoms
 *                  (taken: strict, nearest image on periodic axes, whole system).
 *   orc_wrap_positions  pinned by the documented formula (frac = r . inv(cell), frac mod 1, back;
 *                  nvalchemi/hooks/periodic.py:159-163) and the in-tree masking (:111-113); the
 *                  float32 rounding of the absent Warp kernel is unpinned (computed in double here).
 *
 * Numerical definition of the neighbor set: the pair (i, j, S) is a neighbor iff
 *   d = (r_j - r_i) + (S0*a0 + S1*a1 + S2*a2),  d.d < rc*rc
 * evaluated in IEEE double on the given float32 inputs (each operation rounded once,
 * no fused multiply-add), i.e. to within 1e-15 of exact arithmetic on the inputs.
 * Compile with -ffp-contract=off.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))
#define ORC_VMAX 3.0e38f

/* ------------------------------------------------------------------------------------------
 * per-system geometry
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    double h[9];    /* rows = lattice vectors */
    double hinv[9]; /* inverse, so frac = r . hinv (row vector times matrix) */
    double width[3]; /* perpendicular width of the cell along each lattice direction */
    int per[3];
    int has_cell;
} orc_sys_t;

static void orc_inv3(const double* m, double* inv) {
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

static void orc_sys_init(orc_sys_t* s, const float* cell, const uint8_t* pbc) {
    int d, k;
    if (cell) {
        for (k = 0; k < 9; ++k) s->h[k] = (double)cell[k];
        s->has_cell = 1;
    } else {
        for (k = 0; k < 9; ++k) s->h[k] = (k % 4 == 0) ? 1.0 : 0.0;
        s->has_cell = 0;
    }
    orc_inv3(s->h, s->hinv);
    for (d = 0; d < 3; ++d) {
        /* column d of hinv is the reciprocal vector of lattice direction d */
        double nx = s->hinv[0 + d], ny = s->hinv[3 + d], nz = s->hinv[6 + d];
        s->width[d] = 1.0 / sqrt(nx * nx + ny * ny + nz * nz);
        s->per[d] = (cell && pbc) ? (pbc[d] != 0) : 0;
    }
}

static inline void orc_frac(const orc_sys_t* s, const float* r, double* f) {
    double x = r[0], y = r[1], z = r[2];
    f[0] = x * s->hinv[0] + y * s->hinv[3] + z * s->hinv[6];
    f[1] = x * s->hinv[1] + y * s->hinv[4] + z * s->hinv[7];
    f[2] = x * s->hinv[2] + y * s->hinv[5] + z * s->hinv[8];
}

/* the one definition of the pair separation, shared by the neighbor test and LJ */
static inline double orc_pair_d2(const float* ri, const float* rj, const int* S, const double* h,
                                 double* d) {
    double tx = ((double)S[0] * h[0] + (double)S[1] * h[3]) + (double)S[2] * h[6];
    double ty = ((double)S[0] * h[1] + (double)S[1] * h[4]) + (double)S[2] * h[7];
    double tz = ((double)S[0] * h[2] + (double)S[1] * h[5]) + (double)S[2] * h[8];
    d[0] = ((double)rj[0] - (double)ri[0]) + tx;
    d[1] = ((double)rj[1] - (double)ri[1]) + ty;
    d[2] = ((double)rj[2] - (double)ri[2]) + tz;
    return (d[0] * d[0] + d[1] * d[1]) + d[2] * d[2];
}

static inline int orc_half_keep(int i, int j, const int* S) {
    /* half list: each undirected pair once; i<j, and for self images the
       lexicographically positive shift */
    if (i != j) return i < j;
    if (S[0] != 0) return S[0] > 0;
    if (S[1] != 0) return S[1] > 0;
    return S[2] > 0;
}

/* ------------------------------------------------------------------------------------------
 * brute-force neighbor enumeration: every pair of the same system, every image in range.
 * Writes records (i, j, sx, sy, sz) into out (capacity cap records); returns the total count
 * (which may exceed cap: nothing is written past cap).
 * ---------------------------------------------------------------------------------------- */
ORC_API int64_t orc_nl_brute(const float* pos, const float* cell, const uint8_t* pbc,
                             const int32_t* batch_ptr, int32_t n_systems, double cutoff,
                             int32_t half, int64_t cap, int32_t* out) {
    int64_t total = 0;
    double rc2 = cutoff * cutoff;
    for (int s = 0; s < n_systems; ++s) {
        orc_sys_t sys;
        orc_sys_init(&sys, cell ? cell + 9 * s : NULL, pbc ? pbc + 3 * s : NULL);
        int a0 = batch_ptr[s], a1 = batch_ptr[s + 1];
        int n = a1 - a0;
        int Q[3];
        for (int d = 0; d < 3; ++d)
            Q[d] = sys.per[d] ? (int)floor(cutoff / sys.width[d] * (1.0 + 1e-9)) + 1 : 0;
        int* wrap = (int*)malloc(sizeof(int) * 3 * (n > 0 ? n : 1));
        for (int i = 0; i < n; ++i) {
            double f[3];
            orc_frac(&sys, pos + 3 * (a0 + i), f);
            for (int d = 0; d < 3; ++d) wrap[3 * i + d] = sys.per[d] ? (int)floor(f[d]) : 0;
        }
        for (int i = 0; i < n; ++i) {
            const float* ri = pos + 3 * (a0 + i);
            for (int j = 0; j < n; ++j) {
                const float* rj = pos + 3 * (a0 + j);
                for (int qx = -Q[0]; qx <= Q[0]; ++qx)
                    for (int qy = -Q[1]; qy <= Q[1]; ++qy)
                        for (int qz = -Q[2]; qz <= Q[2]; ++qz) {
                            int S[3];
                            double d[3];
                            S[0] = qx - wrap[3 * j + 0] + wrap[3 * i + 0];
                            S[1] = qy - wrap[3 * j + 1] + wrap[3 * i + 1];
                            S[2] = qz - wrap[3 * j + 2] + wrap[3 * i + 2];
                            if (i == j && S[0] == 0 && S[1] == 0 && S[2] == 0) continue;
                            if (!(orc_pair_d2(ri, rj, S, sys.h, d) < rc2)) continue;
                            if (half && !orc_half_keep(a0 + i, a0 + j, S)) continue;
                            if (total < cap) {
                                int32_t* o = out + 5 * total;
                                o[0] = a0 + i;
                                o[1] = a0 + j;
                                o[2] = S[0];
                                o[3] = S[1];
                                o[4] = S[2];
                            }
                            ++total;
                        }
            }
        }
        free(wrap);
    }
    return total;
}

/* ------------------------------------------------------------------------------------------
 * cell-list neighbor build into the reference's dense layout:
 *   neighbor_matrix (N,K) int32, rows valid in [0, num_neighbors[i]), the rest = fill (N)
 *   num_neighbors   (N)   int32, counts keep running past K (overflow signalling)
 *   shifts          (N,K,3) int32 or NULL
 * Steps: bin (wrapped fractional coordinates; bounding box on non-periodic axes) ->
 * histogram -> exclusive scan -> counting-sort scatter -> stencil search with the exact test.
 * ---------------------------------------------------------------------------------------- */
static inline int orc_floordiv(int a, int b) {
    int q = a / b, r = a % b;
    return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q;
}

ORC_API int32_t orc_nl_cell(const float* pos, const float* cell, const uint8_t* pbc,
                            const int32_t* batch_ptr, int32_t n_systems, double cutoff,
                            int32_t half, int32_t K, int32_t n_total, int32_t* nm, int32_t* nn,
                            int32_t* shifts) {
    double rc2 = cutoff * cutoff;
    double rcb = cutoff * (1.0 + 1.0 / 1024.0); /* binning margin: candidates are a superset */
    for (int64_t t = 0; t < (int64_t)n_total * K; ++t) nm[t] = n_total;
    if (shifts) memset(shifts, 0, sizeof(int32_t) * 3 * (size_t)n_total * K);
    memset(nn, 0, sizeof(int32_t) * (size_t)n_total);

#pragma omp parallel for schedule(dynamic, 1)
    for (int s = 0; s < n_systems; ++s) {
        orc_sys_t sys;
        orc_sys_init(&sys, cell ? cell + 9 * s : NULL, pbc ? pbc + 3 * s : NULL);
        int a0 = batch_ptr[s], a1 = batch_ptr[s + 1];
        int n = a1 - a0;
        if (n <= 0) continue;
        double* fr = (double*)malloc(sizeof(double) * 3 * n);
        int* wrap = (int*)malloc(sizeof(int) * 3 * n);
        double lo[3] = {0, 0, 0}, ext[3] = {1, 1, 1};
        double fmin[3] = {1e300, 1e300, 1e300}, fmax[3] = {-1e300, -1e300, -1e300};
        for (int i = 0; i < n; ++i) {
            orc_frac(&sys, pos + 3 * (a0 + i), fr + 3 * i);
            for (int d = 0; d < 3; ++d) {
                if (fr[3 * i + d] < fmin[d]) fmin[d] = fr[3 * i + d];
                if (fr[3 * i + d] > fmax[d]) fmax[d] = fr[3 * i + d];
            }
        }
        int nc[3], R[3];
        for (int d = 0; d < 3; ++d) {
            if (!sys.per[d]) {
                lo[d] = fmin[d];
                ext[d] = fmax[d] - fmin[d];
                if (!(ext[d] > 0)) ext[d] = 1e-30;
            }
            double span = ext[d] * sys.width[d]; /* perpendicular extent of the binned slab */
            int c = (int)floor(span / rcb);
            if (c < 1) c = 1;
            if (c > 1024) c = 1024;
            nc[d] = c;
        }
        while ((int64_t)nc[0] * nc[1] * nc[2] > (int64_t)(n > 8 ? n : 8)) {
            int m = 0;
            if (nc[1] > nc[m]) m = 1;
            if (nc[2] > nc[m]) m = 2;
            if (nc[m] == 1) break;
            nc[m] = (nc[m] + 1) / 2;
        }
        for (int d = 0; d < 3; ++d) {
            double cw = ext[d] * sys.width[d] / nc[d];
            if (!sys.per[d] && nc[d] == 1) { R[d] = 0; continue; }
            R[d] = (int)ceil(rcb / cw);
            if (!sys.per[d] && R[d] > nc[d] - 1) R[d] = nc[d] - 1;
        }
        int ncell = nc[0] * nc[1] * nc[2];
        int* cid = (int*)malloc(sizeof(int) * n);
        int* start = (int*)calloc((size_t)ncell + 1, sizeof(int));
        int* order = (int*)malloc(sizeof(int) * n);
        for (int i = 0; i < n; ++i) {
            int c[3];
            for (int d = 0; d < 3; ++d) {
                double f = fr[3 * i + d];
                int w = 0;
                if (sys.per[d]) {
                    w = (int)floor(f);
                    f -= (double)w;
                }
                wrap[3 * i + d] = w;
                int b = (int)floor((f - lo[d]) / ext[d] * nc[d]);
                if (b < 0) b = 0;
                if (b > nc[d] - 1) b = nc[d] - 1;
                c[d] = b;
            }
            cid[i] = (c[0] * nc[1] + c[1]) * nc[2] + c[2];
            start[cid[i] + 1]++;
        }
        for (int c = 0; c < ncell; ++c) start[c + 1] += start[c];
        int* fill = (int*)malloc(sizeof(int) * (ncell > 0 ? ncell : 1));
        memcpy(fill, start, sizeof(int) * ncell);
        for (int i = 0; i < n; ++i) order[fill[cid[i]]++] = i;

        for (int i = 0; i < n; ++i) {
            const float* ri = pos + 3 * (a0 + i);
            int ci = cid[i];
            int cz = ci % nc[2], cy = (ci / nc[2]) % nc[1], cx = ci / (nc[2] * nc[1]);
            int count = 0;
            int32_t* row = nm + (int64_t)(a0 + i) * K;
            int32_t* srow = shifts ? shifts + (int64_t)(a0 + i) * K * 3 : NULL;
            for (int ox = -R[0]; ox <= R[0]; ++ox) {
                int gx = cx + ox, qx = 0;
                if (sys.per[0]) { qx = orc_floordiv(gx, nc[0]); gx -= qx * nc[0]; }
                else if (gx < 0 || gx >= nc[0]) continue;
                for (int oy = -R[1]; oy <= R[1]; ++oy) {
                    int gy = cy + oy, qy = 0;
                    if (sys.per[1]) { qy = orc_floordiv(gy, nc[1]); gy -= qy * nc[1]; }
                    else if (gy < 0 || gy >= nc[1]) continue;
                    for (int oz = -R[2]; oz <= R[2]; ++oz) {
                        int gz = cz + oz, qz = 0;
                        if (sys.per[2]) { qz = orc_floordiv(gz, nc[2]); gz -= qz * nc[2]; }
                        else if (gz < 0 || gz >= nc[2]) continue;
                        int c2 = (gx * nc[1] + gy) * nc[2] + gz;
                        for (int t = start[c2]; t < start[c2 + 1]; ++t) {
                            int j = order[t];
                            int S[3];
                            double d[3];
                            S[0] = qx - wrap[3 * j + 0] + wrap[3 * i + 0];
                            S[1] = qy - wrap[3 * j + 1] + wrap[3 * i + 1];
                            S[2] = qz - wrap[3 * j + 2] + wrap[3 * i + 2];
                            if (i == j && S[0] == 0 && S[1] == 0 && S[2] == 0) continue;
                            if (!(orc_pair_d2(ri, pos + 3 * (a0 + j), S, sys.h, d) < rc2))
                                continue;
                            if (half && !orc_half_keep(a0 + i, a0 + j, S)) continue;
                            if (count < K) {
                                row[count] = a0 + j;
                                if (srow) {
                                    srow[3 * count + 0] = S[0];
                                    srow[3 * count + 1] = S[1];
                                    srow[3 * count + 2] = S[2];
                                }
                            }
                            ++count;
                        }
                    }
                }
            }
            nn[a0 + i] = count;
        }
        free(fill); free(order); free(start); free(cid); free(wrap); free(fr);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Lennard-Jones over the dense neighbor matrix.  Pair math in double on the float32 inputs,
 * one rounding to float32 on output (reference: "Internal math is performed in float64",
 * nvalchemi/models/_ops/lj.py:49-50).  Plain truncation at the cutoff, no energy shift.
 *   u(r)  = 4 eps [ (sigma/r)^12 - (sigma/r)^6 ]
 *   e_i   = 1/2 sum_j u(r_ij)         (full list)   -> atomic_energies (N)
 *   F_i   = sum_j u'(r_ij) d_ij / r_ij,  d_ij = r_j - r_i + S.cell
 *   W     = -dE/d(strain) = -1/2 sum_ij u'(r) d (x) d / r   per system, row-major (B,9)
 *   E_sys = fp64 sum over the system's atoms of the float32-rounded e_i, then cast
 *           (nvalchemi/models/lj.py:467-477)
 * Half list: each pair once; e split half/half, force applied to both atoms.
 * ---------------------------------------------------------------------------------------- */
ORC_API int32_t orc_lj_matrix_switched(const float* pos, const float* cells, const int32_t* nm,
                                       const int32_t* shifts, const int32_t* nn, const int32_t* batch_idx,
                                       int32_t n_atoms, int32_t K, int32_t n_systems, int32_t fill_value,
                                       double epsilon, double sigma, double cutoff, double switch_width,
                                       int32_t half, float* atomic_energies, float* forces, float* virials,
                                       float* system_energies);

ORC_API int32_t orc_lj_matrix(const float* pos, const float* cells, const int32_t* nm,
                              const int32_t* shifts, const int32_t* nn, const int32_t* batch_idx,
                              int32_t n_atoms, int32_t K, int32_t n_systems, int32_t fill_value,
                              double epsilon, double sigma, double cutoff, int32_t half,
                              float* atomic_energies, float* forces, float* virials,
                              float* system_energies) {
    return orc_lj_matrix_switched(pos, cells, nm, shifts, nn, batch_idx, n_atoms, K, n_systems, fill_value,
                                  epsilon, sigma, cutoff, 0.0, half, atomic_energies, forces, virials,
                                  system_energies);
}

/* switch_width > 0: u(r) is multiplied by S(t) = 1 - 10 t^3 + 15 t^4 - 6 t^5, t = (r - r_on) / width,
 * r_on = cutoff - width, for r_on < r < cutoff (nvalchemi/models/_ops/lj.py:158-160 describes a
 * "C2-continuous switching region applied between cutoff - switch_width and cutoff"; the polynomial
 * itself is in the absent kernel library: this is the one of least degree with S(0) = 1, S(1) = 0 and
 * zero first and second derivatives at both ends). */
ORC_API int32_t orc_lj_matrix_switched(const float* pos, const float* cells, const int32_t* nm,
                                       const int32_t* shifts, const int32_t* nn, const int32_t* batch_idx,
                                       int32_t n_atoms, int32_t K, int32_t n_systems, int32_t fill_value,
                                       double epsilon, double sigma, double cutoff, double switch_width,
                                       int32_t half, float* atomic_energies, float* forces, float* virials,
                                       float* system_energies) {
    double rc2 = cutoff * cutoff, sig2 = sigma * sigma;
    double r_on = cutoff - switch_width;
    double* e = (double*)calloc((size_t)n_atoms, sizeof(double));
    double* f = (double*)calloc((size_t)n_atoms * 3, sizeof(double));
    double* w = (double*)calloc((size_t)n_systems * 9, sizeof(double));
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        double h[9];
        for (int k = 0; k < 9; ++k) h[k] = (double)cells[9 * s + k];
        int cnt = nn[i] < K ? nn[i] : K;
        for (int k = 0; k < cnt; ++k) {
            int j = nm[(int64_t)i * K + k];
            if (j >= fill_value || j < 0) continue;
            int S[3] = {0, 0, 0};
            double d[3];
            if (shifts) {
                const int32_t* sp = shifts + ((int64_t)i * K + k) * 3;
                S[0] = sp[0]; S[1] = sp[1]; S[2] = sp[2];
            }
            double r2 = orc_pair_d2(pos + 3 * i, pos + 3 * j, S, h, d);
            if (!(r2 < rc2)) continue;
            double ir2 = 1.0 / r2;
            double s2 = sig2 * ir2, s6 = s2 * s2 * s2, s12 = s6 * s6;
            double u = 4.0 * epsilon * (s12 - s6);
            double g = -24.0 * epsilon * (2.0 * s12 - s6) * ir2; /* u'(r)/r */
            if (switch_width > 0.0) {
                double r = sqrt(r2);
                if (r > r_on) {
                    double t = (r - r_on) / switch_width;
                    double S = 1.0 - 10.0 * t * t * t + 15.0 * t * t * t * t - 6.0 * t * t * t * t * t;
                    double dS = (-30.0 * t * t + 60.0 * t * t * t - 30.0 * t * t * t * t) / switch_width;
                    g = g * S + u * dS / r;
                    u = u * S;
                }
            }
            double pf = half ? 1.0 : 0.5;
            if (half) {
                e[i] += 0.5 * u;
                e[j] += 0.5 * u;
                for (int a = 0; a < 3; ++a) { f[3 * i + a] += g * d[a]; f[3 * j + a] -= g * d[a]; }
            } else {
                e[i] += 0.5 * u;
                for (int a = 0; a < 3; ++a) f[3 * i + a] += g * d[a];
            }
            for (int a = 0; a < 3; ++a)
                for (int b = 0; b < 3; ++b) w[9 * s + 3 * a + b] -= pf * g * d[a] * d[b];
        }
    }
    for (int i = 0; i < n_atoms; ++i) {
        atomic_energies[i] = (float)e[i];
        for (int a = 0; a < 3; ++a) forces[3 * i + a] = (float)f[3 * i + a];
    }
    if (virials)
        for (int k = 0; k < 9 * n_systems; ++k) virials[k] = (float)w[k];
    if (system_energies) {
        double* acc = (double*)calloc((size_t)n_systems, sizeof(double));
        for (int i = 0; i < n_atoms; ++i) acc[batch_idx[i]] += (double)atomic_energies[i];
        for (int s = 0; s < n_systems; ++s) system_energies[s] = (float)acc[s];
        free(acc);
    }
    free(e); free(f); free(w);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * BAOAB Langevin half step B-A-O-A (nvalchemi/dynamics/_ops/langevin.py:52-117 documents the
 * splitting; the kernel and its random generator are in the absent library).  float32, one
 * rounding per operation:
 *   v += (F/m)(dt/2) ; r += v (dt/2) ; v = c1 v + c2 xi ; r += v (dt/2)
 *   c1 = exp(-gamma dt), c2 = sqrt((kT/m)(1 - c1^2)) in double, rounded once
 * xi: Philox4x32-10 (Salmon et al., SC'11), key = 64-bit seed, counter = (atom, 0, 0, 0), two
 * Box-Muller pairs in double, the first three deviates used.
 * ---------------------------------------------------------------------------------------- */
ORC_API void orc_philox4x32_10(const uint32_t* counter, const uint32_t* key, uint32_t* out) {
    const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
    uint32_t c0 = counter[0], c1 = counter[1], c2 = counter[2], c3 = counter[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)M0 * c0, p1 = (uint64_t)M1 * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += W0; k1 += W1;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

ORC_API void orc_langevin_normals(uint64_t seed, int32_t atom, double* xi /* 4 */) {
    uint32_t ctr[4] = {(uint32_t)atom, 0u, 0u, 0u};
    uint32_t key[2] = {(uint32_t)(seed & 0xffffffffu), (uint32_t)(seed >> 32)};
    uint32_t w[4];
    orc_philox4x32_10(ctr, key, w);
    for (int p = 0; p < 2; ++p) {
        double u1 = ((double)w[2 * p] + 1.0) * (1.0 / 4294967296.0);
        double u2 = (double)w[2 * p + 1] * (1.0 / 4294967296.0);
        double radius = sqrt(-2.0 * log(u1)), angle = 6.283185307179586476925286766559 * u2;
        xi[2 * p] = radius * cos(angle);
        xi[2 * p + 1] = radius * sin(angle);
    }
}

ORC_API void orc_langevin_half_step(float* pos, float* vel, const float* forces, const float* masses,
                                    const float* dt, const float* kT, const float* friction, uint64_t seed,
                                    const int32_t* batch_idx, const uint8_t* active, int32_t n_atoms) {
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        if (active && !active[s]) continue;
        float m = masses[i], h = dt[s], hh = 0.5f * h;
        double c1d = exp(-(double)friction[s] * (double)h);
        float c1 = (float)c1d;
        float c2 = (float)sqrt(((double)kT[s] / (double)m) * (1.0 - c1d * c1d));
        double xi[4];
        orc_langevin_normals(seed, i, xi);
        for (int a = 0; a < 3; ++a) {
            float v = vel[3 * i + a], r = pos[3 * i + a];
            float acc = forces[3 * i + a] / m;
            float kick = acc * hh;
            v = v + kick;
            float drift = v * hh;
            r = r + drift;
            float damped = c1 * v, noise = c2 * (float)xi[a];
            v = damped + noise;
            drift = v * hh;
            r = r + drift;
            vel[3 * i + a] = v;
            pos[3 * i + a] = r;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * FIRE 2.0, one step on the forces of the current positions (unit masses):
 *   P = sum F.v, VV = sum v.v, FF = sum F.F per system (double)
 *   P > 0 :  a = 1 - alpha, b = alpha sqrt(VV / FF)  (0 when FF <= 1e-20);  count += 1;
 *            count > delaystep:  dt = min(dt dtgrow, tmax), alpha *= alphashrink
 *   P <= 0:  count = 0; alpha = alpha0; back = dt / 2; dt dtshrink >= tmin: dt *= dtshrink;
 *            r -= back v; v = 0
 *   v += dt F;   P > 0: v = a v + b F;   dr = dt v
 *   m = largest |dr_i| of the system;  m > maxstep: dr *= maxstep / m;   r += dr
 * float32 per-atom arithmetic, one rounding per operation; the sums in double.
 * ---------------------------------------------------------------------------------------- */
ORC_API void orc_fire2_step(float* pos, float* vel, const float* forces, const int32_t* batch_idx, float* alpha,
                            float* dt, int32_t* nsteps_inc, float* vf, float* v_sumsq, float* f_sumsq,
                            float* max_norm, int32_t delaystep, double dtgrow, double dtshrink, double alphashrink,
                            double alpha0, double tmax, double tmin, double maxstep, const uint8_t* active,
                            int32_t n_atoms, int32_t n_systems) {
    const size_t M = (size_t)(n_systems > 0 ? n_systems : 1);
    double* acc = (double*)calloc(M * 3, sizeof(double));
    float* mixa = (float*)malloc(sizeof(float) * M);
    float* mixb = (float*)malloc(sizeof(float) * M);
    float* back = (float*)malloc(sizeof(float) * M);
    float* big = (float*)calloc(M, sizeof(float));
    uint8_t* up = (uint8_t*)calloc(M, 1);
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        for (int a = 0; a < 3; ++a) {
            double v = vel[3 * i + a], f = forces[3 * i + a];
            acc[3 * s + 0] += f * v;
            acc[3 * s + 1] += v * v;
            acc[3 * s + 2] += f * f;
        }
    }
    for (int s = 0; s < n_systems; ++s) {
        double P = acc[3 * s], VV = acc[3 * s + 1], FF = acc[3 * s + 2];
        if (vf) vf[s] = (float)P;
        if (v_sumsq) v_sumsq[s] = (float)VV;
        if (f_sumsq) f_sumsq[s] = (float)FF;
        mixa[s] = 1.0f; mixb[s] = 0.0f; back[s] = 0.0f;
        if (active && !active[s]) continue;
        if (P > 0.0) {
            float al = alpha[s];
            up[s] = 1;
            mixa[s] = 1.0f - al;
            mixb[s] = (FF > 1e-20) ? (float)((double)al * sqrt(VV / FF)) : 0.0f;
            nsteps_inc[s] += 1;
            if (nsteps_inc[s] > delaystep) {
                float nd = dt[s] * (float)dtgrow;
                dt[s] = nd < (float)tmax ? nd : (float)tmax;
                alpha[s] = al * (float)alphashrink;
            }
        } else {
            nsteps_inc[s] = 0;
            alpha[s] = (float)alpha0;
            back[s] = 0.5f * dt[s];
            float nd = dt[s] * (float)dtshrink;
            if (nd >= (float)tmin) dt[s] = nd;
        }
    }
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        if (active && !active[s]) continue;
        float h = dt[s], dr[3];
        for (int a = 0; a < 3; ++a) {
            float f = forces[3 * i + a], v = vel[3 * i + a];
            if (!up[s]) {
                float undo = back[s] * v;
                pos[3 * i + a] = pos[3 * i + a] - undo;
                v = 0.0f;
            }
            float kick = h * f;
            v = v + kick;
            if (up[s]) {
                float va = mixa[s] * v, fb = mixb[s] * f;
                v = va + fb;
            }
            v = fminf(fmaxf(v, -ORC_VMAX), ORC_VMAX);
            vel[3 * i + a] = v;
            dr[a] = h * v;
        }
        float top = fmaxf(fmaxf(fabsf(dr[0]), fabsf(dr[1])), fabsf(dr[2]));
        float nrm = 0.0f;
        if (top > 0.0f) {
            float a0 = dr[0] / top, a1 = dr[1] / top, a2 = dr[2] / top;
            nrm = top * sqrtf((a0 * a0 + a1 * a1) + a2 * a2);
        }
        if (nrm > big[s] || nrm != nrm) big[s] = nrm;
    }
    for (int s = 0; s < n_systems; ++s)
        if (max_norm && !(active && !active[s])) max_norm[s] = big[s];
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        if (active && !active[s]) continue;
        float h = dt[s];
        float sc = big[s] > (float)maxstep ? (float)maxstep / big[s] : 1.0f;
        for (int a = 0; a < 3; ++a) {
            float dr = h * vel[3 * i + a];
            dr = dr * sc;
            pos[3 * i + a] = pos[3 * i + a] + dr;
        }
    }
    free(acc); free(mixa); free(mixb); free(back); free(big); free(up);
}

/* ------------------------------------------------------------------------------------------
 * Nose-Hoover chain, half-step propagator of the thermostat (Martyna, Tuckerman, Tobias, Klein 1996).
 * Per system, with KE2 = sum m v^2, N_f degrees of freedom, chain velocities u_k (eta_dot), chain
 * positions eta_k, masses Q_k, and d = w dt for each Suzuki-Yoshida weight w in turn:
 *   u_C   += G_C d/4                    G_1 = (KE2 - N_f kT) / Q_1,  G_k = (Q_{k-1} u_{k-1}^2 - kT) / Q_k
 *   k = C-1 .. 1:  u_k *= exp(-u_{k+1} d/8);  u_k += G_k d/4;  u_k *= exp(-u_{k+1} d/8)
 *   s = exp(-u_1 d/2);  scale *= s;  KE2 *= s^2
 *   eta_k += u_k d/2                    (every k)
 *   k = 1 .. C-1:  u_k *= exp(-u_{k+1} d/8);  u_k += G_k d/4;  u_k *= exp(-u_{k+1} d/8)
 *   u_C   += G_C d/4
 * and finally v *= scale.  Called once before and once after the velocity-Verlet core of a step with
 * the full dt, it advances the thermostat by dt/2 each time.  Chain arithmetic in double on the
 * float32 state, results rounded once when stored; velocities are multiplied by the float32 scale.
 * ---------------------------------------------------------------------------------------- */
static int orc_ys_weights(int order, double* w) {
    if (order == 3) {
        double a = 1.0 / (2.0 - cbrt(2.0));
        w[0] = a; w[1] = 1.0 - 2.0 * a; w[2] = a;
        return 3;
    }
    if (order == 5) {
        double a = 1.0 / (4.0 - cbrt(4.0));
        w[0] = a; w[1] = a; w[2] = 1.0 - 4.0 * a; w[3] = a; w[4] = a;
        return 5;
    }
    w[0] = 1.0;
    return 1;
}

ORC_API void orc_nhc_chain_update(float* vel, const float* masses, float* eta, float* eta_dot, const float* Q,
                                  const float* kT, const float* dt, const float* ndof, float* ke2,
                                  float* total_scale, const int32_t* batch_idx, const uint8_t* active,
                                  int32_t compute_ke, int32_t chain_length, int32_t yoshida_order,
                                  int32_t n_atoms, int32_t n_systems) {
    const int C = chain_length;
    double* sum = (double*)calloc((size_t)(n_systems > 0 ? n_systems : 1), sizeof(double));
    if (compute_ke) {
        for (int i = 0; i < n_atoms; ++i) {
            double vx = vel[3 * i], vy = vel[3 * i + 1], vz = vel[3 * i + 2];
            sum[batch_idx[i]] += (double)masses[i] * ((vx * vx + vy * vy) + vz * vz);
        }
    } else {
        for (int s = 0; s < n_systems; ++s) sum[s] = (double)ke2[s];
    }
    double w[5];
    const int nw = orc_ys_weights(yoshida_order, w);
    for (int s = 0; s < n_systems; ++s) {
        if (active && !active[s]) continue;
        double u[16], x[16], q[16];
        for (int k = 0; k < C; ++k) {
            u[k] = eta_dot[s * C + k];
            x[k] = eta[s * C + k];
            q[k] = Q[s * C + k];
        }
        const double kt = kT[s], nf = ndof[s], h = dt[s];
        double k2 = sum[s], scale = 1.0;
        if (compute_ke) ke2[s] = (float)k2;
        for (int iw = 0; iw < nw; ++iw) {
            const double d = w[iw] * h, d2 = 0.5 * d, d4 = 0.25 * d, d8 = 0.125 * d;
            /* from the end of the chain to the particles */
            {
                double g = (C > 1) ? (q[C - 2] * u[C - 2] * u[C - 2] - kt) / q[C - 1] : (k2 - nf * kt) / q[0];
                u[C - 1] += g * d4;
            }
            for (int k = C - 2; k >= 0; --k) {
                double aa = exp(-d8 * u[k + 1]);
                double g = (k == 0) ? (k2 - nf * kt) / q[0] : (q[k - 1] * u[k - 1] * u[k - 1] - kt) / q[k];
                u[k] = (u[k] * aa + g * d4) * aa;
            }
            {
                double sc = exp(-d2 * u[0]);
                scale *= sc;
                k2 *= sc * sc;
            }
            for (int k = 0; k < C; ++k) x[k] += d2 * u[k];
            /* and back */
            for (int k = 0; k < C - 1; ++k) {
                double aa = exp(-d8 * u[k + 1]);
                double g = (k == 0) ? (k2 - nf * kt) / q[0] : (q[k - 1] * u[k - 1] * u[k - 1] - kt) / q[k];
                u[k] = (u[k] * aa + g * d4) * aa;
            }
            {
                double g = (C > 1) ? (q[C - 2] * u[C - 2] * u[C - 2] - kt) / q[C - 1] : (k2 - nf * kt) / q[0];
                u[C - 1] += g * d4;
            }
        }
        for (int k = 0; k < C; ++k) {
            eta_dot[s * C + k] = (float)u[k];
            eta[s * C + k] = (float)x[k];
        }
        total_scale[s] = (float)scale;
    }
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        if (active && !active[s]) continue;
        float sc = total_scale[s];
        vel[3 * i] *= sc;
        vel[3 * i + 1] *= sc;
        vel[3 * i + 2] *= sc;
    }
    free(sum);
}

/* r += v dt (nvalchemi/dynamics/_ops/nose_hoover.py:291-325) */
ORC_API void orc_nhc_position_update(float* pos, const float* vel, const float* dt, const int32_t* batch_idx,
                                     const uint8_t* active, int32_t n_atoms) {
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        if (active && !active[s]) continue;
        float h = dt[s];
        for (int a = 0; a < 3; ++a) {
            float step = vel[3 * i + a] * h;
            pos[3 * i + a] = pos[3 * i + a] + step;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * velocity Verlet halves, float32, per-system dt (reference docstrings:
 *   r(t+dt) = r + v dt + 1/2 (F/m) dt^2 ;  v(t+dt/2) = v + 1/2 (F/m) dt ;  v(t+dt) = v + 1/2 (F'/m) dt)
 * Association used (each operation rounded once, no fma):
 *   a = F/m ; vh = v + a*(0.5*dt) ; r' = r + vh*dt
 * `active` (n_systems bytes or NULL): systems with 0 are left untouched.
 * ---------------------------------------------------------------------------------------- */
ORC_API void orc_vv_pre(float* pos, float* vel, const float* forces, const float* masses,
                        const float* dt, const int32_t* batch_idx, const uint8_t* active,
                        int32_t n_atoms) {
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        if (active && !active[s]) continue;
        float h = dt[s], hh = 0.5f * h, m = masses[i];
        for (int a = 0; a < 3; ++a) {
            float acc = forces[3 * i + a] / m;
            float kick = acc * hh;
            float vh = vel[3 * i + a] + kick;
            float dr = vh * h;
            vel[3 * i + a] = vh;
            pos[3 * i + a] = pos[3 * i + a] + dr;
        }
    }
}

ORC_API void orc_vv_post(float* vel, const float* forces, const float* masses, const float* dt,
                         const int32_t* batch_idx, const uint8_t* active, int32_t n_atoms) {
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        if (active && !active[s]) continue;
        float hh = 0.5f * dt[s], m = masses[i];
        for (int a = 0; a < 3; ++a) {
            float acc = forces[3 * i + a] / m;
            float kick = acc * hh;
            vel[3 * i + a] = vel[3 * i + a] + kick;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * FIRE step (vanilla branch).  PARITY UNPINNED against the reference: the step itself is in a
 * kernel library that is not in the reference's tree.  The order below is the one the reference's
 * own sentences give, each choice with the sentence that decides it:
 *   1 reductions vf = sum F.v, vv = sum v.v, ff = sum F.F per system over the velocities and
 *     forces AS PASSED IN (double accumulation): nvalchemi/distributed/_dynamics_coordinator.py:
 *     296-322,325-396 computes them before the call from the same arrays and hands them over with
 *     compute_reductions=False as "the ones the op would compute"; _ops/fire.py:317-322.
 *   2 MD integration with the STORED dt: v1 = v + dt F/m (clamped to +-3e38) ; dr = dt v1 ;
 *     |dr| > maxstep -> dr *= maxstep/|dr| per atom ; r += dr.  "Performs an MD integration step
 *     followed by FIRE velocity mixing and adaptive parameter updates" (_ops/fire.py:270-272),
 *     "full FIRE step (MD integration + mixing)" (optimizers/fire.py:31-32); the per-atom clamp:
 *     _dynamics_coordinator.py:329-331.  Semi-implicit Euler (kick, then drift) and the norm of
 *     the clamp are this file's choice: no sentence decides them.
 *   3 mixing with the STORED alpha (test/distributed/test_fire_dd.py:39-50: every atom is meant to
 *     mix with the alpha of before the update):
 *       P >= 0 : v <- (1-alpha) v1 + alpha sqrt(vv/ff) F      P < 0 : v <- 0
 *   4 parameter update:  P >= 0 : n+ += 1 ; if n+ > n_min : dt = min(dt f_inc, dt_max),
 *     alpha *= f_alpha        P < 0 : n+ = 0 ; dt = max(dt f_dec, dt_min) ; alpha = alpha_start
 * Where the zero of P belongs is not said anywhere.  It goes with the downhill branch here
 * because, with the reductions taken at entry and the velocities zeroed after the integration, a
 * system that starts at rest (P = 0 on every entry) would otherwise never gain a velocity.
 * n+ > n_min (rather than >=) is likewise undecided.
 * Every atom of a system uses the same pre-update scalars.  vf/vv/ff outputs are the
 * float32-rounded reductions.  |dr| is evaluated scaled by its largest component, so it cannot
 * overflow.
 * ---------------------------------------------------------------------------------------- */
ORC_API void orc_fire_step(float* pos, float* vel, const float* forces, const float* masses,
                           float* alpha, float* dt, const float* alpha_start,
                           const float* f_alpha, const float* dt_min, const float* dt_max,
                           const float* maxstep, int32_t* n_pos, const int32_t* n_min,
                           const float* f_dec, const float* f_inc, float* vf, float* vv,
                           float* ff, const int32_t* batch_idx, const uint8_t* active,
                           int32_t n_atoms, int32_t n_systems) {
    double* acc = (double*)calloc((size_t)n_systems * 3, sizeof(double));
    float* mixa = (float*)malloc(sizeof(float) * n_systems);
    float* mixb = (float*)malloc(sizeof(float) * n_systems);
    float* dtu = (float*)malloc(sizeof(float) * n_systems);
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        for (int a = 0; a < 3; ++a) {
            double v = vel[3 * i + a], f = forces[3 * i + a];
            acc[3 * s + 0] += f * v;
            acc[3 * s + 1] += v * v;
            acc[3 * s + 2] += f * f;
        }
    }
    for (int s = 0; s < n_systems; ++s) {
        double P = acc[3 * s], VV = acc[3 * s + 1], FF = acc[3 * s + 2];
        vf[s] = (float)P; vv[s] = (float)VV; ff[s] = (float)FF;
        dtu[s] = dt[s]; mixa[s] = 1.0f; mixb[s] = 0.0f;
        if (active && !active[s]) continue;
        if (P >= 0.0) {
            float al = alpha[s];
            mixa[s] = 1.0f - al;
            mixb[s] = (FF > 0.0) ? (float)((double)al * sqrt(VV / FF)) : 0.0f;
            n_pos[s] += 1;
            if (n_pos[s] > n_min[s]) {
                float nd = dt[s] * f_inc[s];
                dt[s] = nd < dt_max[s] ? nd : dt_max[s];
                alpha[s] = al * f_alpha[s];
            }
        } else {
            mixa[s] = 0.0f; mixb[s] = 0.0f;
            n_pos[s] = 0;
            float nd = dt[s] * f_dec[s];
            dt[s] = nd > dt_min[s] ? nd : dt_min[s];
            alpha[s] = alpha_start[s];
        }
    }
    for (int i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        if (active && !active[s]) continue;
        float h = dtu[s], m = masses[i], ms = maxstep[s];
        float dr[3], v[3];
        for (int a = 0; a < 3; ++a) {
            float f = forces[3 * i + a];
            float acc1 = f / m;
            v[a] = vel[3 * i + a] + (h * acc1);
            v[a] = fminf(fmaxf(v[a], -ORC_VMAX), ORC_VMAX); /* keep dr finite */
            dr[a] = h * v[a];
        }
        /* |dr| without overflow: scale by the largest component first */
        float big = fmaxf(fmaxf(fabsf(dr[0]), fabsf(dr[1])), fabsf(dr[2]));
        float nrm = 0.0f;
        if (big > 0.0f) {
            float a0 = dr[0] / big, a1 = dr[1] / big, a2 = dr[2] / big;
            nrm = big * sqrtf((a0 * a0 + a1 * a1) + a2 * a2);
        }
        if (nrm > ms) {
            float sc = ms / nrm;
            for (int a = 0; a < 3; ++a) dr[a] = dr[a] * sc;
        }
        for (int a = 0; a < 3; ++a) {
            float f = forces[3 * i + a];
            vel[3 * i + a] = (mixa[s] * v[a]) + (mixb[s] * f);
            pos[3 * i + a] = pos[3 * i + a] + dr[a];
        }
    }
    free(acc); free(mixa); free(mixb); free(dtu);
}

/* per-system max over atoms of the float32 force norm (reference: vector_norm then
 * scatter amax, nvalchemi/dynamics/base.py:266,336-349); systems with no atoms give -inf */
ORC_API void orc_fmax(const float* forces, const int32_t* batch_idx, int32_t n_atoms,
                      int32_t n_systems, float* fmax) {
    for (int s = 0; s < n_systems; ++s) fmax[s] = -INFINITY;
    for (int i = 0; i < n_atoms; ++i) {
        const float* f = forces + 3 * i;
        float n = sqrtf((f[0] * f[0] + f[1] * f[1]) + f[2] * f[2]);
        int s = batch_idx[i];
        if (n > fmax[s]) fmax[s] = n;
    }
}

ORC_API int32_t orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Verlet-skin displacement test.  flags (M) are cleared, then set for systems holding an atom
 * that moved more than threshold from ref; with cell/pbc the nearest image on periodic axes.
 * With update_reference, ref <- cur for all atoms of flagged systems. */
ORC_API void orc_rebuild_check(float* ref, const float* cur, const int32_t* batch_idx, const float* cell,
                               const uint8_t* pbc, int32_t n_atoms, int32_t n_systems, double threshold,
                               int32_t update_reference, uint8_t* flags) {
    int i, k;
    for (i = 0; i < n_systems; ++i) flags[i] = 0;
    for (i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        double d[3];
        for (k = 0; k < 3; ++k) d[k] = (double)cur[3 * (size_t)i + k] - (double)ref[3 * (size_t)i + k];
        if (cell && pbc && (pbc[3 * s] | pbc[3 * s + 1] | pbc[3 * s + 2])) {
            orc_sys_t sys;
            double f[3];
            orc_sys_init(&sys, cell + 9 * (size_t)s, pbc + 3 * (size_t)s);
            f[0] = (d[0] * sys.hinv[0] + d[1] * sys.hinv[3]) + d[2] * sys.hinv[6];
            f[1] = (d[0] * sys.hinv[1] + d[1] * sys.hinv[4]) + d[2] * sys.hinv[7];
            f[2] = (d[0] * sys.hinv[2] + d[1] * sys.hinv[5]) + d[2] * sys.hinv[8];
            for (k = 0; k < 3; ++k)
                if (sys.per[k]) f[k] -= rint(f[k]);
            for (k = 0; k < 3; ++k) d[k] = (f[0] * sys.h[k] + f[1] * sys.h[3 + k]) + f[2] * sys.h[6 + k];
        }
        if ((d[0] * d[0] + d[1] * d[1]) + d[2] * d[2] > threshold * threshold) flags[s] = 1;
    }
    if (update_reference)
        for (i = 0; i < n_atoms; ++i)
            if (flags[batch_idx[i]])
                for (k = 0; k < 3; ++k) ref[3 * (size_t)i + k] = cur[3 * (size_t)i + k];
}

/* Wrap into the cell: all three fractional coordinates mod 1, back to Cartesian, and of that
 * the components whose own pbc flag is set (the others keep their old value). */
ORC_API void orc_wrap_positions(float* pos, const float* cell, const uint8_t* pbc, const int32_t* batch_idx,
                                int32_t n_atoms) {
    int i, k;
    for (i = 0; i < n_atoms; ++i) {
        int s = batch_idx[i];
        orc_sys_t sys;
        double f[3], w[3];
        if (!(pbc[3 * s] | pbc[3 * s + 1] | pbc[3 * s + 2])) continue;
        orc_sys_init(&sys, cell + 9 * (size_t)s, pbc + 3 * (size_t)s);
        {
            double x = pos[3 * (size_t)i], y = pos[3 * (size_t)i + 1], z = pos[3 * (size_t)i + 2];
            f[0] = (x * sys.hinv[0] + y * sys.hinv[3]) + z * sys.hinv[6];
            f[1] = (x * sys.hinv[1] + y * sys.hinv[4]) + z * sys.hinv[7];
            f[2] = (x * sys.hinv[2] + y * sys.hinv[5]) + z * sys.hinv[8];
        }
        for (k = 0; k < 3; ++k) f[k] -= floor(f[k]);
        for (k = 0; k < 3; ++k) w[k] = (f[0] * sys.h[k] + f[1] * sys.h[3 + k]) + f[2] * sys.h[6 + k];
        for (k = 0; k < 3; ++k)
            if (sys.per[k]) pos[3 * (size_t)i + k] = (float)w[k];
    }
}
