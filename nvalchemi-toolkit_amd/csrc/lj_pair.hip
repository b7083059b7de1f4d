// Lennard-Jones energy / force / virial over the dense neighbor matrix, gfx950.
//
// Reference interface: nvalchemi::lj_energy_forces_batch and
// nvalchemi::lj_energy_forces_virial_batch (nvalchemi/models/_ops/lj.py:116-216,246-321),
// plus the per-system fp64 energy scatter of nvalchemi/models/lj.py:467-477, fused here.
//
// Work decomposition: a workgroup of 512 lanes owns a run of consecutive rows of the matrix and takes
// them one system at a time, with that system's positions staged in LDS when they fit (atom order
// carries no spatial locality); LPR lanes of a wavefront own one row (LPR = 8..64 chosen from the row
// width) and read its indices, and its shifts where they are needed, as 16-byte vectors; the row sum
// is a reduction inside the wavefront.  Where the neighbor list's search radius is below half of
// every perpendicular width of a system's cell, the shifts are not read at all but follow from the
// positions (the listed image of a pair is then the nearest one): 4 instead of 16 bytes per pair.
// Per-system energy and virial go through LDS accumulators and one fp64 atomic per workgroup and
// system.  Pair math is double on the float32 inputs ("internal math is performed in float64",
// nvalchemi/models/_ops/lj.py:49-50).
// Systems too large to stage whole take lj_tiles_kernel instead: it walks the units of the neighbor search again
// and stages each unit's tile, which the build leaves described (nvamd_nl_build_extras).
// Bound: with the shifts read, HBM; with the shifts derived, the double-precision pair arithmetic
// (about 64 vector instructions per pair) and the latency of its operands.
#include <mutex>

#include "common.h"
#include "geom.h"

#ifndef NVAMD_LJ_UNROLL
#define NVAMD_LJ_UNROLL 4
#endif
#ifndef NVAMD_LJ_UNROLL_DERIVED
#define NVAMD_LJ_UNROLL_DERIVED 8
#endif
namespace nvamd {
namespace {

constexpr int kBlock = 256;

struct LjArgs {
    const float* pos;
    const float* cells;
    const int32_t* nm;
    const int32_t* shifts;
    const int32_t* nn;
    const int32_t* bidx;
    int32_t n_atoms, K, n_systems, fill;
    double c4eps, c24eps, sig2, rc2;
    float* e_atom;
    float* forces;
    double* sys_acc;  // (B, 1 + 9): energy then virial, fp64, zeroed before the launch
    unsigned n_blocks;
    int rows_per_block;
    const int32_t* order;      // (N) row k of the kernel's walk is atom order[k]; null: the identity
    const int32_t* sys_first;  // (B) first atom of each non-empty system
    const int32_t* sys_last;   // (B) one past its last atom
    const struct LjSysImage* sys_image;  // (B) how the images of its pairs are found
    int lds_atoms;             // stage positions in LDS when the systems of a run have at most this many atoms
    double list_rc;            // cutoff the neighbor list was built with (0: unknown, shifts are always read)
    double r_on, inv_sw;       // switching region [r_on, cutoff] and 1 / its width (0, 0: no switching)
};

// Switching between r_on and the cutoff: u(r) S(t), t = (r - r_on) / width,
// S = 1 - t^3 (10 - 15 t + 6 t^2): the polynomial of least degree with S(0) = 1, S(1) = 0 and
// vanishing first and second derivatives at both ends (energy, force and force gradient stay
// continuous).  On entry u is the pair energy and gg = u'(r) / r; both are replaced.
__device__ __forceinline__ void apply_switch(const LjArgs& a, double r2, double& u, double& gg) {
    const double r = __builtin_sqrt(r2);
    if (!(r > a.r_on)) return;
    const double t = (r - a.r_on) * a.inv_sw;
    const double omt = 1.0 - t;
    const double S = 1.0 - t * t * t * (10.0 - 15.0 * t + 6.0 * t * t);
    const double dS = -30.0 * t * t * omt * omt * a.inv_sw;
    gg = gg * S + u * dS / r;
    u = u * S;
}

// Sum over the LPR lanes of a row, valid in the row's first lane only.  Steps below 16 lanes are
// data-parallel moves inside a row of 16 lanes (lane i takes lane i + o): no lane numbers to keep in
// registers and no trip through the LDS crossbar.
template <int O>
__device__ __forceinline__ double lane_above(double v) {
    static_assert(O >= 1 && O < 16, "a shift inside a row of 16 lanes");
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), 0x100 + O, 0xf, 0xf, true);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), 0x100 + O, 0xf, 0xf, true);
    return __hiloint2double(hi, lo);
}
template <int LPR>
__device__ __forceinline__ double group_sum(double v) {
    if (LPR > 32) v += __shfl_xor(v, 32, kWave);
    if (LPR > 16) v += __shfl_xor(v, 16, kWave);
    if (LPR > 8) v += lane_above<8>(v);
    if (LPR > 4) v += lane_above<4>(v);
    if (LPR > 2) v += lane_above<2>(v);
    if (LPR > 1) v += lane_above<1>(v);
    return v;
}

constexpr int kSysSlots = 8;      // consecutive systems a workgroup accumulates in LDS
constexpr int kLdsAtoms = 4096;   // positions of this many consecutive atoms fit the LDS stage
constexpr int kBlockFull = 512;   // workgroup size of the full-list kernel
constexpr int kStageLoads = 12;   // loads a thread keeps in flight while it stages positions

// How the images of a system's listed pairs are found.
struct LjSysImage {
    int img;         // 0: read the shifts; 1: shift = -rint((r_j - r_i) . H^-1); 2: the same per component (diagonal cell)
    float hinv[9];   // inverse cell
    double diag[6];  // diagonal of the cell and of its inverse (img == 2)
    int pad[2];
};
static_assert(sizeof(LjSysImage) == 96, "carved from the workspace 96 bytes a system");

// first/last atom of every non-empty system, from the non-decreasing batch_idx; the thread that
// finds a system's first atom also decides how the images of its pairs will be found
__global__ __launch_bounds__(kBlock) void lj_sys_range_kernel(const int32_t* __restrict__ bidx, int n_atoms,
                                                              const float* __restrict__ cells, double list_rc,
                                                              int32_t* __restrict__ first,
                                                              int32_t* __restrict__ last,
                                                              LjSysImage* __restrict__ image,
                                                              double* __restrict__ sys_acc, int n_acc) {
    int i = blockIdx.x * kBlock + threadIdx.x;
    // (the per-system accumulators start at zero: cleared here rather than by a launch of their own)
    if (sys_acc && i < n_acc) sys_acc[i] = 0.0;
    if (i >= n_atoms) return;
    int s = bidx[i];
    if (i == n_atoms - 1 || bidx[i + 1] != s) last[s] = i + 1;
    if (!(i == 0 || bidx[i - 1] != s)) return;
    first[s] = i;
    // shifts need not be read when the list's cutoff is below half of every perpendicular
    // width of the cell (1 / |column of the inverse|): then no pair has two listed images
    LjSysImage im;
    im.img = 0;
    for (int k = 0; k < 9; ++k) im.hinv[k] = 0.f;
    for (int k = 0; k < 6; ++k) im.diag[k] = 0.0;
    im.pad[0] = im.pad[1] = 0;
    if (cells && list_rc > 0.0) {
        const float* c = cells + 9 * (size_t)s;
        double h[9], hv[9];
        for (int k = 0; k < 9; ++k) h[k] = (double)c[k];
        inv3(h, hv);  // (a singular cell gives infinities or NaNs: they fail the test below)
        int ok = 1;
        const double lim = 1.0 / (2.0002 * list_rc);  // |column| must stay below this
        for (int k = 0; k < 3; ++k) {
            const double n2 = hv[k] * hv[k] + hv[3 + k] * hv[3 + k] + hv[6 + k] * hv[6 + k];
            if (!(n2 < lim * lim)) ok = 0;
        }
        for (int k = 0; k < 9; ++k) im.hinv[k] = (float)hv[k];
        if (ok && h[1] == 0.0 && h[2] == 0.0 && h[3] == 0.0 && h[5] == 0.0 && h[6] == 0.0 && h[7] == 0.0) {
            ok = 2;
            for (int k = 0; k < 3; ++k) {
                im.diag[k] = h[4 * k];
                im.diag[3 + k] = hv[4 * k];
            }
        }
        im.img = ok;
    }
    image[s] = im;
}

// One pass over the rows [row0, row_end).  LDS_POS: neighbor positions come from the LDS stage
// (atoms [span0, span0 + span_n)), otherwise from global memory.
// 1/x for a normal, positive x: hardware estimate and two Newton steps (full double
// precision without the scaling and fix-up steps of a general division)
__device__ __forceinline__ double reciprocal(double x) {
    double y = __builtin_amdgcn_rcp(x);
    y = __builtin_fma(y, __builtin_fma(-x, y, 1.0), y);
    y = __builtin_fma(y, __builtin_fma(-x, y, 1.0), y);
    return y;
}

// IMG: the shifts are not read.  Every pair of the list is closer than half of every
// perpendicular width of its cell, so the listed image is the nearest one and its shift is
// -rint((r_j - r_i) . H^-1) (float32 is ample: the listed image's fractional components stay
// below 0.49995 in magnitude).
// energy, force and virial terms of one pair inside the cutoff
template <bool VIRIAL, bool SWITCH>
__device__ __forceinline__ void pair_terms(const LjArgs& a, double r2, double d0, double d1, double d2, double& e,
                                           double& fx, double& fy, double& fz, double& w0, double& w1, double& w2,
                                           double& w3, double& w4, double& w5) {
    // with q6 = (sigma^2 / r^2)^3:  u = 4 eps q6 (q6 - 1),  u'(r)/r = 4 eps q6 (6 - 12 q6) / r^2
    // (one per-launch constant per instruction, the others are literals: nothing to move into vector registers)
    const double ir2 = reciprocal(r2);
    const double q2 = a.sig2 * ir2;
    const double q6 = (q2 * q2) * q2;
    const double aq = a.c4eps * q6;
    double uu = __builtin_fma(aq, q6, -aq);
    double gg = (aq * ir2) * __builtin_fma(q6, -12.0, 6.0);
    if (SWITCH) apply_switch(a, r2, uu, gg);
    e += 0.5 * uu;
    fx += gg * d0;
    fy += gg * d1;
    fz += gg * d2;
    if (VIRIAL) {
        double hg = -0.5 * gg;
        w0 += hg * d0 * d0;
        w1 += hg * d0 * d1;
        w2 += hg * d0 * d2;
        w3 += hg * d1 * d1;
        w4 += hg * d1 * d2;
        w5 += hg * d2 * d2;
    }
}

// IMG == 2: the same for a cell with zero off-diagonal terms, where each component stands alone:
// d_k = dd_k - rint(dd_k / h_kk) h_kk in double (the product is exact, so the fused multiply-add
// rounds exactly like the add of the tabulated shift . cell).
__device__ __forceinline__ double uniform_double(const double* p) {
    const int lo = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int*>(p)[0]);
    const int hi = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int*>(p)[1]);
    return __hiloint2double(hi, lo);
}

template <int LPR, bool VIRIAL, bool SHIFTS, bool SYS, bool LDS_POS, bool VEC, int IMG, bool SWITCH>
__device__ __forceinline__ void lj_rows(const LjArgs& a, int row0, int row_end, int sys_base,
                                        const float* __restrict__ s_pos, int span0, int span_n,
                                        const double (*s_shift)[3], int table_sys, const float* s_hinv,
                                        const double* s_diag, double (*s_acc)[VIRIAL ? 7 : 1]) {
    float hi[9];
    double hd[3], hdi[3];
    if (IMG == 1) {
#pragma unroll
        for (int k = 0; k < 9; ++k)
            hi[k] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(s_hinv[k])));
    }
    if (IMG == 2) {
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            hd[k] = uniform_double(s_diag + k);
            hdi[k] = uniform_double(s_diag + 3 + k);
        }
    }
    // Images derived from the positions (IMG != 0) are only taken on the promise that the matrix is the neighbor
    // build's own (neighbor_list_cutoff > 0): entries below a row's count are then atoms of the row's system and
    // are not checked one by one.
    constexpr bool TRUST = IMG != 0;
    constexpr int G = kBlockFull / LPR;
    const int g = threadIdx.x / LPR;
    const int sub = threadIdx.x % LPR;
    for (int k_row = row0 + g; k_row < row_end; k_row += G) {
        const int i = a.order ? a.order[k_row] : k_row;
        double e = 0.0, fx = 0.0, fy = 0.0, fz = 0.0;
        double w0 = 0.0, w1 = 0.0, w2 = 0.0, w3 = 0.0, w4 = 0.0, w5 = 0.0;  // xx xy xz yy yz zz
        const int sys = a.bidx[i];
        int cnt = a.nn[i];
        cnt = cnt < a.K ? cnt : a.K;
        const float* pi = a.pos + 3 * (size_t)i;
        const float xi = pi[0], yi = pi[1], zi = pi[2];
        // shift . cell comes from the LDS table of the system in hand (shifts of -1, 0, 1) or, for
        // anything else, from the cell in memory: the nine cell components stay out of the registers
        const bool tabled = SHIFTS && sys == table_sys;
        const float* cell_row = SHIFTS ? a.cells + 9 * (size_t)sys : nullptr;
        const int32_t* row = a.nm + (size_t)i * a.K;
        const int32_t* srow = SHIFTS ? a.shifts + (size_t)i * a.K * 3 : nullptr;
        // UNROLL row entries per lane are in flight at once: first every index and shift of the
        // chunk, then every neighbor position, then the arithmetic (the loop is latency bound
        // otherwise: two dependent trips to memory per entry)
        constexpr int UNROLL = (IMG == 2 && VEC) ? NVAMD_LJ_UNROLL_DERIVED : NVAMD_LJ_UNROLL;
        const int last_quad = cnt > 0 ? ((cnt - 1) & ~3) : 0;  // lanes beyond it re-read it: no extra lines
        for (int k0 = 0; k0 < cnt; k0 += UNROLL * LPR) {
            int jj[UNROLL], s0[UNROLL], s1[UNROLL], s2[UNROLL];
            float xj[UNROLL], yj[UNROLL], zj[UNROLL];
            // TRUST: entry u of this lane's chunk is a listed pair iff u < n_mine (the other entries are kept
            // out by this number alone: their indices are never looked at)
            const int n_mine = VEC ? cnt - (k0 + UNROLL * sub) : (cnt - k0 - sub + LPR - 1) / LPR;
            if (VEC) {
                // each lane owns four consecutive entries: one 16-byte load of indices and three
                // of shifts, so a row is read as contiguous 256 + 768 byte runs (K % 4 == 0)
                const int kb = k0 + UNROLL * sub;
#pragma unroll
                for (int v = 0; v < UNROLL / 4; ++v) {
                    const int kv = kb + 4 * v;
                    const int kq = kv < last_quad ? kv : last_quad;  // never past the row's last used quad
                    const int4 j4 = *reinterpret_cast<const int4*>(row + kq);
                    jj[4 * v + 0] = j4.x; jj[4 * v + 1] = j4.y; jj[4 * v + 2] = j4.z; jj[4 * v + 3] = j4.w;
                    if (SHIFTS && IMG == 0) {
                        const int4* sp = reinterpret_cast<const int4*>(srow + 3 * kq);
                        const int4 sa = sp[0], sb = sp[1], sc = sp[2];
                        s0[4 * v + 0] = sa.x; s1[4 * v + 0] = sa.y; s2[4 * v + 0] = sa.z;
                        s0[4 * v + 1] = sa.w; s1[4 * v + 1] = sb.x; s2[4 * v + 1] = sb.y;
                        s0[4 * v + 2] = sb.z; s1[4 * v + 2] = sb.w; s2[4 * v + 2] = sc.x;
                        s0[4 * v + 3] = sc.y; s1[4 * v + 3] = sc.z; s2[4 * v + 3] = sc.w;
                    }
                }
                if (!SHIFTS || IMG != 0) {
#pragma unroll
                    for (int u = 0; u < UNROLL; ++u) s0[u] = s1[u] = s2[u] = 0;
                }
                if (!TRUST) {
#pragma unroll
                    for (int u = 0; u < UNROLL; ++u)
                        if (kb + u >= cnt) jj[u] = -1;
                }
            } else {
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                // clamped, unconditional loads (slot cnt-1 exists): nothing to wait for in between
                const int k = k0 + u * LPR + sub;
                const int kq = k < cnt ? k : cnt - 1;
                jj[u] = row[kq];
                s0[u] = s1[u] = s2[u] = 0;
                if (SHIFTS && IMG == 0) {
                    s0[u] = srow[3 * kq + 0];
                    s1[u] = srow[3 * kq + 1];
                    s2[u] = srow[3 * kq + 2];
                }
                if (!TRUST && k >= cnt) jj[u] = -1;
            }
            }
            if (TRUST && LDS_POS) {
                // indices below the count are atoms of the row's own system (the list is the neighbor
                // build's): the staged span holds them all.  The clamp keeps the reads of the slots
                // beyond the count, and of a list that breaks the promise, inside the stage.
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    unsigned at = (unsigned)(jj[u] - span0);
                    at = at < (unsigned)(span_n - 1) ? at : (unsigned)(span_n - 1);
                    at = __umul24(at, 3u);  // (a full-rate multiply: the stage holds fewer than 2^24 atoms)
                    xj[u] = s_pos[at + 0];
                    yj[u] = s_pos[at + 1];
                    zj[u] = s_pos[at + 2];
                }
            } else if (TRUST) {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    unsigned j = (unsigned)jj[u];
                    j = j < (unsigned)(a.n_atoms - 1) ? j : (unsigned)(a.n_atoms - 1);
                    const float* pj = a.pos + 3 * (size_t)j;
                    xj[u] = pj[0];
                    yj[u] = pj[1];
                    zj[u] = pj[2];
                }
            } else if (LDS_POS) {
                // every lane reads the stage (a neighbor outside the staged span reads the span's first atom for
                // now); the lanes with such a neighbor, if there are any at all, fetch it from memory afterwards
                unsigned outside = 0;
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const bool ok = jj[u] >= 0 && jj[u] < a.fill;
                    const int j = ok ? jj[u] : i;
                    if (!ok) jj[u] = -1;
                    const unsigned rel = (unsigned)(j - span0);
                    const bool in_span = rel < (unsigned)span_n;
                    outside |= in_span ? 0u : (1u << u);
                    const unsigned at = in_span ? rel : 0u;
                    xj[u] = s_pos[3 * at + 0];
                    yj[u] = s_pos[3 * at + 1];
                    zj[u] = s_pos[3 * at + 2];
                }
                if (__builtin_expect(__builtin_amdgcn_ballot_w64(outside != 0) != 0, 0)) {
#pragma unroll
                    for (int u = 0; u < UNROLL; ++u) {
                        if (outside & (1u << u)) {
                            const float* pj = a.pos + 3 * (size_t)(jj[u] >= 0 ? jj[u] : i);
                            xj[u] = pj[0];
                            yj[u] = pj[1];
                            zj[u] = pj[2];
                        }
                    }
                }
            } else {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const bool ok = jj[u] >= 0 && jj[u] < a.fill;
                    const int j = ok ? jj[u] : i;
                    if (!ok) jj[u] = -1;
                    const float* pj = a.pos + 3 * (size_t)j;
                    xj[u] = pj[0];
                    yj[u] = pj[1];
                    zj[u] = pj[2];
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                double t0 = 0.0, t1 = 0.0, t2 = 0.0;
                if (IMG == 2) {
                    double d0, d1, d2;
                    const double r2 = pair_d2_nearest_diagonal(xi, yi, zi, xj[u], yj[u], zj[u], hd, hdi, d0, d1, d2);
                    if (u >= n_mine || !(r2 < a.rc2)) continue;
                    pair_terms<VIRIAL, SWITCH>(a, r2, d0, d1, d2, e, fx, fy, fz, w0, w1, w2, w3, w4, w5);
                    continue;
                }
                if (IMG == 1) {
                    const float dx = xj[u] - xi, dy = yj[u] - yi, dz = zj[u] - zi;
                    s0[u] = -(int)__builtin_rintf(dx * hi[0] + dy * hi[3] + dz * hi[6]);
                    s1[u] = -(int)__builtin_rintf(dx * hi[1] + dy * hi[4] + dz * hi[7]);
                    s2[u] = -(int)__builtin_rintf(dx * hi[2] + dy * hi[5] + dz * hi[8]);
                }
                if (SHIFTS) {
                    const unsigned c0 = (unsigned)(s0[u] + 1), c1 = (unsigned)(s1[u] + 1), c2 = (unsigned)(s2[u] + 1);
                    if (tabled && c0 < 3u && c1 < 3u && c2 < 3u) {
                        const double* t = s_shift[(c0 * 3 + c1) * 3 + c2];
                        t0 = t[0];
                        t1 = t[1];
                        t2 = t[2];
                    } else if (TRUST ? u < n_mine : jj[u] >= 0) {
                        shift_vector(cell_row, s0[u], s1[u], s2[u], t0, t1, t2);
                    }
                }
                double d0, d1, d2;
                double r2 = pair_d2_shifted(xi, yi, zi, xj[u], yj[u], zj[u], t0, t1, t2, d0, d1, d2);
                if ((TRUST ? u >= n_mine : jj[u] < 0) || !(r2 < a.rc2)) continue;
                pair_terms<VIRIAL, SWITCH>(a, r2, d0, d1, d2, e, fx, fy, fz, w0, w1, w2, w3, w4, w5);
            }
        }
        e = group_sum<LPR>(e);
        fx = group_sum<LPR>(fx);
        fy = group_sum<LPR>(fy);
        fz = group_sum<LPR>(fz);
        if (VIRIAL) {
            w0 = group_sum<LPR>(w0);
            w1 = group_sum<LPR>(w1);
            w2 = group_sum<LPR>(w2);
            w3 = group_sum<LPR>(w3);
            w4 = group_sum<LPR>(w4);
            w5 = group_sum<LPR>(w5);
        }
        if (sub == 0) {
            const float ef = (float)e;
            a.e_atom[i] = ef;
            float* fo = a.forces + 3 * (size_t)i;
            fo[0] = (float)fx;
            fo[1] = (float)fy;
            fo[2] = (float)fz;
            if (SYS) {
                // the reference sums the float32-rounded atomic energies in double
                const int slot = sys - sys_base;
                if (slot >= 0 && slot < kSysSlots) {
                    atomicAdd(&s_acc[slot][0], (double)ef);
                    if (VIRIAL) {
                        atomicAdd(&s_acc[slot][1], w0); atomicAdd(&s_acc[slot][2], w1);
                        atomicAdd(&s_acc[slot][3], w2); atomicAdd(&s_acc[slot][4], w3);
                        atomicAdd(&s_acc[slot][5], w4); atomicAdd(&s_acc[slot][6], w5);
                    }
                } else {
                    double* out = a.sys_acc + 10 * (size_t)sys;
                    atomic_add_f64(out + 0, (double)ef);
                    if (VIRIAL) {
                        atomic_add_f64(out + 1, w0); atomic_add_f64(out + 2, w1);
                        atomic_add_f64(out + 3, w2); atomic_add_f64(out + 5, w3);
                        atomic_add_f64(out + 6, w4); atomic_add_f64(out + 9, w5);
                    }
                }
            }
        }
    }
}

template <int LPR, bool VIRIAL, bool SHIFTS, bool SYS, bool VEC, bool SWITCH>
// (six waves per SIMD: three workgroups per CU; the virial variant needs more registers than that leaves)
// What a whole workgroup reads at one address while it finds its system (batch index, walk order, the
// system's range and cell) comes in as read-only arguments of their own: nothing in the kernel can be seen
// to write them, so this chain of dependent loads goes through the scalar cache.
__global__ __launch_bounds__(kBlockFull, (VIRIAL || SWITCH) ? 4 : 6) void lj_matrix_kernel(
    LjArgs a, const int32_t* __restrict__ bidx_ro, const int32_t* __restrict__ order_ro,
    const int32_t* __restrict__ first_ro, const int32_t* __restrict__ last_ro, const float* __restrict__ cells_ro,
    const LjSysImage* __restrict__ image_ro) {
    constexpr int NV = VIRIAL ? 7 : 1;
    __shared__ double s_acc[kSysSlots][NV];
    __shared__ float s_pos[3 * kLdsAtoms];
    __shared__ double s_shift[27][3];  // shift . cell of the system in hand, shifts -1..1 per axis

    // a workgroup owns rows_per_block consecutive rows; workgroups are numbered so that each
    // XCD walks one contiguous eighth of the atoms
    const unsigned lb = xcd_contiguous_block(blockIdx.x, a.n_blocks);
    if (lb >= a.n_blocks) return;
    const int row0 = (int)lb * a.rows_per_block;
    const int row_end = (row0 + a.rows_per_block) < a.n_atoms ? (row0 + a.rows_per_block) : a.n_atoms;
    if (row0 >= row_end) return;
    const int sys_lo = bidx_ro[order_ro ? order_ro[row0] : row0];
    if (SYS && threadIdx.x < kSysSlots * NV) (&s_acc[0][0])[threadIdx.x] = 0.0;

    // Neighbors live in the system of their row: the rows are taken one system at a time, with
    // that system's positions staged in LDS when they fit (atom order carries no spatial
    // locality, so gathers through the caches move a whole line per 12 useful bytes).
    for (int r = row0; r < row_end;) {
        const int sys = bidx_ro[order_ro ? order_ro[r] : r];
        const int span0 = first_ro[sys];
        const int span_end = last_ro[sys];
        const int span_n = span_end - span0;
        // rows of this system inside the block; a batch index that is not sorted (a system in
        // several pieces) makes the range meaningless: then the rest of the block goes unstaged
        const bool range_ok = span0 <= r && r < span_end;
        const int seg_end = (range_ok && span_end < row_end) ? span_end : row_end;
        const bool staged = range_ok && span_n <= a.lds_atoms;
        // (what the set-up of a system derives from the thread's number is worked out again for every
        // system: kept in registers across the rows instead, it is spilled to scratch memory)
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        if (staged) {
            // kStageLoads loads of a thread are in flight together (clamped rather than branched over, so that
            // none of them waits for a condition): a copy with one load outstanding per thread costs a round trip
            // to memory per 512 words, which for a system of a few thousand atoms is most of a workgroup's life
            const float* src = a.pos + 3 * (size_t)span0;
            const int n_words = 3 * span_n;
            for (int base = 0; base < n_words; base += kStageLoads * kBlockFull) {
                float v[kStageLoads];
#pragma unroll
                for (int k = 0; k < kStageLoads; ++k) {
                    const int t = base + k * kBlockFull + tid;
                    v[k] = src[t < n_words ? t : n_words - 1];
                }
#pragma unroll
                for (int k = 0; k < kStageLoads; ++k) {
                    const int t = base + k * kBlockFull + tid;
                    if (t < n_words) s_pos[t] = v[k];
                }
            }
        }
        if (SHIFTS && tid < 27) {
            const int t = tid;
            shift_vector(cells_ro + 9 * (size_t)sys, t / 9 - 1, (t / 3) % 3 - 1, t % 3 - 1, s_shift[t][0], s_shift[t][1],
                         s_shift[t][2]);
        }
        __syncthreads();
        // (whether this system's shifts follow from the positions alone was decided with its range)
        const LjSysImage& image = image_ro[sys];
        const int img = SHIFTS ? image.img : 0;
        const float* s_hinv = image.hinv;
        const double* s_diag = image.diag;
#define NVAMD_LJ_ROWS(STAGED, IMG)                                                                              \
    lj_rows<LPR, VIRIAL, SHIFTS, SYS, STAGED, VEC, (SHIFTS ? IMG : 0), SWITCH>(                                  \
        a, r, seg_end, sys_lo, s_pos, STAGED ? span0 : 0, STAGED ? span_n : 0, s_shift, sys, s_hinv, s_diag, s_acc)
        if (staged) {
            if (img == 2) NVAMD_LJ_ROWS(true, 2);
            else if (img == 1) NVAMD_LJ_ROWS(true, 1);
            else NVAMD_LJ_ROWS(true, 0);
        } else {
            if (img == 2) NVAMD_LJ_ROWS(false, 2);
            else if (img == 1) NVAMD_LJ_ROWS(false, 1);
            else NVAMD_LJ_ROWS(false, 0);
        }
#undef NVAMD_LJ_ROWS
        r = seg_end;
        if (r < row_end) __syncthreads();  // the stage is about to be overwritten
    }

    if (SYS) {
        __syncthreads();
        if (threadIdx.x < kSysSlots * NV) {
            const int slot = threadIdx.x / NV, k = threadIdx.x % NV;
            const double v = s_acc[slot][k];
            if (v != 0.0 && sys_lo + slot < a.n_systems) {
                // k: 0 energy, 1..6 the upper triangle xx xy xz yy yz zz of the virial
                const int where = (k == 0) ? 0 : (k <= 3 ? k : (k <= 5 ? k + 1 : 9));
                atomic_add_f64(a.sys_acc + 10 * (size_t)(sys_lo + slot) + where, v);
            }
        }
    }
}

// ---- systems too large to stage: the tiles of the neighbor search, walked again ---------------------------
// The neighbor search (nvamd_nl_build_tiles) handles a unit of work, the atoms of a short run of cells, against one
// tile: the atoms of the run's stencil cells in a fixed order in LDS.  It leaves behind the atoms' coordinates in
// cell order, per unit a record that lays the tile out as slices of that order, and per listed pair the place of
// the neighbor in the tile (16 bits).  A workgroup here takes a few consecutive units, copies their tiles into LDS
// with contiguous reads, and the pair arithmetic finds every neighbor there by its tile index: no gather from
// memory per pair (a cache line for twelve bytes, from all over the array, when atom numbers carry no locality).
constexpr int kTileUnits = 4;        // consecutive units a workgroup takes at a time (about three rounds of 64 rows)
constexpr int kTilePool = 4096;      // atoms of their tiles staged at a time (48 KB)
constexpr int kTileCells = 64;       // stencil cells in a unit's record
constexpr int kTileRecord = NVAMD_NL_TILE_RECORD_INTS / 2;  // 8-byte words per record
static_assert(kTileRecord == 2 + kTileCells, "two words of header, one per stencil cell");
static_assert(NVAMD_NL_TILE_ATOMS <= kTilePool, "one tile always fits the pool");

struct LjTiles {
    const uint16_t* index;   // (N, K)
    const float4* xyz;       // (N) cell order
    const int2* records;     // (units, kTileRecord)
    const int32_t* count;    // (1)
    int capacity;            // records that the table has room for
};

// rows [0, n_rows) of the staged units: row rr belongs to staged unit q with s_row0[q] <= rr < s_row0[q + 1]
template <bool VIRIAL, bool SYS, int IMG>
__device__ __forceinline__ void lj_tile_rows(const LjArgs& a, const LjTiles& t, int n_rows, const int4* s_unit,
                                             const int* s_row0, const int* s_tile0, const float* __restrict__ s_pos,
                                             const double (*s_shift)[3], const float* cells_sys, const float* s_hinv,
                                             const double* s_diag, int sys, int sys_base,
                                             double (*s_acc)[VIRIAL ? 7 : 1]) {
    constexpr int LPR = 8, G = kBlockFull / LPR, UNROLL = 8;
    float hi[9];
    double hd[3], hdi[3];
    if (IMG == 1) {
#pragma unroll
        for (int k = 0; k < 9; ++k) hi[k] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(s_hinv[k])));
    }
    if (IMG == 2) {
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            hd[k] = uniform_double(s_diag + k);
            hdi[k] = uniform_double(s_diag + 3 + k);
        }
    }
    const int g = threadIdx.x / LPR, sub = threadIdx.x % LPR;
    for (int rr = g; rr < n_rows; rr += G) {
        int q = 0;
#pragma unroll
        for (int k = 1; k < kTileUnits; ++k) q += rr >= s_row0[k] ? 1 : 0;
        const int4 un = s_unit[q];  // first row, rows, system, atoms in the tile (or -1)
        const float4 me = t.xyz[un.x + (rr - s_row0[q])];
        const int i = __float_as_int(me.w);
        const float xi = me.x, yi = me.y, zi = me.z;
        int cnt = a.nn[i];
        cnt = cnt < a.K ? cnt : a.K;
        const bool tiled = un.w > 0;
        const int tile_last = tiled ? un.w - 1 : 0, tile0 = s_tile0[q];
        const uint16_t* trow = t.index + (size_t)i * a.K;
        const int32_t* row = a.nm + (size_t)i * a.K;
        const int last_oct = cnt > 0 ? ((cnt - 1) & ~7) : 0;  // lanes beyond it re-read it: no extra lines
        double e = 0.0, fx = 0.0, fy = 0.0, fz = 0.0;
        double w0 = 0.0, w1 = 0.0, w2 = 0.0, w3 = 0.0, w4 = 0.0, w5 = 0.0;
        for (int k0 = 0; k0 < cnt; k0 += UNROLL * LPR) {
            const int kb = k0 + UNROLL * sub;
            const int n_mine = cnt - kb;  // entry u of this lane's eight is a listed pair iff u < n_mine
            const int kq = kb < last_oct ? kb : last_oct;
            float xj[UNROLL], yj[UNROLL], zj[UNROLL];
            if (__builtin_expect(tiled, 1)) {
                const int4 w = *reinterpret_cast<const int4*>(trow + kq);
                const unsigned packed[4] = {(unsigned)w.x, (unsigned)w.y, (unsigned)w.z, (unsigned)w.w};
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    // (the clamp keeps the reads of the slots beyond the count inside the tile)
                    int at = (int)((u & 1) ? packed[u / 2] >> 16 : packed[u / 2] & 0xffffu);
                    at = at < tile_last ? at : tile_last;
                    at = (int)__umul24((unsigned)(at + tile0), 3u);
                    xj[u] = s_pos[at + 0];
                    yj[u] = s_pos[at + 1];
                    zj[u] = s_pos[at + 2];
                }
            } else {
                // a unit whose stencil is not one tile: its neighbors come from memory
                const int4 ja = *reinterpret_cast<const int4*>(row + kq), jb = *reinterpret_cast<const int4*>(row + kq + 4);
                const int jj[UNROLL] = {ja.x, ja.y, ja.z, ja.w, jb.x, jb.y, jb.z, jb.w};
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    unsigned j = (unsigned)jj[u];
                    j = j < (unsigned)(a.n_atoms - 1) ? j : (unsigned)(a.n_atoms - 1);
                    const float* pj = a.pos + 3 * (size_t)j;
                    xj[u] = pj[0];
                    yj[u] = pj[1];
                    zj[u] = pj[2];
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                double d0, d1, d2, r2;
                if (IMG == 2) {
                    r2 = pair_d2_nearest_diagonal(xi, yi, zi, xj[u], yj[u], zj[u], hd, hdi, d0, d1, d2);
                } else {
                    const float dx = xj[u] - xi, dy = yj[u] - yi, dz = zj[u] - zi;
                    const int s0 = -(int)__builtin_rintf(dx * hi[0] + dy * hi[3] + dz * hi[6]);
                    const int s1 = -(int)__builtin_rintf(dx * hi[1] + dy * hi[4] + dz * hi[7]);
                    const int s2 = -(int)__builtin_rintf(dx * hi[2] + dy * hi[5] + dz * hi[8]);
                    const unsigned c0 = (unsigned)(s0 + 1), c1 = (unsigned)(s1 + 1), c2 = (unsigned)(s2 + 1);
                    double t0 = 0.0, t1 = 0.0, t2 = 0.0;
                    if (c0 < 3u && c1 < 3u && c2 < 3u) {
                        const double* tv = s_shift[(c0 * 3 + c1) * 3 + c2];
                        t0 = tv[0];
                        t1 = tv[1];
                        t2 = tv[2];
                    } else if (u < n_mine) {
                        shift_vector(cells_sys, s0, s1, s2, t0, t1, t2);
                    }
                    r2 = pair_d2_shifted(xi, yi, zi, xj[u], yj[u], zj[u], t0, t1, t2, d0, d1, d2);
                }
                if (u >= n_mine || !(r2 < a.rc2)) continue;
                pair_terms<VIRIAL, false>(a, r2, d0, d1, d2, e, fx, fy, fz, w0, w1, w2, w3, w4, w5);
            }
        }
        e = group_sum<LPR>(e);
        fx = group_sum<LPR>(fx);
        fy = group_sum<LPR>(fy);
        fz = group_sum<LPR>(fz);
        if (VIRIAL) {
            w0 = group_sum<LPR>(w0); w1 = group_sum<LPR>(w1); w2 = group_sum<LPR>(w2);
            w3 = group_sum<LPR>(w3); w4 = group_sum<LPR>(w4); w5 = group_sum<LPR>(w5);
        }
        if (sub == 0) {
            const float ef = (float)e;
            a.e_atom[i] = ef;
            float* fo = a.forces + 3 * (size_t)i;
            fo[0] = (float)fx;
            fo[1] = (float)fy;
            fo[2] = (float)fz;
            if (SYS) {
                const int slot = sys - sys_base;
                if (slot >= 0 && slot < kSysSlots) {
                    atomicAdd(&s_acc[slot][0], (double)ef);
                    if (VIRIAL) {
                        atomicAdd(&s_acc[slot][1], w0); atomicAdd(&s_acc[slot][2], w1);
                        atomicAdd(&s_acc[slot][3], w2); atomicAdd(&s_acc[slot][4], w3);
                        atomicAdd(&s_acc[slot][5], w4); atomicAdd(&s_acc[slot][6], w5);
                    }
                } else {
                    double* out = a.sys_acc + 10 * (size_t)sys;
                    atomic_add_f64(out + 0, (double)ef);
                    if (VIRIAL) {
                        atomic_add_f64(out + 1, w0); atomic_add_f64(out + 2, w1);
                        atomic_add_f64(out + 3, w2); atomic_add_f64(out + 5, w3);
                        atomic_add_f64(out + 6, w4); atomic_add_f64(out + 9, w5);
                    }
                }
            }
        }
    }
}

template <bool VIRIAL, bool SYS>
__global__ __launch_bounds__(kBlockFull, VIRIAL ? 4 : 6) void lj_tiles_kernel(
    LjArgs a, LjTiles t, const int2* __restrict__ records_ro, const int32_t* __restrict__ count_ro,
    const float* __restrict__ cells_ro, const LjSysImage* __restrict__ image_ro) {
    constexpr int NV = VIRIAL ? 7 : 1;
    __shared__ double s_acc[kSysSlots][NV];
    __shared__ float s_pos[3 * kTilePool];
    __shared__ int2 s_cells[kTileUnits][kTileCells];  // per stencil cell: first slot of the cell order, offset in the tile
    __shared__ int4 s_unit[kTileUnits];               // first row, rows, system, atoms in the tile (or -1)
    __shared__ int4 s_staged[kTileUnits];             // the units staged together, renumbered from 0
    __shared__ int s_row0[kTileUnits + 1];            // their first rows in the numbering of the rounds
    __shared__ int s_tile0[kTileUnits + 1];           // where their tiles begin in the pool
    __shared__ int s_plan[2];                         // how many units are staged together, and the system they share
    __shared__ double s_shift[27][3];

    // units are dealt to the 8 XCDs in contiguous eighths (consecutive workgroups go to the XCDs round-robin), so
    // that the slices of the cell order that neighboring tiles share stay in one L2
    // (a count that the table cannot hold is not this build's: nothing past the table is read)
    const int counted = count_ro[0];
    const int total = counted < 0 ? 0 : (counted < t.capacity ? counted : t.capacity);
    const int n_groups = (total + kTileUnits - 1) / kTileUnits;
    const int per_xcd = (n_groups + 7) / 8;
    const int xcd = blockIdx.x % 8, slot0 = blockIdx.x / 8, stride = gridDim.x / 8;
    if (SYS && threadIdx.x < kSysSlots * NV) (&s_acc[0][0])[threadIdx.x] = 0.0;

    for (int gs = slot0; gs < per_xcd; gs += stride) {
        // NOTE: every thread of the workgroup takes the same path through this loop body
        const int grp = xcd * per_xcd + gs;
        if (grp >= n_groups) break;
        const int u0 = grp * kTileUnits;
        const int nq = (total - u0) < kTileUnits ? (total - u0) : kTileUnits;
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        {
            const int q = tid / kTileCells, c = tid % kTileCells;
            if (q < nq) {
                const int2* rec = records_ro + (size_t)(u0 + q) * kTileRecord;
                const int2 rows = rec[0], what = rec[1];
                if (c == 0) s_unit[q] = make_int4(rows.x, rows.y, what.x, rows.y > 0 ? what.y : -1);
                if (what.y > 0) s_cells[q][c] = rec[2 + c];
            }
        }
        __syncthreads();
        const int sys_base = s_unit[0].z;
        for (int q0 = 0; q0 < nq;) {
            // units staged together: consecutive ones of one system whose tiles fit the pool
            if (tid == 0) {
                const int sys = s_unit[q0].z;
                int q1 = q0, atoms = 0, rows = 0;
                while (q1 < nq && s_unit[q1].z == sys) {
                    const int4 un = s_unit[q1];
                    const int n = un.w > 0 ? un.w : 0;
                    if (atoms + n > kTilePool) break;
                    s_staged[q1 - q0] = un;
                    s_row0[q1 - q0] = rows;
                    s_tile0[q1 - q0] = atoms;
                    atoms += n;
                    rows += un.y;
                    ++q1;
                }
                for (int k = q1 - q0; k <= kTileUnits; ++k) {
                    s_row0[k] = k == q1 - q0 ? rows : 0x7fffffff;
                    s_tile0[k] = atoms;
                }
                s_plan[0] = q1 - q0;
                s_plan[1] = sys;
            }
            if (tid < 27) {
                const int sys = s_unit[q0].z;
                shift_vector(cells_ro + 9 * (size_t)sys, tid / 9 - 1, (tid / 3) % 3 - 1, tid % 3 - 1, s_shift[tid][0],
                             s_shift[tid][1], s_shift[tid][2]);
            }
            __syncthreads();
            const int n_staged = s_plan[0], sys = s_plan[1];
            const int n_rows = s_row0[n_staged], n_pool = s_tile0[n_staged];
            // ---- the tiles into the pool: thread t takes atoms t, t + 512, ... of the pool, kTileLoads loads in flight
            constexpr int kTileLoads = 4;
            for (int base = 0; base < n_pool; base += kTileLoads * kBlockFull) {
                float4 p[kTileLoads];
#pragma unroll
                for (int k = 0; k < kTileLoads; ++k) {
                    const int at = base + k * kBlockFull + tid;
                    const int f_all = at < n_pool ? at : n_pool - 1;
                    int q = 0;
#pragma unroll
                    for (int m = 1; m < kTileUnits; ++m) q += f_all >= s_tile0[m] ? 1 : 0;
                    const int f = f_all - s_tile0[q];
                    const int2* cells = s_cells[q0 + q];
                    int c = 0;  // the stencil cell that holds atom f of the tile
#pragma unroll
                    for (int step = kTileCells / 2; step > 0; step >>= 1)
                        if (cells[c + step].y <= f) c += step;
                    p[k] = t.xyz[cells[c].x + (f - cells[c].y)];
                }
#pragma unroll
                for (int k = 0; k < kTileLoads; ++k) {
                    const int at = base + k * kBlockFull + tid;
                    if (at < n_pool) {
                        s_pos[3 * at + 0] = p[k].x;
                        s_pos[3 * at + 1] = p[k].y;
                        s_pos[3 * at + 2] = p[k].z;
                    }
                }
            }
            __syncthreads();
            const LjSysImage& image = image_ro[sys];
            const int img = image.img;
            if (img == 2) {
                lj_tile_rows<VIRIAL, SYS, 2>(a, t, n_rows, s_staged, s_row0, s_tile0, s_pos, s_shift,
                                             cells_ro + 9 * (size_t)sys, image.hinv, image.diag, sys, sys_base, s_acc);
            } else if (img == 1) {
                lj_tile_rows<VIRIAL, SYS, 1>(a, t, n_rows, s_staged, s_row0, s_tile0, s_pos, s_shift,
                                             cells_ro + 9 * (size_t)sys, image.hinv, image.diag, sys, sys_base, s_acc);
            } else {
                // a cell too narrow for derived images: the shifts are read, the neighbors come from memory
                for (int q = 0; q < n_staged; ++q) {
                    const int4 un = s_staged[q];
                    lj_rows<8, VIRIAL, true, SYS, false, true, 0, false>(a, un.x, un.x + un.y, sys_base, nullptr, 0, 0,
                                                                         s_shift, sys, image.hinv, image.diag, s_acc);
                }
            }
            __syncthreads();  // (the pool and the plan are rewritten next)
            q0 += n_staged;
        }
        if (SYS) {
            // (the systems of the next units may be others: the sums of these go out now)
            if (threadIdx.x < kSysSlots * NV) {
                const int slot = threadIdx.x / NV, k = threadIdx.x % NV;
                const double v = s_acc[slot][k];
                if (v != 0.0 && sys_base + slot < a.n_systems) {
                    const int where = (k == 0) ? 0 : (k <= 3 ? k : (k <= 5 ? k + 1 : 9));
                    atomic_add_f64(a.sys_acc + 10 * (size_t)(sys_base + slot) + where, v);
                }
                s_acc[slot][k] = 0.0;
            }
            __syncthreads();
        }
    }
}

// Half list: each pair once, both atoms updated.  Accumulates in fp64 scratch through
// atomics; one lane per row.  Not tuned: the reference's LJ default is the full list
// (nvalchemi/models/lj.py:115).
struct LjHalfArgs {
    LjArgs a;
    double* atom_acc;  // (N,4): e, fx, fy, fz
};

template <bool VIRIAL, bool SHIFTS>
__global__ __launch_bounds__(kBlock) void lj_half_kernel(LjHalfArgs p) {
    const LjArgs& a = p.a;
    int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.n_atoms) return;
    int sys = a.bidx[i];
    int cnt = a.nn[i];
    cnt = cnt < a.K ? cnt : a.K;
    const float* pi = a.pos + 3 * (size_t)i;
    double h[9];
    const float* c = a.cells + 9 * (size_t)sys;
    for (int k = 0; k < 9; ++k) h[k] = SHIFTS ? (double)c[k] : 0.0;
    double e = 0, fx = 0, fy = 0, fz = 0, w[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (int k = 0; k < cnt; ++k) {
        int j = a.nm[(size_t)i * a.K + k];
        if (j < 0 || j >= a.fill) continue;
        int s0 = 0, s1 = 0, s2 = 0;
        if (SHIFTS) {
            const int32_t* sp = a.shifts + ((size_t)i * a.K + k) * 3;
            s0 = sp[0]; s1 = sp[1]; s2 = sp[2];
        }
        const float* pj = a.pos + 3 * (size_t)j;
        double d[3];
        double r2 = pair_d2_exact(pi[0], pi[1], pi[2], pj[0], pj[1], pj[2], s0, s1, s2, h, d[0], d[1], d[2]);
        if (!(r2 < a.rc2)) continue;
        double ir2 = 1.0 / r2;
        double q2 = a.sig2 * ir2, q6 = q2 * q2 * q2, q12 = q6 * q6;
        double u = a.c4eps * (q12 - q6);
        double gg = -(a.c24eps * (2.0 * q12 - q6)) * ir2;
        if (a.inv_sw > 0.0) apply_switch(a, r2, u, gg);
        e += 0.5 * u;
        fx += gg * d[0]; fy += gg * d[1]; fz += gg * d[2];
        double* aj = p.atom_acc + 4 * (size_t)j;
        atomic_add_f64(aj + 0, 0.5 * u);
        atomic_add_f64(aj + 1, -gg * d[0]);
        atomic_add_f64(aj + 2, -gg * d[1]);
        atomic_add_f64(aj + 3, -gg * d[2]);
        if (VIRIAL)
            for (int x = 0; x < 3; ++x)
                for (int y = 0; y < 3; ++y) w[3 * x + y] -= gg * d[x] * d[y];
    }
    double* ai = p.atom_acc + 4 * (size_t)i;
    atomic_add_f64(ai + 0, e);
    atomic_add_f64(ai + 1, fx);
    atomic_add_f64(ai + 2, fy);
    atomic_add_f64(ai + 3, fz);
    if (VIRIAL && a.sys_acc)
        for (int k = 0; k < 9; ++k)
            if (w[k] != 0.0) atomic_add_f64(a.sys_acc + 10 * (size_t)sys + 1 + k, w[k]);
}

__global__ __launch_bounds__(kBlock) void lj_half_finish_kernel(const double* __restrict__ atom_acc,
                                                                const int32_t* __restrict__ bidx,
                                                                float* __restrict__ e_atom,
                                                                float* __restrict__ forces,
                                                                double* __restrict__ sys_acc,
                                                                int n_atoms) {
    int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const double* ai = atom_acc + 4 * (size_t)i;
    float ef = (float)ai[0];
    e_atom[i] = ef;
    forces[3 * (size_t)i + 0] = (float)ai[1];
    forces[3 * (size_t)i + 1] = (float)ai[2];
    forces[3 * (size_t)i + 2] = (float)ai[3];
    if (sys_acc) atomic_add_f64(sys_acc + 10 * (size_t)bidx[i], (double)ef);
}

__global__ __launch_bounds__(kBlock) void clear_f64_kernel(double* p, size_t n) {
    size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t < n) p[t] = 0.0;
}

// The per-system sums leave as float32 (the symmetric half of the virial was accumulated: it is mirrored), and the
// accumulators go back to zero, so that a call that reuses the workspace's tables (and with them skips the kernel
// that clears the accumulators) starts from zero.
__global__ __launch_bounds__(kBlock) void lj_sys_finish_clear_kernel(double* __restrict__ sys_acc,
                                                                     float* __restrict__ sys_e,
                                                                     float* __restrict__ virials, int m) {
    __shared__ double s_v[kBlock / 10 * 10];
    // a workgroup takes whole systems (25 of them): the mirrored reads stay inside its own slice
    constexpr int kPer = kBlock / 10;
    const int s0 = (int)blockIdx.x * kPer;
    const int t = (int)threadIdx.x;
    const bool on = t < kPer * 10 && s0 + t / 10 < m;
    const size_t at = 10 * (size_t)s0 + (size_t)t;
    double v = 0.0;
    if (on) {
        v = sys_acc[at];
        s_v[t] = v;
    }
    __syncthreads();
    if (!on) return;
    sys_acc[at] = 0.0;
    const int s = s0 + t / 10, k = t % 10;
    if (k == 0) {
        if (sys_e) sys_e[s] = (float)v;
    } else if (virials) {
        const int c = k - 1;
        const int r = c / 3, q = c % 3;
        if (r > q) v = s_v[t - k + 1 + 3 * q + r];
        virials[9 * (size_t)s + c] = (float)v;
    }
}

template <int LPR>
void launch_full(const LjArgs& a, bool virial, bool shifts, bool sys, hipStream_t st) {
    constexpr int G = kBlockFull / LPR;
    LjArgs b = a;
    // a workgroup owns a run of consecutive rows: long enough to amortise the staging of its
    // systems' positions and to keep per-system sums in LDS, short enough to fill the chip
    int rows = 512;
    while (rows > 4 * G && (a.n_atoms + rows - 1) / rows < 256 * 6) rows /= 2;
    // a batch that still leaves most of the chip idle: shorter runs, down to one pass of the workgroup, until there
    // are three workgroups for every two CUs (measured on batches of 4 000 to 500 000 atoms: 23 -> 12 us at 4 000
    // atoms, 25 -> 18 us at 32 000; from 128 000 atoms on the runs above are as fast or faster)
    while (rows > G && (a.n_atoms + rows - 1) / rows < 384) rows /= 2;
    rows = (rows + G - 1) / G * G;
    // With work for more than two rounds of resident workgroups (three per CU, two with the virial) and systems
    // small enough to be staged, equal shares for a whole number of rounds: the last round is then as full as the
    // others, and longer runs stage their systems' positions less often (2 % on 256 boxes of 3900 atoms; for one
    // large system, whose positions are not staged, it is 1 % slower and is left alone).
    const long long slots = 256LL * ((virial || a.inv_sw > 0.0) ? 2 : 3);
    const long long rounds = (long long)a.n_atoms / (slots * 512);
    if (rounds >= 2 && a.n_systems > 0 && a.n_atoms / a.n_systems <= a.lds_atoms) {
        // shares for that number of rounds or for one more, whichever leaves the last round fuller: the time goes as
        // (rounds actually needed) x (rows + what a workgroup spends before its first row, about 21 rows' worth:
        // 256 boxes of 3900 atoms take 0.132 ms with 704 rows in two rounds, 0.128 ms with 448 rows in three)
        long long best = -1;
        for (long long r = rounds; r <= rounds + 1; ++r) {
            const long long share = ((long long)a.n_atoms + slots * r - 1) / (slots * r);
            const long long rr = (share + G - 1) / G * G;
            const long long blocks = ((long long)a.n_atoms + rr - 1) / rr;
            const long long cost = ((blocks + slots - 1) / slots) * (rr + 21);
            if (best < 0 || cost < best) {
                best = cost;
                rows = (int)rr;
            }
        }
    }
    b.rows_per_block = rows;
    b.n_blocks = (unsigned)((a.n_atoms + rows - 1) / rows);
    unsigned per = (b.n_blocks + 7) / 8;
    dim3 grid(per * 8), blk(kBlockFull);
    // 16-byte row loads need aligned rows: K a multiple of 4 and aligned base pointers
    const bool vec = a.K >= 4 && a.K % 4 == 0 && aligned16(a.nm) && (!a.shifts || aligned16(a.shifts));
    const bool sw = a.inv_sw > 0.0;
#define NVAMD_LJ_LAUNCH(V, S, Y, W)                                                                  \
    {                                                                                                \
        if (vec) hipLaunchKernelGGL((lj_matrix_kernel<LPR, V, S, Y, true, W>), grid, blk, 0, st, b, b.bidx, b.order, b.sys_first, b.sys_last, b.cells, b.sys_image); \
        else hipLaunchKernelGGL((lj_matrix_kernel<LPR, V, S, Y, false, W>), grid, blk, 0, st, b, b.bidx, b.order, b.sys_first, b.sys_last, b.cells, b.sys_image);    \
        return;                                                                                      \
    }
#define NVAMD_LJ_CASE(V, S, Y)                                                                 \
    if (virial == V && shifts == S && sys == Y) {                                              \
        if (sw) NVAMD_LJ_LAUNCH(V, S, Y, true) else NVAMD_LJ_LAUNCH(V, S, Y, false)            \
    }
    NVAMD_LJ_CASE(false, false, false)
    NVAMD_LJ_CASE(false, false, true)
    NVAMD_LJ_CASE(false, true, false)
    NVAMD_LJ_CASE(false, true, true)
    NVAMD_LJ_CASE(true, false, true)
    NVAMD_LJ_CASE(true, true, true)
#undef NVAMD_LJ_CASE
#undef NVAMD_LJ_LAUNCH
}

int lanes_per_row(int K) {
    if (K <= 384) return 8;  // (rows are much shorter than K on average: twice the longest row of the first build)
    if (K <= 512) return 16;
    return 32;
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_lj_workspace_bytes(int32_t n_atoms, int32_t n_systems, int32_t half_list,
                                              size_t* bytes) {
    if (!bytes || n_atoms < 0 || n_systems < 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj workspace: bad argument");
    size_t b = align_up((size_t)(n_systems > 0 ? n_systems : 1) * 10 * sizeof(double));
    b += 2 * align_up((size_t)(n_systems > 0 ? n_systems : 1) * sizeof(int32_t));
    b += align_up((size_t)(n_systems > 0 ? n_systems : 1) * sizeof(LjSysImage));
    if (half_list) b += align_up((size_t)(n_atoms > 0 ? n_atoms : 1) * 4 * sizeof(double));
    *bytes = b;
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_lj_energy_forces(const float* positions, const float* cells,
                                            const int32_t* neighbor_matrix,
                                            const int32_t* neighbor_matrix_shifts,
                                            const int32_t* num_neighbors, const int32_t* batch_idx,
                                            int32_t n_atoms, int32_t max_neighbors,
                                            int32_t n_systems, int32_t fill_value, double epsilon,
                                            double sigma, double cutoff, double switch_width,
                                            int32_t half_list, float* atomic_energies, float* forces,
                                            float* virials, float* system_energies, void* workspace,
                                            size_t workspace_bytes, void* stream) {
    return nvamd_lj_energy_forces_hinted(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors,
                                         batch_idx, nullptr, 0.0, n_atoms, max_neighbors, n_systems, fill_value, epsilon,
                                         sigma, cutoff, switch_width, half_list, atomic_energies, forces, virials,
                                         system_energies, workspace, workspace_bytes, stream);
}

// The one implementation behind the three entry points; `workspace` is device memory of at least
// nvamd_lj_workspace_bytes(n_atoms, n_systems, half_list) bytes, wherever it comes from.
static int32_t lj_energy_forces_impl(const float* positions, const float* cells, const int32_t* neighbor_matrix,
                                     const int32_t* neighbor_matrix_shifts, const int32_t* num_neighbors,
                                     const int32_t* batch_idx, const int32_t* row_order, double neighbor_list_cutoff,
                                     int32_t n_atoms, int32_t max_neighbors, int32_t n_systems, int32_t fill_value,
                                     double epsilon, double sigma, double cutoff, double switch_width,
                                     int32_t half_list, float* atomic_energies, float* forces, float* virials,
                                     float* system_energies, void* workspace, size_t workspace_bytes, void* stream,
                                     int32_t reuse_tables = 0, const LjTiles* tiles = nullptr) {
    if (n_atoms < 0 || n_systems < 0 || max_neighbors < 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj: negative size");
    if (!(switch_width >= 0.0) || switch_width > cutoff)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj: switch_width %g outside [0, cutoff]", switch_width);
    if (n_atoms > 0 && (!positions || !num_neighbors || !batch_idx || !atomic_energies || !forces))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj: null per-atom buffer");
    if (n_atoms > 0 && max_neighbors > 0 && !neighbor_matrix)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj: null neighbor matrix");
    if (neighbor_matrix_shifts && !cells)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj: shifts given without cells");
    size_t need = 0;
    nvamd_lj_workspace_bytes(n_atoms, n_systems, half_list, &need);
    const bool want_sys = (virials != nullptr) || (system_energies != nullptr);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "lj: workspace %zu < %zu bytes", workspace_bytes, need);

    hipStream_t st = static_cast<hipStream_t>(stream);
    LjArgs a;
    a.pos = positions;
    a.cells = cells;
    a.nm = neighbor_matrix;
    a.shifts = neighbor_matrix_shifts;
    a.nn = num_neighbors;
    a.bidx = batch_idx;
    a.n_atoms = n_atoms;
    a.K = max_neighbors;
    a.n_systems = n_systems;
    a.fill = fill_value < n_atoms ? fill_value : n_atoms;  // indices at or above are padding
    a.c4eps = 4.0 * epsilon;
    a.c24eps = 24.0 * epsilon;
    a.sig2 = sigma * sigma;
    a.rc2 = cutoff * cutoff;
    a.e_atom = atomic_energies;
    a.forces = forces;
    a.sys_acc = nullptr;
    a.n_blocks = 0;
    a.rows_per_block = 0;
    a.order = half_list ? nullptr : row_order;  // (the half-list kernel walks rows in index order)
    a.sys_first = nullptr;
    a.sys_last = nullptr;
    a.sys_image = nullptr;
    a.lds_atoms = kLdsAtoms;
    a.r_on = switch_width > 0.0 ? cutoff - switch_width : 0.0;
    a.inv_sw = switch_width > 0.0 ? 1.0 / switch_width : 0.0;
    // (a list built with a smaller cutoff than the potential's would be the caller's mistake:
    // the larger of the two is the safe bound)
    a.list_rc = (neighbor_list_cutoff > 0.0 && !half_list)
                    ? (neighbor_list_cutoff > cutoff ? neighbor_list_cutoff : cutoff)
                    : 0.0;
    const bool shifts = neighbor_matrix_shifts != nullptr;
    char* w = static_cast<char*>(workspace);
    const size_t nsys = (size_t)(n_systems > 0 ? n_systems : 1);
    int32_t* sys_first = reinterpret_cast<int32_t*>(w + align_up(nsys * 10 * sizeof(double)));
    int32_t* sys_last = reinterpret_cast<int32_t*>(w + align_up(nsys * 10 * sizeof(double)) +
                                                   align_up(nsys * sizeof(int32_t)));
    LjSysImage* sys_image = reinterpret_cast<LjSysImage*>(w + align_up(nsys * 10 * sizeof(double)) +
                                                          2 * align_up(nsys * sizeof(int32_t)));
    char* w_half = w + align_up(nsys * 10 * sizeof(double)) + 2 * align_up(nsys * sizeof(int32_t)) +
                   align_up(nsys * sizeof(LjSysImage));
    // the full-list path clears the accumulators in its range kernel when there are at least as many atoms
    // as accumulator words
    const bool clear_with_ranges = !half_list && (size_t)n_atoms >= (size_t)n_systems * 10;
    // the tables (and the cleared accumulators) of the previous call stand: full list only
    const bool reuse = reuse_tables && !half_list && n_atoms > 0;
    if (want_sys && n_systems > 0) {
        a.sys_acc = reinterpret_cast<double*>(w);
        size_t n = (size_t)n_systems * 10;
        if (!clear_with_ranges && !reuse)
            hipLaunchKernelGGL(clear_f64_kernel, dim3((unsigned)((n + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                               st, a.sys_acc, n);
    }
    if (n_atoms > 0) {
        if (half_list) {
            LjHalfArgs p;
            p.a = a;
            p.atom_acc = reinterpret_cast<double*>(w_half);
            size_t n = (size_t)n_atoms * 4;
            hipLaunchKernelGGL(clear_f64_kernel, dim3((unsigned)((n + kBlock - 1) / kBlock)), dim3(kBlock),
                               0, st, p.atom_acc, n);
            dim3 grid((n_atoms + kBlock - 1) / kBlock), blk(kBlock);
            const bool vir = virials != nullptr;
            if (vir && shifts) hipLaunchKernelGGL((lj_half_kernel<true, true>), grid, blk, 0, st, p);
            else if (vir) hipLaunchKernelGGL((lj_half_kernel<true, false>), grid, blk, 0, st, p);
            else if (shifts) hipLaunchKernelGGL((lj_half_kernel<false, true>), grid, blk, 0, st, p);
            else hipLaunchKernelGGL((lj_half_kernel<false, false>), grid, blk, 0, st, p);
            hipLaunchKernelGGL(lj_half_finish_kernel, grid, blk, 0, st, p.atom_acc, batch_idx,
                               atomic_energies, forces, a.sys_acc, n_atoms);
        } else {
            const bool vir = virials != nullptr;
            const bool sys = a.sys_acc != nullptr;
            if (!reuse)
                hipLaunchKernelGGL(lj_sys_range_kernel, dim3((n_atoms + kBlock - 1) / kBlock), dim3(kBlock), 0, st,
                                   batch_idx, n_atoms, shifts ? cells : nullptr, a.list_rc, sys_first, sys_last, sys_image,
                                   clear_with_ranges ? a.sys_acc : nullptr, n_systems * 10);
            a.sys_first = sys_first;
            a.sys_last = sys_last;
            a.sys_image = sys_image;
            // the tiles of the neighbor search walked again: images derived, per-system sums wanted
            if (tiles) {
                // (persistent workgroups, three to a CU; the number of units lives on the device)
                int dev = 0, cus = 256;
                hipGetDevice(&dev);
                hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
                dim3 grid((unsigned)((3 * cus + 7) / 8 * 8)), blk(kBlockFull);
                if (vir)
                    hipLaunchKernelGGL((lj_tiles_kernel<true, true>), grid, blk, 0, st, a, *tiles, tiles->records,
                                       tiles->count, a.cells, a.sys_image);
                else if (sys)
                    hipLaunchKernelGGL((lj_tiles_kernel<false, true>), grid, blk, 0, st, a, *tiles, tiles->records,
                                       tiles->count, a.cells, a.sys_image);
                else
                    hipLaunchKernelGGL((lj_tiles_kernel<false, false>), grid, blk, 0, st, a, *tiles, tiles->records,
                                       tiles->count, a.cells, a.sys_image);
            } else
            switch (lanes_per_row(max_neighbors)) {
                case 8: launch_full<8>(a, vir, shifts, sys, st); break;
                case 16: launch_full<16>(a, vir, shifts, sys, st); break;
                case 32: launch_full<32>(a, vir, shifts, sys, st); break;
                default: launch_full<64>(a, vir, shifts, sys, st); break;
            }
        }
    }
    if (want_sys && n_systems > 0) {
        // (the accumulators are left at zero for a call that reuses the tables)
        constexpr int kPer = kBlock / 10;
        hipLaunchKernelGGL(lj_sys_finish_clear_kernel, dim3((n_systems + kPer - 1) / kPer), dim3(kBlock), 0, st,
                           a.sys_acc, system_energies, virials, n_systems);
    }
    NVAMD_LAUNCH_CHECK("lj launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_lj_energy_forces_hinted(const float* positions, const float* cells,
                                                    const int32_t* neighbor_matrix,
                                                    const int32_t* neighbor_matrix_shifts,
                                                    const int32_t* num_neighbors, const int32_t* batch_idx,
                                                    const int32_t* row_order, double neighbor_list_cutoff,
                                                    int32_t n_atoms,
                                                    int32_t max_neighbors, int32_t n_systems, int32_t fill_value,
                                                    double epsilon, double sigma, double cutoff,
                                                    double switch_width, int32_t half_list, float* atomic_energies,
                                                    float* forces, float* virials, float* system_energies,
                                                    void* workspace, size_t workspace_bytes, void* stream) {
    return lj_energy_forces_impl(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors, batch_idx,
                                 row_order, neighbor_list_cutoff, n_atoms, max_neighbors, n_systems, fill_value, epsilon,
                                 sigma, cutoff, switch_width, half_list, atomic_energies, forces, virials,
                                 system_energies, workspace, workspace_bytes, stream);
}

NVAMD_EXPORT int32_t nvamd_lj_energy_forces_repeat(const float* positions, const float* cells,
                                                    const int32_t* neighbor_matrix,
                                                    const int32_t* neighbor_matrix_shifts,
                                                    const int32_t* num_neighbors, const int32_t* batch_idx,
                                                    const int32_t* row_order, double neighbor_list_cutoff,
                                                    int32_t n_atoms, int32_t max_neighbors, int32_t n_systems,
                                                    int32_t fill_value, double epsilon, double sigma, double cutoff,
                                                    double switch_width, int32_t reuse_tables, float* atomic_energies,
                                                    float* forces, float* virials, float* system_energies,
                                                    void* workspace, size_t workspace_bytes, void* stream) {
    return lj_energy_forces_impl(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors, batch_idx,
                                 row_order, neighbor_list_cutoff, n_atoms, max_neighbors, n_systems, fill_value, epsilon,
                                 sigma, cutoff, switch_width, /*half_list=*/0, atomic_energies, forces, virials,
                                 system_energies, workspace, workspace_bytes, stream, reuse_tables ? 1 : 0);
}

NVAMD_EXPORT int32_t nvamd_lj_energy_forces_tiles(const float* positions, const float* cells,
                                                   const int32_t* neighbor_matrix,
                                                   const int32_t* neighbor_matrix_shifts,
                                                   const int32_t* num_neighbors, const int32_t* batch_idx,
                                                   const int32_t* row_order, const uint16_t* tile_index,
                                                   const float* ordered_positions, const int32_t* tile_records,
                                                   const int32_t* tile_count, double neighbor_list_cutoff,
                                                   int32_t n_atoms, int32_t max_neighbors, int32_t n_systems,
                                                   int32_t fill_value, double epsilon, double sigma, double cutoff,
                                                   int32_t reuse_tables, float* atomic_energies, float* forces,
                                                   float* virials, float* system_energies, void* workspace,
                                                   size_t workspace_bytes, void* stream) {
    if (n_atoms > 0 && n_systems > 0) {
        if (!row_order || !tile_index || !ordered_positions || !tile_records || !tile_count)
            return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj tiles: null buffer");
        if (!cells || !neighbor_matrix_shifts || !(neighbor_list_cutoff > 0.0))
            return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj tiles: cells, shifts and the build's cutoff are needed");
        if (max_neighbors < 8 || max_neighbors % 8 != 0 || !aligned16(neighbor_matrix) || !aligned16(tile_index) ||
            !aligned16(ordered_positions))
            return fail(NVAMD_ERR_UNSUPPORTED, "lj tiles: rows of 16-byte words are needed (max_neighbors a multiple of 8)");
    }
    size_t capacity = 0;
    nvamd_nl_tile_records(n_atoms, n_systems, &capacity);
    const LjTiles tiles{tile_index, reinterpret_cast<const float4*>(ordered_positions),
                        reinterpret_cast<const int2*>(tile_records), tile_count,
                        (int)(capacity < 0x7fffffffull ? capacity : 0x7fffffffull)};
    return lj_energy_forces_impl(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors, batch_idx,
                                 row_order, neighbor_list_cutoff, n_atoms, max_neighbors, n_systems, fill_value, epsilon,
                                 sigma, cutoff, /*switch_width=*/0.0, /*half_list=*/0, atomic_energies, forces, virials,
                                 system_energies, workspace, workspace_bytes, stream, reuse_tables ? 1 : 0,
                                 (n_atoms > 0 && n_systems > 0) ? &tiles : nullptr);
}

// ---- the variant that allocates nothing ------------------------------------------------------
// For callers that cannot allocate or bring a workspace (code under HIP graph capture, tight serving
// loops): the pair kernel's scratch (per-system fp64 accumulators, first and last atom of each
// system) lives in a file-scope device array of fixed size.  Every GPU holds its own copy of the
// array at its own address, found once per device with hipGetSymbolAddress; from then on only that
// pointer is used (the array's name is a host-side stand-in, not a device address).
namespace {
constexpr int kStaticMaxSystems = NVAMD_LJ_STATIC_MAX_SYSTEMS;
constexpr size_t kStaticScratchBytes = NVAMD_LJ_STATIC_SCRATCH_BYTES;
constexpr int kStaticMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kStaticMaxDevices];  // per device; null until the first call on it
static std::mutex g_scratch_mutex;

NVAMD_EXPORT int32_t nvamd_lj_energy_forces_static(const float* positions, const float* cells,
                                                    const int32_t* neighbor_matrix,
                                                    const int32_t* neighbor_matrix_shifts,
                                                    const int32_t* num_neighbors, const int32_t* batch_idx,
                                                    const int32_t* row_order, double neighbor_list_cutoff,
                                                    int32_t n_atoms, int32_t max_neighbors, int32_t n_systems,
                                                    int32_t fill_value, double epsilon, double sigma, double cutoff,
                                                    double switch_width, float* atomic_energies, float* forces,
                                                    float* virials, float* system_energies, void* stream) {
    if (n_systems > kStaticMaxSystems)
        return fail(NVAMD_ERR_UNSUPPORTED, "lj (static scratch): %d systems, the built-in scratch holds at most %d",
                    (int)n_systems, kStaticMaxSystems);
    size_t need = 0;
    if (nvamd_lj_workspace_bytes(n_atoms, n_systems, 0, &need) != NVAMD_OK) return NVAMD_ERR_INVALID_ARGUMENT;
    if (need > kStaticScratchBytes)
        return fail(NVAMD_ERR_UNSUPPORTED, "lj (static scratch): needs %zu bytes, has %zu", need, kStaticScratchBytes);
    int dev = -1;
    int32_t rc = check_hip(hipGetDevice(&dev), "lj (static scratch): hipGetDevice");
    if (rc != NVAMD_OK) return rc;
    if (dev < 0 || dev >= kStaticMaxDevices)
        return fail(NVAMD_ERR_UNSUPPORTED, "lj (static scratch): device %d out of range", dev);
    void* ptr = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_scratch_ptr[dev]) {
            void* p = nullptr;
            rc = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "lj (static scratch): hipGetSymbolAddress");
            if (rc != NVAMD_OK) return rc;
            if (!p) return fail(NVAMD_ERR_HIP, "lj (static scratch): null symbol address on device %d", dev);
            g_scratch_ptr[dev] = p;
        }
        ptr = g_scratch_ptr[dev];
    }
    // full list only: the half-list kernel needs 32 bytes of scratch per atom
    return lj_energy_forces_impl(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors, batch_idx,
                                 row_order, neighbor_list_cutoff, n_atoms, max_neighbors, n_systems, fill_value, epsilon,
                                 sigma, cutoff, switch_width, /*half_list=*/0, atomic_energies, forces, virials,
                                 system_energies, ptr, kStaticScratchBytes, stream);
}
