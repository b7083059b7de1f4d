// The float64 forms of the hot path's arithmetic kernels for gfx950: velocity Verlet, FIRE, FIRE 2.0, the
// per-system maximum force and the Lennard-Jones pair kernel.  (The thermostats' float64 forms are
// instantiations of their own kernels: langevin.hip, nhc.hip; the skin test and the wrap likewise.)
//
// The reference's custom ops take float32 or float64 arrays (nvalchemi/dynamics/_ops/_bridge.py
// `_vec_type` / `_scalar_type`, nvalchemi/dynamics/_ops/fire.py:281-287,
// nvalchemi/models/_ops/lj.py:116-216); every configuration it quotes figures on is float32, which
// is what the tuned kernels of this library serve.  These are the same formulas, in the same order
// of operations, on doubles: one lane per atom (or LPR lanes per row of the neighbor matrix),
// coalesced streams, no staging in LDS.  They are bound by HBM like their float32 counterparts and
// move twice the bytes.
#include "common.h"
#include "geom.h"

#pragma clang fp contract(off)

namespace nvamd {
namespace {

constexpr int kBlock = 256;

// ---- velocity Verlet (nvalchemi/dynamics/_ops/velocity_verlet.py:50-92, 102-138) -------------
template <bool PRE>
__global__ __launch_bounds__(kBlock) void vv_f64_kernel(double* __restrict__ pos, double* __restrict__ vel,
                                                        const double* __restrict__ frc,
                                                        const double* __restrict__ masses,
                                                        const double* __restrict__ dt,
                                                        const int32_t* __restrict__ bidx,
                                                        const uint8_t* __restrict__ active, uint32_t n_elems) {
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_elems) return;
    const uint32_t atom = e / 3u;
    const int s = bidx[atom];
    if (active && !active[s]) return;
    const double m = masses[atom], h = dt[s];
    const double a = frc[e] / m;
    const double kick = a * (0.5 * h);
    const double vh = vel[e] + kick;
    vel[e] = vh;
    if (PRE) {
        const double dr = vh * h;
        pos[e] = pos[e] + dr;
    }
}

template <bool PRE>
int32_t launch_vv_f64(double* pos, double* vel, const double* frc, const double* masses, const double* dt,
                      const int32_t* bidx, const uint8_t* active, int32_t n_atoms, void* stream) {
    if (n_atoms < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "n_atoms < 0");
    if (n_atoms == 0) return NVAMD_OK;
    if ((PRE && !pos) || !vel || !frc || !masses || !dt || !bidx)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "velocity Verlet (float64): null buffer");
    if ((int64_t)n_atoms * 3 > 0x7fffffff)
        return fail(NVAMD_ERR_UNSUPPORTED, "velocity Verlet: more than 2^31/3 atoms");
    const uint32_t n_elems = 3u * (uint32_t)n_atoms;
    hipLaunchKernelGGL(vv_f64_kernel<PRE>, dim3((n_elems + kBlock - 1) / kBlock), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), pos, vel, frc, masses, dt, bidx, active, n_elems);
    NVAMD_LAUNCH_CHECK("velocity Verlet (float64) launch");
    return NVAMD_OK;
}

// ---- segmented reductions inside a wavefront (batch_idx is non-decreasing) --------------------
template <int NV>
__device__ __forceinline__ bool wave_segmented_sum(int seg, double (&v)[NV]) {
    const int lane = lane_id();
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const int seg_up = __shfl_down(seg, o, kWave);
        const bool take = (lane + o < kWave) && (seg_up == seg);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const double up = __shfl_down(v[k], o, kWave);
            if (take) v[k] += up;
        }
    }
    const int seg_prev = __shfl_up(seg, 1, kWave);
    return lane == 0 || seg_prev != seg;
}

// ---- per-system maximum force norm (nvalchemi/dynamics/base.py:304-349) ------------------------
// max over a system's atoms as an atomic max on the order-preserving 64-bit image of the doubles
__device__ __forceinline__ unsigned long long double_order_key(double d) {
    const unsigned long long b = (unsigned long long)__double_as_longlong(d);
    return (b >> 63) ? ~b : (b | 0x8000000000000000ull);
}
__device__ __forceinline__ double double_from_order_key(unsigned long long k) {
    const unsigned long long b = (k >> 63) ? (k & 0x7fffffffffffffffull) : ~k;
    return __longlong_as_double((long long)b);
}

__global__ __launch_bounds__(kBlock) void fmax_init_f64_kernel(unsigned long long* keys, int m) {
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s < m) keys[s] = double_order_key(-__builtin_inf());
}

__global__ __launch_bounds__(kBlock) void fmax_f64_kernel(const double* __restrict__ frc,
                                                          const int32_t* __restrict__ bidx,
                                                          unsigned long long* __restrict__ keys, int n_atoms) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const double x = frc[3 * (size_t)i], y = frc[3 * (size_t)i + 1], z = frc[3 * (size_t)i + 2];
    double n = sqrt((x * x + y * y) + z * z);
    // NaN must win, as it does in a max reduction over the values: it maps above every number
    const unsigned long long key = (n != n) ? 0xffffffffffffffffull : double_order_key(n);
    atomicMax(keys + bidx[i], key);
}

__global__ __launch_bounds__(kBlock) void fmax_finish_f64_kernel(const unsigned long long* keys, double* fmax, int m) {
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    const unsigned long long k = keys[s];
    fmax[s] = (k == 0xffffffffffffffffull) ? __builtin_nan("") : double_from_order_key(k);
}

// ---- FIRE (nvalchemi/dynamics/_ops/fire.py:79-140, order of :270-272) ---------------------------
constexpr double kFireVmax64 = 1.0e300;

struct FireScratch64 {
    double* acc;     // (M,3): sum F.v, sum v.v, sum F.F
    double* mix_a;   // (M) factor on v
    double* mix_b;   // (M) factor on F
    double* dt_use;  // (M) time step of the MD sub-step
};

__global__ __launch_bounds__(kBlock) void fire_clear_f64_kernel(double* acc, int n) {
    const int t = blockIdx.x * kBlock + threadIdx.x;
    if (t < n) acc[t] = 0.0;
}

__global__ __launch_bounds__(kBlock) void fire_reduce_f64_kernel(const double* __restrict__ vel,
                                                                 const double* __restrict__ frc,
                                                                 const int32_t* __restrict__ bidx,
                                                                 double* __restrict__ acc, int n_atoms) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    double v[3] = {0.0, 0.0, 0.0};
    int seg = -1 - (i - n_atoms);  // distinct negative ids past the end: never merged
    if (i < n_atoms) {
        seg = bidx[i];
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            const double vv = vel[3 * (size_t)i + a], ff = frc[3 * (size_t)i + a];
            v[0] += ff * vv;
            v[1] += vv * vv;
            v[2] += ff * ff;
        }
    }
    const bool head = wave_segmented_sum<3>(seg, v);
    if (head && i < n_atoms) {
        atomic_add_f64(acc + 3 * (size_t)seg + 0, v[0]);
        atomic_add_f64(acc + 3 * (size_t)seg + 1, v[1]);
        atomic_add_f64(acc + 3 * (size_t)seg + 2, v[2]);
    }
}

__global__ __launch_bounds__(kBlock) void fire_import_f64_kernel(const double* vf, const double* vv, const double* ff,
                                                                 double* acc, int m) {
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    acc[3 * s + 0] = vf[s];
    acc[3 * s + 1] = vv[s];
    acc[3 * s + 2] = ff[s];
}

__global__ __launch_bounds__(kBlock) void fire_params_f64_kernel(
    double* __restrict__ alpha, double* __restrict__ dt, const double* __restrict__ alpha_start,
    const double* __restrict__ f_alpha, const double* __restrict__ dt_min, const double* __restrict__ dt_max,
    int32_t* __restrict__ n_pos, const int32_t* __restrict__ n_min, const double* __restrict__ f_dec,
    const double* __restrict__ f_inc, double* __restrict__ vf, double* __restrict__ vv, double* __restrict__ ff,
    const uint8_t* __restrict__ active, FireScratch64 ws, int write_reductions, int m) {
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    const double P = ws.acc[3 * s + 0], VV = ws.acc[3 * s + 1], FF = ws.acc[3 * s + 2];
    if (write_reductions) {
        vf[s] = P;
        vv[s] = VV;
        ff[s] = FF;
    }
    const double h_stored = dt[s];  // the MD sub-step integrates with the time step of before the update
    double h = h_stored;
    double ma = 1.0, mb = 0.0;
    if (!active || active[s]) {
        if (P >= 0.0) {
            const double al = alpha[s];
            ma = 1.0 - al;
            mb = (FF > 0.0) ? al * sqrt(VV / FF) : 0.0;
            const int np = n_pos[s] + 1;
            n_pos[s] = np;
            if (np > n_min[s]) {
                const double nd = h * f_inc[s];
                const double cap = dt_max[s];
                h = nd < cap ? nd : cap;
                alpha[s] = al * f_alpha[s];
            }
        } else {
            ma = 0.0;
            mb = 0.0;
            n_pos[s] = 0;
            const double nd = h * f_dec[s];
            const double lo = dt_min[s];
            h = nd > lo ? nd : lo;
            alpha[s] = alpha_start[s];
        }
        dt[s] = h;
    }
    ws.mix_a[s] = ma;
    ws.mix_b[s] = mb;
    ws.dt_use[s] = h_stored;
}

__global__ __launch_bounds__(kBlock) void fire_update_f64_kernel(double* __restrict__ pos, double* __restrict__ vel,
                                                                 const double* __restrict__ frc,
                                                                 const double* __restrict__ masses,
                                                                 const double* __restrict__ maxstep,
                                                                 const int32_t* __restrict__ bidx,
                                                                 const uint8_t* __restrict__ active, FireScratch64 ws,
                                                                 int n_atoms) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const int s = bidx[i];
    if (active && !active[s]) return;
    const double ma = ws.mix_a[s], mb = ws.mix_b[s], h = ws.dt_use[s], ms = maxstep[s], m = masses[i];
    const size_t b = 3 * (size_t)i;
    double v[3], dr[3], f[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        f[a] = frc[b + a];
        const double acc = f[a] / m;
        v[a] = vel[b + a] + (h * acc);
        v[a] = fmin(fmax(v[a], -kFireVmax64), kFireVmax64);  // keep dr finite
        dr[a] = h * v[a];
    }
    // |dr| without overflow: scale by the largest component first
    const double big = fmax(fmax(fabs(dr[0]), fabs(dr[1])), fabs(dr[2]));
    double nrm = 0.0;
    if (big > 0.0) {
        const double a0 = dr[0] / big, a1 = dr[1] / big, a2 = dr[2] / big;
        nrm = big * sqrt((a0 * a0 + a1 * a1) + a2 * a2);
    }
    if (nrm > ms) {
        const double sc = ms / nrm;
#pragma unroll
        for (int a = 0; a < 3; ++a) dr[a] = dr[a] * sc;
    }
    // the mixing comes after the integration and acts on the kicked velocity
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        vel[b + a] = (ma * v[a]) + (mb * f[a]);
        pos[b + a] = pos[b + a] + dr[a];
    }
}

// ---- Lennard-Jones over the neighbor matrix (nvalchemi/models/_ops/lj.py:116-216, 246-321) ------
struct Lj64Args {
    const double* pos;
    const double* cells;
    const int32_t* nm;
    const int32_t* shifts;
    const int32_t* nn;
    const int32_t* bidx;
    int32_t n_atoms, K, fill, half;
    double c4eps, c24eps, sig2, rc2, r_on, inv_sw;
    double* e_atom;   // (N)
    double* forces;   // (N,3)
    double* sys_acc;  // (B,10): energy then virial, or null
};

constexpr int kLpr = 8;  // lanes per row

__device__ __forceinline__ double group8_sum(double v) {
    v += __shfl_xor(v, 4, kWave);
    v += __shfl_xor(v, 2, kWave);
    v += __shfl_xor(v, 1, kWave);
    return v;
}

// Full list: a row's owner receives the whole pair force and half the pair energy.  Half list: the
// kernel runs over the rows as they are and adds the partner's share with atomics (outputs cleared first).
template <bool HALF>
__global__ __launch_bounds__(kBlock) void lj_f64_kernel(Lj64Args a) {
    const int i = (int)((blockIdx.x * (unsigned)kBlock + threadIdx.x) / kLpr);
    const int sub = threadIdx.x % kLpr;
    if (i >= a.n_atoms) return;  // (whole groups of 8 lanes leave together)
    const int sys = a.bidx[i];
    int cnt = a.nn[i];
    cnt = cnt < a.K ? cnt : a.K;
    const double xi = a.pos[3 * (size_t)i], yi = a.pos[3 * (size_t)i + 1], zi = a.pos[3 * (size_t)i + 2];
    double h[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) h[k] = (a.shifts && a.cells) ? a.cells[9 * (size_t)sys + k] : 0.0;
    double e = 0.0, fx = 0.0, fy = 0.0, fz = 0.0;
    double w[6] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0};  // xx xy xz yy yz zz
    for (int k = sub; k < cnt; k += kLpr) {
        const int j = a.nm[(size_t)i * a.K + k];
        if (j < 0 || j >= a.fill) continue;
        int s0 = 0, s1 = 0, s2 = 0;
        if (a.shifts) {
            const int32_t* sp = a.shifts + ((size_t)i * a.K + k) * 3;
            s0 = sp[0];
            s1 = sp[1];
            s2 = sp[2];
        }
        double d0, d1, d2;
        const double r2 = pair_d2_exact(xi, yi, zi, a.pos[3 * (size_t)j], a.pos[3 * (size_t)j + 1],
                                        a.pos[3 * (size_t)j + 2], s0, s1, s2, h, d0, d1, d2);
        if (!(r2 < a.rc2)) continue;
        const double ir2 = 1.0 / r2;
        const double q2 = a.sig2 * ir2, q6 = q2 * q2 * q2, q12 = q6 * q6;
        double uu = a.c4eps * (q12 - q6);
        double gg = -(a.c24eps * (2.0 * q12 - q6)) * ir2;  // u'(r)/r
        if (a.inv_sw > 0.0) {
            const double r = sqrt(r2);
            if (r > a.r_on) {
                const double t = (r - a.r_on) * a.inv_sw, omt = 1.0 - t;
                const double S = 1.0 - t * t * t * (10.0 - 15.0 * t + 6.0 * t * t);
                const double dS = -30.0 * t * t * omt * omt * a.inv_sw;
                gg = gg * S + uu * dS / r;
                uu = uu * S;
            }
        }
        e += 0.5 * uu;
        fx += gg * d0;
        fy += gg * d1;
        fz += gg * d2;
        if (HALF) {
            atomic_add_f64(a.e_atom + j, 0.5 * uu);
            atomic_add_f64(a.forces + 3 * (size_t)j + 0, -gg * d0);
            atomic_add_f64(a.forces + 3 * (size_t)j + 1, -gg * d1);
            atomic_add_f64(a.forces + 3 * (size_t)j + 2, -gg * d2);
        }
        const double hg = HALF ? -gg : -0.5 * gg;
        w[0] += hg * d0 * d0;
        w[1] += hg * d0 * d1;
        w[2] += hg * d0 * d2;
        w[3] += hg * d1 * d1;
        w[4] += hg * d1 * d2;
        w[5] += hg * d2 * d2;
    }
    e = group8_sum(e);
    fx = group8_sum(fx);
    fy = group8_sum(fy);
    fz = group8_sum(fz);
    if (a.sys_acc) {
#pragma unroll
        for (int k = 0; k < 6; ++k) w[k] = group8_sum(w[k]);
    }
    if (sub != 0) return;
    if (HALF) {
        atomic_add_f64(a.e_atom + i, e);
        atomic_add_f64(a.forces + 3 * (size_t)i + 0, fx);
        atomic_add_f64(a.forces + 3 * (size_t)i + 1, fy);
        atomic_add_f64(a.forces + 3 * (size_t)i + 2, fz);
    } else {
        a.e_atom[i] = e;
        a.forces[3 * (size_t)i + 0] = fx;
        a.forces[3 * (size_t)i + 1] = fy;
        a.forces[3 * (size_t)i + 2] = fz;
    }
    if (a.sys_acc) {
        double* out = a.sys_acc + 10 * (size_t)sys;
        // (full list: a system's energy is the sum of its atoms' energies, added below once they are final)
        atomic_add_f64(out + 1, w[0]);
        atomic_add_f64(out + 2, w[1]);
        atomic_add_f64(out + 3, w[2]);
        atomic_add_f64(out + 5, w[3]);
        atomic_add_f64(out + 6, w[4]);
        atomic_add_f64(out + 9, w[5]);
    }
}

__global__ __launch_bounds__(kBlock) void lj_f64_clear_kernel(double* p, size_t n) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t < n) p[t] = 0.0;
}

// per-system energy: sum of the atomic energies (their own precision; nvalchemi/models/lj.py:467-477)
__global__ __launch_bounds__(kBlock) void lj_f64_sys_energy_kernel(const double* __restrict__ e_atom,
                                                                   const int32_t* __restrict__ bidx,
                                                                   double* __restrict__ sys_acc, int n_atoms) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    double v[1] = {0.0};
    int seg = -1 - (i - n_atoms);
    if (i < n_atoms) {
        seg = bidx[i];
        v[0] = e_atom[i];
    }
    const bool head = wave_segmented_sum<1>(seg, v);
    if (head && i < n_atoms) atomic_add_f64(sys_acc + 10 * (size_t)seg, v[0]);
}

__global__ __launch_bounds__(kBlock) void lj_f64_finish_kernel(const double* __restrict__ sys_acc,
                                                               double* __restrict__ sys_e,
                                                               double* __restrict__ virials, int m) {
    const int t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= m * 10) return;
    const int s = t / 10, k = t % 10;
    double v = sys_acc[t];
    if (k == 0) {
        if (sys_e) sys_e[s] = v;
    } else if (virials) {
        const int c = k - 1, r = c / 3, q = c % 3;
        if (r > q) v = sys_acc[10 * (size_t)s + 1 + 3 * q + r];  // the symmetric half was accumulated: mirror it
        virials[9 * (size_t)s + c] = v;
    }
}

// ---- FIRE 2.0 (nvalchemi/dynamics/_ops/fire.py:467-557; the float32 form is in integrators.hip) ----
//   P > 0 :  a = 1 - alpha, b = alpha sqrt(VV / FF); count += 1; past delaystep: dt grows, alpha decays
//   P <= 0:  count = 0; alpha = alpha0; r -= (dt/2) v; v = 0; dt shrinks while it stays >= tmin
//   v += dt F;  P > 0: v = a v + b F;  dr = dt v, scaled so that the system's largest |dr| stays within maxstep
struct Fire2Scratch64 {
    double* acc;                // (M,3): sum F.v, sum v.v, sum F.F
    double* mix_a;              // (M) factor on the kicked v
    double* mix_b;              // (M) factor on F
    double* back;               // (M) length of the step back (0: none)
    unsigned long long* big;    // (M) largest |dr| of the system, as the bits of a double >= 0 (NaN above all)
    double* up;                 // (M) P > 0 (1.0 / 0.0)
};

struct Fire2Params64 {
    int delaystep;
    double dtgrow, dtshrink, alphashrink, alpha0, tmax, tmin, maxstep;
};

__global__ __launch_bounds__(kBlock) void fire2_params_f64_kernel(double* __restrict__ alpha, double* __restrict__ dt,
                                                                  int32_t* __restrict__ count, double* vf, double* vv,
                                                                  double* ff, const uint8_t* __restrict__ active,
                                                                  Fire2Scratch64 ws, Fire2Params64 p, int m) {
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    const double P = ws.acc[3 * s + 0], VV = ws.acc[3 * s + 1], FF = ws.acc[3 * s + 2];
    if (vf) vf[s] = P;
    if (vv) vv[s] = VV;
    if (ff) ff[s] = FF;
    double ma = 1.0, mb = 0.0, bk = 0.0, up = 0.0;
    if (!active || active[s]) {
        if (P > 0.0) {
            const double al = alpha[s];
            up = 1.0;
            ma = 1.0 - al;
            mb = (FF > 1e-20) ? al * sqrt(VV / FF) : 0.0;
            const int c = count[s] + 1;
            count[s] = c;
            if (c > p.delaystep) {
                const double nd = dt[s] * p.dtgrow;
                dt[s] = nd < p.tmax ? nd : p.tmax;
                alpha[s] = al * p.alphashrink;
            }
        } else {
            count[s] = 0;
            alpha[s] = p.alpha0;
            bk = 0.5 * dt[s];
            const double nd = dt[s] * p.dtshrink;
            if (nd >= p.tmin) dt[s] = nd;
        }
    }
    ws.mix_a[s] = ma;
    ws.mix_b[s] = mb;
    ws.back[s] = bk;
    ws.big[s] = 0ull;
    ws.up[s] = up;
}

// new velocities (and the step back), and the largest displacement they would give
__global__ __launch_bounds__(kBlock) void fire2_kick_f64_kernel(double* __restrict__ pos, double* __restrict__ vel,
                                                                const double* __restrict__ frc,
                                                                const double* __restrict__ dt,
                                                                const int32_t* __restrict__ bidx,
                                                                const uint8_t* __restrict__ active, Fire2Scratch64 ws,
                                                                int n_atoms) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const int s = bidx[i];
    if (active && !active[s]) return;
    const double h = dt[s], ma = ws.mix_a[s], mb = ws.mix_b[s], bk = ws.back[s];
    const bool up = ws.up[s] != 0.0;
    const size_t b = 3 * (size_t)i;
    double dr[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        const double f = frc[b + a];
        double v = vel[b + a];
        if (!up) {
            const double undo = bk * v;
            pos[b + a] = pos[b + a] - undo;
            v = 0.0;
        }
        const double kick = h * f;
        v = v + kick;
        if (up) {
            const double va = ma * v, fb = mb * f;
            v = va + fb;
        }
        v = fmin(fmax(v, -kFireVmax64), kFireVmax64);
        vel[b + a] = v;
        dr[a] = h * v;
    }
    const double top = fmax(fmax(fabs(dr[0]), fabs(dr[1])), fabs(dr[2]));
    double nrm = 0.0;
    if (top > 0.0) {
        const double a0 = dr[0] / top, a1 = dr[1] / top, a2 = dr[2] / top;
        nrm = top * sqrt((a0 * a0 + a1 * a1) + a2 * a2);
    }
    // norms are >= 0 or NaN: their bit patterns order like unsigned integers, the canonical NaN above all
    const unsigned long long key = (top != top || nrm != nrm) ? 0x7ff8000000000000ull
                                                              : (unsigned long long)__double_as_longlong(nrm);
    atomicMax(ws.big + s, key);
}

__global__ __launch_bounds__(kBlock) void fire2_drift_f64_kernel(double* __restrict__ pos, const double* __restrict__ vel,
                                                                 const double* __restrict__ dt,
                                                                 const int32_t* __restrict__ bidx,
                                                                 const uint8_t* __restrict__ active, Fire2Scratch64 ws,
                                                                 double maxstep, double* __restrict__ max_norm,
                                                                 int n_atoms) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const int s = bidx[i];
    if (active && !active[s]) return;
    const double h = dt[s], big = __longlong_as_double((long long)ws.big[s]);
    const double sc = big > maxstep ? maxstep / big : 1.0;
    const size_t b = 3 * (size_t)i;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        double dr = h * vel[b + a];
        dr = dr * sc;
        pos[b + a] = pos[b + a] + dr;
    }
    if (max_norm && (i == 0 || bidx[i - 1] != s)) max_norm[s] = big;
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_vv_position_update_f64(double* positions, double* velocities, const double* forces,
                                                  const double* masses, const double* dt, const int32_t* batch_idx,
                                                  const uint8_t* active, int32_t n_atoms, int32_t n_systems,
                                                  void* stream) {
    (void)n_systems;
    return launch_vv_f64<true>(positions, velocities, forces, masses, dt, batch_idx, active, n_atoms, stream);
}

NVAMD_EXPORT int32_t nvamd_vv_velocity_finalize_f64(double* velocities, const double* forces_new, const double* masses,
                                                    const double* dt, const int32_t* batch_idx, const uint8_t* active,
                                                    int32_t n_atoms, int32_t n_systems, void* stream) {
    (void)n_systems;
    return launch_vv_f64<false>(nullptr, velocities, forces_new, masses, dt, batch_idx, active, n_atoms, stream);
}

NVAMD_EXPORT int32_t nvamd_f64_workspace_bytes(int32_t n_systems, size_t* bytes) {
    if (!bytes || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "float64 workspace: bad argument");
    // FIRE: (M,3) sums + three (M) factors; FIRE 2.0: (M,3) sums + five (M) words; LJ: (M,10) sums; fmax: (M) keys
    // -- the largest of them
    *bytes = align_up((size_t)(n_systems > 0 ? n_systems : 1) * 10 * sizeof(double));
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_segment_fmax_f64(const double* forces, const int32_t* batch_idx, int32_t n_atoms,
                                            int32_t n_systems, double* fmax, void* workspace, size_t workspace_bytes,
                                            void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fmax: negative size");
    if (n_systems == 0) return NVAMD_OK;
    if (!fmax || (n_atoms > 0 && (!forces || !batch_idx))) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fmax: null buffer");
    size_t need = 0;
    nvamd_f64_workspace_bytes(n_systems, &need);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "fmax (float64): workspace %zu < %zu bytes", workspace_bytes, need);
    hipStream_t st = static_cast<hipStream_t>(stream);
    unsigned long long* keys = static_cast<unsigned long long*>(workspace);
    const dim3 gm((n_systems + kBlock - 1) / kBlock), blk(kBlock);
    hipLaunchKernelGGL(fmax_init_f64_kernel, gm, blk, 0, st, keys, n_systems);
    if (n_atoms > 0)
        hipLaunchKernelGGL(fmax_f64_kernel, dim3((n_atoms + kBlock - 1) / kBlock), blk, 0, st, forces, batch_idx, keys,
                           n_atoms);
    hipLaunchKernelGGL(fmax_finish_f64_kernel, gm, blk, 0, st, keys, fmax, n_systems);
    NVAMD_LAUNCH_CHECK("fmax (float64) launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_fire_step_f64(double* positions, double* velocities, const double* forces,
                                         const double* masses, double* alpha, double* dt, const double* alpha_start,
                                         const double* f_alpha, const double* dt_min, const double* dt_max,
                                         const double* maxstep, int32_t* n_steps_positive, const int32_t* n_min,
                                         const double* f_dec, const double* f_inc, const int32_t* uphill_flag,
                                         double* vf, double* vv, double* ff, const int32_t* batch_idx,
                                         int32_t compute_reductions, const uint8_t* active, int32_t n_atoms,
                                         int32_t n_systems, void* workspace, size_t workspace_bytes, void* stream) {
    (void)uphill_flag;  // vanilla FIRE only, as for float32: the caller passes zeros
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire: negative size");
    if (n_systems == 0) return NVAMD_OK;
    if (!alpha || !dt || !alpha_start || !f_alpha || !dt_min || !dt_max || !maxstep || !n_steps_positive || !n_min ||
        !f_dec || !f_inc || !vf || !vv || !ff)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire (float64): null per-system buffer");
    if (n_atoms > 0 && (!positions || !velocities || !forces || !masses || !batch_idx))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire (float64): null per-atom buffer");
    size_t need = 0;
    nvamd_f64_workspace_bytes(n_systems, &need);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "fire (float64): workspace %zu < %zu bytes", workspace_bytes, need);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int M = n_systems;
    FireScratch64 ws;
    ws.acc = static_cast<double*>(workspace);
    ws.mix_a = ws.acc + 3 * (size_t)M;
    ws.mix_b = ws.mix_a + M;
    ws.dt_use = ws.mix_b + M;
    const dim3 gm((M + kBlock - 1) / kBlock), blk(kBlock);
    if (compute_reductions) {
        hipLaunchKernelGGL(fire_clear_f64_kernel, dim3((3 * M + kBlock - 1) / kBlock), blk, 0, st, ws.acc, 3 * M);
        if (n_atoms > 0)
            hipLaunchKernelGGL(fire_reduce_f64_kernel, dim3((n_atoms + kBlock - 1) / kBlock), blk, 0, st, velocities,
                               forces, batch_idx, ws.acc, n_atoms);
    } else {
        hipLaunchKernelGGL(fire_import_f64_kernel, gm, blk, 0, st, vf, vv, ff, ws.acc, M);
    }
    hipLaunchKernelGGL(fire_params_f64_kernel, gm, blk, 0, st, alpha, dt, alpha_start, f_alpha, dt_min, dt_max,
                       n_steps_positive, n_min, f_dec, f_inc, vf, vv, ff, active, ws, compute_reductions ? 1 : 0, M);
    if (n_atoms > 0)
        hipLaunchKernelGGL(fire_update_f64_kernel, dim3((n_atoms + kBlock - 1) / kBlock), blk, 0, st, positions,
                           velocities, forces, masses, maxstep, batch_idx, active, ws, n_atoms);
    NVAMD_LAUNCH_CHECK("fire (float64) launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_lj_energy_forces_f64(const double* positions, const double* cells,
                                                const int32_t* neighbor_matrix, const int32_t* neighbor_matrix_shifts,
                                                const int32_t* num_neighbors, const int32_t* batch_idx, int32_t n_atoms,
                                                int32_t max_neighbors, int32_t n_systems, int32_t fill_value,
                                                double epsilon, double sigma, double cutoff, double switch_width,
                                                int32_t half_list, double* atomic_energies, double* forces,
                                                double* virials, double* system_energies, void* workspace,
                                                size_t workspace_bytes, void* stream) {
    if (n_atoms < 0 || n_systems < 0 || max_neighbors < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj: negative size");
    if (!(switch_width >= 0.0) || switch_width > cutoff)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj: switch_width %g outside [0, cutoff]", switch_width);
    if (n_atoms > 0 && (!positions || !num_neighbors || !batch_idx || !atomic_energies || !forces))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj (float64): null per-atom buffer");
    if (n_atoms > 0 && max_neighbors > 0 && !neighbor_matrix)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj (float64): null neighbor matrix");
    if (neighbor_matrix_shifts && !cells) return fail(NVAMD_ERR_INVALID_ARGUMENT, "lj: shifts given without cells");
    const bool want_sys = virials != nullptr || system_energies != nullptr;
    size_t need = 0;
    nvamd_f64_workspace_bytes(n_systems, &need);
    if (want_sys && (!workspace || workspace_bytes < need))
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "lj (float64): workspace %zu < %zu bytes", workspace_bytes, need);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 blk(kBlock);
    auto blocks = [](size_t n) { return dim3((unsigned)((n + kBlock - 1) / kBlock)); };
    Lj64Args a;
    a.pos = positions;
    a.cells = cells;
    a.nm = neighbor_matrix;
    a.shifts = neighbor_matrix_shifts;
    a.nn = num_neighbors;
    a.bidx = batch_idx;
    a.n_atoms = n_atoms;
    a.K = max_neighbors;
    a.fill = fill_value < n_atoms ? fill_value : n_atoms;
    a.half = half_list ? 1 : 0;
    a.c4eps = 4.0 * epsilon;
    a.c24eps = 24.0 * epsilon;
    a.sig2 = sigma * sigma;
    a.rc2 = cutoff * cutoff;
    a.r_on = switch_width > 0.0 ? cutoff - switch_width : 0.0;
    a.inv_sw = switch_width > 0.0 ? 1.0 / switch_width : 0.0;
    a.e_atom = atomic_energies;
    a.forces = forces;
    a.sys_acc = nullptr;
    if (want_sys && n_systems > 0) {
        a.sys_acc = static_cast<double*>(workspace);
        hipLaunchKernelGGL(lj_f64_clear_kernel, blocks((size_t)n_systems * 10), blk, 0, st, a.sys_acc,
                           (size_t)n_systems * 10);
    }
    if (n_atoms > 0) {
        if (half_list) {
            hipLaunchKernelGGL(lj_f64_clear_kernel, blocks((size_t)n_atoms), blk, 0, st, atomic_energies, (size_t)n_atoms);
            hipLaunchKernelGGL(lj_f64_clear_kernel, blocks((size_t)n_atoms * 3), blk, 0, st, forces, (size_t)n_atoms * 3);
            hipLaunchKernelGGL(lj_f64_kernel<true>, blocks((size_t)n_atoms * kLpr), blk, 0, st, a);
        } else {
            hipLaunchKernelGGL(lj_f64_kernel<false>, blocks((size_t)n_atoms * kLpr), blk, 0, st, a);
        }
        if (a.sys_acc)
            hipLaunchKernelGGL(lj_f64_sys_energy_kernel, blocks((size_t)n_atoms), blk, 0, st, atomic_energies, batch_idx,
                               a.sys_acc, n_atoms);
    }
    if (want_sys && n_systems > 0)
        hipLaunchKernelGGL(lj_f64_finish_kernel, blocks((size_t)n_systems * 10), blk, 0, st, a.sys_acc, system_energies,
                           virials, n_systems);
    NVAMD_LAUNCH_CHECK("lj (float64) launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_fire2_step_f64(double* positions, double* velocities, const double* forces,
                                          const int32_t* batch_idx, double* alpha, double* dt, int32_t* nsteps_inc,
                                          double* vf, double* v_sumsq, double* f_sumsq, double* max_norm,
                                          int32_t delaystep, double dtgrow, double dtshrink, double alphashrink,
                                          double alpha0, double tmax, double tmin, double maxstep,
                                          const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* workspace,
                                          size_t workspace_bytes, void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire2: negative size");
    if (n_systems == 0) return NVAMD_OK;
    if (!alpha || !dt || !nsteps_inc) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire2 (float64): null per-system buffer");
    if (n_atoms > 0 && (!positions || !velocities || !forces || !batch_idx))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire2 (float64): null per-atom buffer");
    size_t need = 0;
    nvamd_f64_workspace_bytes(n_systems, &need);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "fire2 (float64): workspace %zu < %zu bytes", workspace_bytes, need);
    const int M = n_systems;
    Fire2Scratch64 ws;  // eight of the workspace's ten words per system
    ws.acc = static_cast<double*>(workspace);
    ws.mix_a = ws.acc + 3 * (size_t)M;
    ws.mix_b = ws.mix_a + M;
    ws.back = ws.mix_b + M;
    ws.big = reinterpret_cast<unsigned long long*>(ws.back + M);
    ws.up = ws.back + 2 * (size_t)M;
    const Fire2Params64 p{delaystep, dtgrow, dtshrink, alphashrink, alpha0, tmax, tmin, maxstep};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 blk(kBlock), gm((M + kBlock - 1) / kBlock), gn((n_atoms + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(fire_clear_f64_kernel, dim3((3 * M + kBlock - 1) / kBlock), blk, 0, st, ws.acc, 3 * M);
    if (n_atoms > 0)
        hipLaunchKernelGGL(fire_reduce_f64_kernel, gn, blk, 0, st, velocities, forces, batch_idx, ws.acc, n_atoms);
    hipLaunchKernelGGL(fire2_params_f64_kernel, gm, blk, 0, st, alpha, dt, nsteps_inc, vf, v_sumsq, f_sumsq, active, ws,
                       p, M);
    if (n_atoms > 0) {
        hipLaunchKernelGGL(fire2_kick_f64_kernel, gn, blk, 0, st, positions, velocities, forces, dt, batch_idx, active,
                           ws, n_atoms);
        hipLaunchKernelGGL(fire2_drift_f64_kernel, gn, blk, 0, st, positions, velocities, dt, batch_idx, active, ws,
                           maxstep, max_norm, n_atoms);
    }
    NVAMD_LAUNCH_CHECK("fire2 (float64) launch");
    return NVAMD_OK;
}
