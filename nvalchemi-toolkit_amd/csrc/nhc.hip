// Nose-Hoover chain thermostat for gfx950: the chain half-step propagator and the drift.
//
// Reference interface: nvalchemi::nhc_chain_update (nvalchemi/dynamics/_ops/nose_hoover.py:143-246)
// and nvalchemi::nhc_position_update (:291-325), called by NVTNoseHoover.pre_update / post_update
// (nvalchemi/dynamics/integrators/nvt_nose_hoover.py:215-281) as
//   chain(dt) - kick(dt/2) - drift(dt) - [forces] - kick(dt/2) - chain(dt);
// the kick, nvalchemi::nhc_velocity_half_step (:248-289), is the velocity half kick of velocity
// Verlet (nvamd_vv_velocity_finalize).  The reference's own kernel is in its kernel library; what
// is computed here is the published propagator (Martyna, Tuckerman, Tobias, Klein, Mol. Phys. 87,
// 1117 (1996)) with one pass of the 3- or 5-weight Suzuki-Yoshida factorisation.
//
// Per system, with KE2 = sum m v^2, chain velocities u_k (eta_dot), positions eta_k, masses Q_k and
// d = w dt for each weight w:
//   u_C += G_C d/4;  for k = C-1..1: u_k = (u_k a + G_k d/4) a, a = exp(-u_{k+1} d/8);
//   s = exp(-u_1 d/2), scale *= s, KE2 *= s^2;  eta_k += u_k d/2;  then the sweep back up,
//   G_1 = (KE2 - N_f kT)/Q_1, G_k = (Q_{k-1} u_{k-1}^2 - kT)/Q_k,
// and v *= scale at the end.  Chain arithmetic in double on the state in the arrays' own type (float32, or
// float64 through the _f64 entry points: the reference's ops take both, nvalchemi/dynamics/_ops/_bridge.py),
// each result rounded once when stored; velocities are multiplied by the scale in that type.
//
// Three launches: sum m v^2 per system (one streaming pass, 20 B/atom, float64 atomics per
// wavefront and system), the chains (one lane per system), the scaling (24 B/atom).  Bound: HBM.
#include "common.h"

namespace nvamd {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxChain = 16;

__global__ __launch_bounds__(kBlock) void nhc_clear_kernel(double* __restrict__ sum, int m) {
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s < m) sum[s] = 0.0;
}

// sum m v^2 per system: a segmented sum inside each wavefront (the batch index is sorted, so a
// system is one run of lanes), then one atomic per wavefront and system
template <typename T>
__global__ __launch_bounds__(kBlock) void nhc_ke2_kernel(const T* __restrict__ vel, const T* __restrict__ masses,
                                                         const int32_t* __restrict__ bidx, int n,
                                                         double* __restrict__ sum) {
#pragma clang fp contract(off)
    const int i = blockIdx.x * kBlock + threadIdx.x;
    const int lane = lane_id();
    int seg = -1 - (i - n);  // lanes past the end: each its own (negative) segment
    double v = 0.0;
    if (i < n) {
        seg = bidx[i];
        const size_t b = 3 * (size_t)i;
        const double vx = vel[b], vy = vel[b + 1], vz = vel[b + 2];
        v = (double)masses[i] * ((vx * vx + vy * vy) + vz * vz);
    }
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const int seg_up = __shfl_down(seg, o, kWave);
        const double up = __shfl_down(v, o, kWave);
        if ((lane + o < kWave) && (seg_up == seg)) v += up;
    }
    const int seg_prev = __shfl_up(seg, 1, kWave);
    if ((lane == 0 || seg_prev != seg) && i < n) atomic_add_f64(sum + seg, v);
}

struct Weights {
    double w[5];
    int n;
};

template <typename T>
__global__ __launch_bounds__(kBlock) void nhc_chain_kernel(T* __restrict__ eta, T* __restrict__ eta_dot,
                                                           const T* __restrict__ Q, const T* __restrict__ kT,
                                                           const T* __restrict__ dt, const T* __restrict__ ndof,
                                                           T* __restrict__ ke2, T* __restrict__ total_scale,
                                                           const double* __restrict__ sum,
                                                           const uint8_t* __restrict__ active, int compute_ke, int C,
                                                           Weights ys, int m) {
#pragma clang fp contract(off)
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    if (active && !active[s]) return;
    double u[kMaxChain], x[kMaxChain], q[kMaxChain];
    for (int k = 0; k < C; ++k) {
        u[k] = eta_dot[(size_t)s * C + k];
        x[k] = eta[(size_t)s * C + k];
        q[k] = Q[(size_t)s * C + k];
    }
    const double kt = kT[s], nf = ndof[s], h = dt[s];
    double k2 = compute_ke ? sum[s] : (double)ke2[s];
    if (compute_ke) ke2[s] = (T)k2;
    double scale = 1.0;
    for (int iw = 0; iw < ys.n; ++iw) {
        const double d = ys.w[iw] * h, d2 = 0.5 * d, d4 = 0.25 * d, d8 = 0.125 * d;
        {
            const double g = (C > 1) ? (q[C - 2] * u[C - 2] * u[C - 2] - kt) / q[C - 1] : (k2 - nf * kt) / q[0];
            u[C - 1] += g * d4;
        }
        for (int k = C - 2; k >= 0; --k) {
            const double aa = exp(-d8 * u[k + 1]);
            const double g = (k == 0) ? (k2 - nf * kt) / q[0] : (q[k - 1] * u[k - 1] * u[k - 1] - kt) / q[k];
            u[k] = (u[k] * aa + g * d4) * aa;
        }
        {
            const double sc = exp(-d2 * u[0]);
            scale *= sc;
            k2 *= sc * sc;
        }
        for (int k = 0; k < C; ++k) x[k] += d2 * u[k];
        for (int k = 0; k < C - 1; ++k) {
            const double aa = exp(-d8 * u[k + 1]);
            const double g = (k == 0) ? (k2 - nf * kt) / q[0] : (q[k - 1] * u[k - 1] * u[k - 1] - kt) / q[k];
            u[k] = (u[k] * aa + g * d4) * aa;
        }
        {
            const double g = (C > 1) ? (q[C - 2] * u[C - 2] * u[C - 2] - kt) / q[C - 1] : (k2 - nf * kt) / q[0];
            u[C - 1] += g * d4;
        }
    }
    for (int k = 0; k < C; ++k) {
        eta_dot[(size_t)s * C + k] = (T)u[k];
        eta[(size_t)s * C + k] = (T)x[k];
    }
    total_scale[s] = (T)scale;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void nhc_scale_kernel(T* __restrict__ vel, const T* __restrict__ total_scale,
                                                           const int32_t* __restrict__ bidx,
                                                           const uint8_t* __restrict__ active, int n) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int s = bidx[i];
    if (active && !active[s]) return;
    const T sc = total_scale[s];
    const size_t b = 3 * (size_t)i;
    vel[b] *= sc;
    vel[b + 1] *= sc;
    vel[b + 2] *= sc;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void nhc_drift_kernel(T* __restrict__ pos, const T* __restrict__ vel,
                                                           const T* __restrict__ dt, const int32_t* __restrict__ bidx,
                                                           const uint8_t* __restrict__ active, int n) {
#pragma clang fp contract(off)
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int s = bidx[i];
    if (active && !active[s]) return;
    const T h = dt[s];
    const size_t b = 3 * (size_t)i;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        const T step = vel[b + a] * h;
        pos[b + a] = pos[b + a] + step;
    }
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_nhc_workspace_bytes(int32_t n_systems, size_t* bytes) {
    if (!bytes || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "nhc workspace: bad argument");
    *bytes = align_up((size_t)(n_systems > 0 ? n_systems : 1) * sizeof(double));
    return NVAMD_OK;
}

namespace {

template <typename T>
int32_t nhc_chain_update(T* velocities, const T* masses, T* eta, T* eta_dot, const T* chain_masses, const T* kT,
                         const T* dt, const T* ndof, T* ke2, T* total_scale, const int32_t* batch_idx,
                         const uint8_t* active, int32_t compute_ke, int32_t chain_length, int32_t yoshida_order,
                         int32_t n_atoms, int32_t n_systems, void* workspace, size_t workspace_bytes, void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "nhc: negative size");
    if (chain_length < 1 || chain_length > kMaxChain)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nhc: chain_length %d outside 1..%d", chain_length, kMaxChain);
    if (yoshida_order != 1 && yoshida_order != 3 && yoshida_order != 5)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nhc: yoshida_order must be 1, 3 or 5, got %d", yoshida_order);
    if (n_systems == 0) return NVAMD_OK;
    if (!eta || !eta_dot || !chain_masses || !kT || !dt || !ndof || !ke2 || !total_scale)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nhc: null per-system buffer");
    if (n_atoms > 0 && (!velocities || !masses || !batch_idx))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nhc: null per-atom buffer");
    size_t need = 0;
    nvamd_nhc_workspace_bytes(n_systems, &need);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "nhc: workspace %zu < %zu bytes", workspace_bytes, need);
    Weights ys;
    if (yoshida_order == 3) {
        const double a = 1.0 / (2.0 - cbrt(2.0));
        ys = Weights{{a, 1.0 - 2.0 * a, a, 0.0, 0.0}, 3};
    } else if (yoshida_order == 5) {
        const double a = 1.0 / (4.0 - cbrt(4.0));
        ys = Weights{{a, a, 1.0 - 4.0 * a, a, a}, 5};
    } else {
        ys = Weights{{1.0, 0.0, 0.0, 0.0, 0.0}, 1};
    }
    double* sum = static_cast<double*>(workspace);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 gm((n_systems + kBlock - 1) / kBlock), gn((n_atoms + kBlock - 1) / kBlock), blk(kBlock);
    if (compute_ke) {
        hipLaunchKernelGGL(nhc_clear_kernel, gm, blk, 0, st, sum, n_systems);
        if (n_atoms > 0) hipLaunchKernelGGL(nhc_ke2_kernel<T>, gn, blk, 0, st, velocities, masses, batch_idx, n_atoms, sum);
    }
    hipLaunchKernelGGL(nhc_chain_kernel<T>, gm, blk, 0, st, eta, eta_dot, chain_masses, kT, dt, ndof, ke2, total_scale,
                       sum, active, compute_ke ? 1 : 0, chain_length, ys, n_systems);
    if (n_atoms > 0)
        hipLaunchKernelGGL(nhc_scale_kernel<T>, gn, blk, 0, st, velocities, total_scale, batch_idx, active, n_atoms);
    NVAMD_LAUNCH_CHECK("nhc launch");
    return NVAMD_OK;
}

template <typename T>
int32_t nhc_position_update(T* positions, const T* velocities, const T* dt, const int32_t* batch_idx,
                            const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "nhc drift: negative size");
    if (n_atoms == 0) return NVAMD_OK;
    if (!positions || !velocities || !dt || !batch_idx) return fail(NVAMD_ERR_INVALID_ARGUMENT, "nhc drift: null buffer");
    hipLaunchKernelGGL(nhc_drift_kernel<T>, dim3((n_atoms + kBlock - 1) / kBlock), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), positions, velocities, dt, batch_idx, active, n_atoms);
    NVAMD_LAUNCH_CHECK("nhc drift launch");
    return NVAMD_OK;
}

}  // namespace

NVAMD_EXPORT int32_t nvamd_nhc_chain_update(float* velocities, const float* masses, float* eta, float* eta_dot,
                                            const float* chain_masses, const float* kT, const float* dt,
                                            const float* ndof, float* ke2, float* total_scale,
                                            const int32_t* batch_idx, const uint8_t* active, int32_t compute_ke,
                                            int32_t chain_length, int32_t yoshida_order, int32_t n_atoms,
                                            int32_t n_systems, void* workspace, size_t workspace_bytes, void* stream) {
    return nhc_chain_update<float>(velocities, masses, eta, eta_dot, chain_masses, kT, dt, ndof, ke2, total_scale,
                                   batch_idx, active, compute_ke, chain_length, yoshida_order, n_atoms, n_systems,
                                   workspace, workspace_bytes, stream);
}

NVAMD_EXPORT int32_t nvamd_nhc_chain_update_f64(double* velocities, const double* masses, double* eta, double* eta_dot,
                                                const double* chain_masses, const double* kT, const double* dt,
                                                const double* ndof, double* ke2, double* total_scale,
                                                const int32_t* batch_idx, const uint8_t* active, int32_t compute_ke,
                                                int32_t chain_length, int32_t yoshida_order, int32_t n_atoms,
                                                int32_t n_systems, void* workspace, size_t workspace_bytes,
                                                void* stream) {
    return nhc_chain_update<double>(velocities, masses, eta, eta_dot, chain_masses, kT, dt, ndof, ke2, total_scale,
                                    batch_idx, active, compute_ke, chain_length, yoshida_order, n_atoms, n_systems,
                                    workspace, workspace_bytes, stream);
}

NVAMD_EXPORT int32_t nvamd_nhc_position_update(float* positions, const float* velocities, const float* dt,
                                               const int32_t* batch_idx, const uint8_t* active, int32_t n_atoms,
                                               int32_t n_systems, void* stream) {
    return nhc_position_update<float>(positions, velocities, dt, batch_idx, active, n_atoms, n_systems, stream);
}

NVAMD_EXPORT int32_t nvamd_nhc_position_update_f64(double* positions, const double* velocities, const double* dt,
                                                   const int32_t* batch_idx, const uint8_t* active, int32_t n_atoms,
                                                   int32_t n_systems, void* stream) {
    return nhc_position_update<double>(positions, velocities, dt, batch_idx, active, n_atoms, n_systems, stream);
}
