// Velocity Verlet, FIRE and the per-system max-force reduction for gfx950.
//
// All three are pure streaming kernels bounded by HBM bandwidth.  The velocity-Verlet
// halves treat the (N,3) arrays as flat float streams and move 16 bytes per lane; the
// per-atom operands (mass, system index, time step) come through the vector L1.
// Arithmetic is float32 with one rounding per operation (no fused multiply-add) so that
// results do not depend on how the compiler schedules the expression.
//
// Reference interfaces: nvalchemi/dynamics/_ops/velocity_verlet.py:50-138,
// nvalchemi/dynamics/_ops/fire.py:79-140, nvalchemi/dynamics/base.py:304-349.
#include "common.h"

#pragma clang fp contract(off)

namespace nvamd {
namespace {

constexpr int kBlock = 256;

// ---- velocity Verlet ----------------------------------------------------------------------
// a = F/m ; v(t+dt/2) = v + a*(dt/2) ; r(t+dt) = r + v(t+dt/2)*dt
__device__ __forceinline__ void vv_pre_elem(float& r, float& v, float f, float m, float h) {
    float a = f / m;
    float kick = a * (0.5f * h);
    float vh = v + kick;
    float dr = vh * h;
    v = vh;
    r = r + dr;
}
__device__ __forceinline__ void vv_post_elem(float& v, float f, float m, float h) {
    float a = f / m;
    float kick = a * (0.5f * h);
    v = v + kick;
}

struct AtomOperands {
    float m, h;
    bool on;
};

__device__ __forceinline__ AtomOperands load_atom(uint32_t atom, const float* __restrict__ masses,
                                                  const float* __restrict__ dt,
                                                  const int32_t* __restrict__ bidx,
                                                  const uint8_t* __restrict__ active) {
    AtomOperands o;
    int s = bidx[atom];
    o.m = masses[atom];
    o.h = dt[s];
    o.on = active ? (active[s] != 0) : true;
    return o;
}

// MODE 0: the closing half kick; 1: half kick and drift; 2: the closing half kick of one step and the half kick and
// drift of the next with the same forces, one after the other per element (the same operations in the same order
// as launches 0 and 1 in a row: the velocity in between is rounded as it would be stored).
template <int MODE>
__device__ __forceinline__ void vv_elem(float& r, float& v, float f, float m, float h) {
    if (MODE != 1) vv_post_elem(v, f, m, h);
    if (MODE != 0) vv_pre_elem(r, v, f, m, h);
}

// One lane owns four consecutive floats of the flat (3N) stream: at most two atoms.
template <int MODE>
__global__ __launch_bounds__(kBlock) void vv_flat_kernel(
    float* __restrict__ pos, float* __restrict__ vel, const float* __restrict__ frc,
    const float* __restrict__ masses, const float* __restrict__ dt,
    const int32_t* __restrict__ bidx, const uint8_t* __restrict__ active, uint32_t n_elems) {
    uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    uint32_t e0 = 4u * t;
    if (e0 >= n_elems) return;
    uint32_t a0 = e0 / 3u;
    uint32_t rem = e0 - 3u * a0;  // position of e0 inside atom a0
    if (e0 + 4u <= n_elems) {
        uint32_t a1 = (e0 + 3u) / 3u;
        AtomOperands o0 = load_atom(a0, masses, dt, bidx, active);
        AtomOperands o1 = (a1 != a0) ? load_atom(a1, masses, dt, bidx, active) : o0;
        float4 v4 = reinterpret_cast<const float4*>(vel)[t];
        float4 f4 = reinterpret_cast<const float4*>(frc)[t];
        float v[4] = {v4.x, v4.y, v4.z, v4.w};
        float f[4] = {f4.x, f4.y, f4.z, f4.w};
        float r[4] = {0.f, 0.f, 0.f, 0.f};
        if (MODE != 0) {
            float4 r4 = reinterpret_cast<const float4*>(pos)[t];
            r[0] = r4.x; r[1] = r4.y; r[2] = r4.z; r[3] = r4.w;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            bool second = (rem + k) >= 3u;
            const AtomOperands& o = second ? o1 : o0;
            if (o.on) vv_elem<MODE>(r[k], v[k], f[k], o.m, o.h);
        }
        reinterpret_cast<float4*>(vel)[t] = make_float4(v[0], v[1], v[2], v[3]);
        if (MODE != 0) reinterpret_cast<float4*>(pos)[t] = make_float4(r[0], r[1], r[2], r[3]);
    } else {
        for (uint32_t e = e0; e < n_elems; ++e) {
            AtomOperands o = load_atom(e / 3u, masses, dt, bidx, active);
            if (!o.on) continue;
            float none = 0.f;
            vv_elem<MODE>(MODE != 0 ? pos[e] : none, vel[e], frc[e], o.m, o.h);
        }
    }
}

// Fallback for buffers that are not 16-byte aligned: one lane per float.
template <int MODE>
__global__ __launch_bounds__(kBlock) void vv_scalar_kernel(
    float* __restrict__ pos, float* __restrict__ vel, const float* __restrict__ frc,
    const float* __restrict__ masses, const float* __restrict__ dt,
    const int32_t* __restrict__ bidx, const uint8_t* __restrict__ active, uint32_t n_elems) {
    uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_elems) return;
    AtomOperands o = load_atom(e / 3u, masses, dt, bidx, active);
    if (!o.on) return;
    float none = 0.f;
    vv_elem<MODE>(MODE != 0 ? pos[e] : none, vel[e], frc[e], o.m, o.h);
}

template <int MODE>
int32_t launch_vv(float* pos, float* vel, const float* frc, const float* masses, const float* dt,
                  const int32_t* bidx, const uint8_t* active, int32_t n_atoms, void* stream) {
    if (n_atoms < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "n_atoms < 0");
    if (n_atoms == 0) return NVAMD_OK;
    if ((MODE != 0 && !pos) || !vel || !frc || !masses || !dt || !bidx)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "velocity Verlet: null buffer");
    if ((int64_t)n_atoms * 3 > 0x7fffffff)
        return fail(NVAMD_ERR_UNSUPPORTED, "velocity Verlet: more than 2^31/3 atoms");
    uint32_t n_elems = 3u * (uint32_t)n_atoms;
    hipStream_t st = static_cast<hipStream_t>(stream);
    bool vec = aligned16(vel) && aligned16(frc) && (MODE == 0 || aligned16(pos));
    if (vec) {
        uint32_t n_threads = (n_elems + 3u) / 4u;
        dim3 grid((n_threads + kBlock - 1) / kBlock);
        hipLaunchKernelGGL(vv_flat_kernel<MODE>, grid, dim3(kBlock), 0, st, pos, vel, frc, masses, dt,
                           bidx, active, n_elems);
    } else {
        dim3 grid((n_elems + kBlock - 1) / kBlock);
        hipLaunchKernelGGL(vv_scalar_kernel<MODE>, grid, dim3(kBlock), 0, st, pos, vel, frc, masses,
                           dt, bidx, active, n_elems);
    }
    NVAMD_LAUNCH_CHECK("velocity Verlet launch");
    return NVAMD_OK;
}

// ---- segmented wave reductions ------------------------------------------------------------
// batch_idx is non-decreasing, so inside a wave every system is one run of lanes.  After
// log2(64) steps the first lane of each run holds the run's total.
template <int NV>
__device__ __forceinline__ bool wave_segmented_sum(int seg, double (&v)[NV]) {
    int lane = lane_id();
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        int seg_up = __shfl_down(seg, o, kWave);
        bool take = (lane + o < kWave) && (seg_up == seg);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            double up = __shfl_down(v[k], o, kWave);
            if (take) v[k] += up;
        }
    }
    int seg_prev = __shfl_up(seg, 1, kWave);
    return lane == 0 || seg_prev != seg;
}

__device__ __forceinline__ bool wave_segmented_max(int seg, float& v) {
    int lane = lane_id();
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        int seg_up = __shfl_down(seg, o, kWave);
        float up = __shfl_down(v, o, kWave);
        // NaN must win, as it does in a max reduction over the values
        if ((lane + o < kWave) && (seg_up == seg)) v = (up > v || up != up) ? up : v;
    }
    int seg_prev = __shfl_up(seg, 1, kWave);
    return lane == 0 || seg_prev != seg;
}

// ---- FIRE -----------------------------------------------------------------------------------
constexpr float kFireVmax = 3.0e38f;

// The sums live in one of two slots, taken in turn from call to call (flip): the kernel that sums into one slot
// clears the other for the next call, and the update kernel, which reads the sum of both slots (the other one is
// zero by then), turns flip over.  So no launch is needed to clear the sums; a new workspace starts as zeros.
struct FireScratch {
    int* flip;       // (1) the slot of this call's sums
    double* acc;     // (M, 2, 3): per system and slot, sum F.v, sum v.v, sum F.F (a system's place does not depend on M)
    float* alpha0;   // (M) mixing parameter of before the update
    float* dt0;      // (M) time step of before the update (the MD sub-step integrates with it)
};

__global__ __launch_bounds__(kBlock) void fire_clear_kernel(double* acc, int n) {
    int t = blockIdx.x * kBlock + threadIdx.x;
    if (t < n) acc[t] = 0.0;
}

// What has to happen before the update besides the sums: the slot of the next call is cleared, and the mixing
// parameter and the time step of before the update are set aside (the update kernel's per-atom threads read them
// there while its per-system threads write the new ones into the caller's arrays).  Done for system s by whoever
// is given it: a thread of the kernel that sums, or of the kernel below.
__device__ __forceinline__ void fire_set_aside(const FireScratch& ws, int slot, int s, int m,
                                               const float* __restrict__ alpha, const float* __restrict__ dt) {
    double* other = ws.acc + 6 * (size_t)s + 3 * (slot ^ 1);
    other[0] = 0.0;
    other[1] = 0.0;
    other[2] = 0.0;
    ws.alpha0[s] = alpha[s];
    ws.dt0[s] = dt[s];
}

// No kernel sums: the caller's sums (compute_reductions = 0) or zeros (no atoms) go into this call's slot.
__global__ __launch_bounds__(kBlock) void fire_import_kernel(const float* __restrict__ alpha,
                                                             const float* __restrict__ dt,
                                                             const float* __restrict__ vf,
                                                             const float* __restrict__ vv,
                                                             const float* __restrict__ ff, FireScratch ws, int m,
                                                             int import_sums) {
    int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    const int slot = ws.flip[0];
    double* mine = ws.acc + 6 * (size_t)s + 3 * slot;
    mine[0] = import_sums ? (double)vf[s] : 0.0;
    mine[1] = import_sums ? (double)vv[s] : 0.0;
    mine[2] = import_sums ? (double)ff[s] : 0.0;
    fire_set_aside(ws, slot, s, m, alpha, dt);
}

// A workgroup takes kFireQuad * kBlock atoms, a thread kFireQuad consecutive ones (read as 16-byte words when the
// arrays allow it); a thread's atoms are nearly always of one system, so they are summed in registers first.
// Inside a wave the threads of one system are then summed with shuffles; the sums of the first kFireSlots systems
// a workgroup meets are collected in LDS and go to memory once per workgroup (a system of a few thousand atoms
// otherwise receives one atomic per wave on the same three addresses, which is what this kernel then waits for).
constexpr int kFireQuad = 4;
constexpr int kFireSlots = 8;

template <bool VEC>
__global__ __launch_bounds__(kBlock) void fire_reduce_kernel(const float* __restrict__ vel,
                                                             const float* __restrict__ frc,
                                                             const int32_t* __restrict__ bidx,
                                                             double* __restrict__ acc_base, int n_atoms,
                                                             int chunks_per_block, FireScratch ws, int m,
                                                             const float* __restrict__ alpha,
                                                             const float* __restrict__ dt) {
    __shared__ double s_acc[kFireSlots][3];
    // (FIRE: the sums go into the slot of this call, and the systems are dealt to the threads of the grid for what
    // else has to happen before the update; FIRE 2.0 passes its own cleared accumulators and no scratch)
    double* acc = acc_base;
    int per_system = 3;  // doubles from one system's sums to the next one's
    if (ws.flip) {
        const int slot = ws.flip[0];
        acc = ws.acc + 3 * slot;
        per_system = 6;
        for (int s = (int)blockIdx.x * kBlock + (int)threadIdx.x; s < m; s += (int)gridDim.x * kBlock)
            fire_set_aside(ws, slot, s, m, alpha, dt);
    }
    // a workgroup takes chunks_per_block consecutive chunks of kFireQuad * kBlock atoms
    const int block_first = (int)blockIdx.x * chunks_per_block * (kFireQuad * kBlock);  // (below n_atoms: the grid is sized so)
    if (threadIdx.x < kFireSlots * 3) (&s_acc[0][0])[threadIdx.x] = 0.0;
    const int seg_lo = bidx[block_first];
    __syncthreads();
    auto deposit = [&](int seg, const double* v) {
        const unsigned slot = (unsigned)(seg - seg_lo);
        if (slot < (unsigned)kFireSlots) {
            atomicAdd(&s_acc[slot][0], v[0]);
            atomicAdd(&s_acc[slot][1], v[1]);
            atomicAdd(&s_acc[slot][2], v[2]);
        } else {
            atomic_add_f64(acc + per_system * (size_t)seg + 0, v[0]);
            atomic_add_f64(acc + per_system * (size_t)seg + 1, v[1]);
            atomic_add_f64(acc + per_system * (size_t)seg + 2, v[2]);
        }
    };
    for (int chunk = 0; chunk < chunks_per_block; ++chunk) {
    const int first = block_first + chunk * (kFireQuad * kBlock);
    if (first >= n_atoms) break;
    const int i0 = first + kFireQuad * (int)threadIdx.x;
    double v[3] = {0.0, 0.0, 0.0};
    int seg = -1 - (int)threadIdx.x;  // distinct negative ids for threads past the end: never merged
    if (i0 < n_atoms) {
        const int n = (n_atoms - i0) < kFireQuad ? (n_atoms - i0) : kFireQuad;
        seg = bidx[i0];
        float x[3 * kFireQuad], f[3 * kFireQuad];
        if (VEC && n == kFireQuad) {
            const float4* xv = reinterpret_cast<const float4*>(vel + 3 * (size_t)i0);
            const float4* fv = reinterpret_cast<const float4*>(frc + 3 * (size_t)i0);
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                const float4 a = xv[q], b = fv[q];
                x[4 * q + 0] = a.x; x[4 * q + 1] = a.y; x[4 * q + 2] = a.z; x[4 * q + 3] = a.w;
                f[4 * q + 0] = b.x; f[4 * q + 1] = b.y; f[4 * q + 2] = b.z; f[4 * q + 3] = b.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < 3 * kFireQuad; ++k) {
                const bool in = k < 3 * n;
                x[k] = in ? vel[3 * (size_t)i0 + k] : 0.f;
                f[k] = in ? frc[3 * (size_t)i0 + k] : 0.f;
            }
        }
#pragma unroll
        for (int q = 0; q < kFireQuad; ++q) {
            double w[3] = {0.0, 0.0, 0.0};
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                const double vv = (double)x[3 * q + c], ff = (double)f[3 * q + c];
                w[0] += ff * vv;
                w[1] += vv * vv;
                w[2] += ff * ff;
            }
            const int sq = q < n ? bidx[i0 + q] : seg;
            if (sq == seg) {
                v[0] += w[0]; v[1] += w[1]; v[2] += w[2];
            } else if (q < n) {
                deposit(sq, w);  // (an atom of the next system inside a thread's four: rare)
            }
        }
    }
    const bool head = wave_segmented_sum<3>(seg, v);
    if (head && seg >= 0) deposit(seg, v);
    }
    __syncthreads();
    if (threadIdx.x < kFireSlots * 3) {
        // (a slot that no atom touched is still zero and names a system that may not exist)
        const double t = (&s_acc[0][0])[threadIdx.x];
        if (t != 0.0) atomic_add_f64(acc + per_system * (size_t)(seg_lo + threadIdx.x / 3) + threadIdx.x % 3, t);
    }
}

void launch_fire_reduce(const float* velocities, const float* forces, const int32_t* batch_idx, double* acc,
                        int n_atoms, hipStream_t st, FireScratch ws = FireScratch{nullptr, nullptr, nullptr, nullptr},
                        int m = 0, const float* alpha = nullptr, const float* dt = nullptr) {
    // about three workgroups per compute unit at most: every workgroup ends with atomics on its systems' sums,
    // which for one large system are the same three addresses for all of them
    const int n_chunks = (n_atoms + kFireQuad * kBlock - 1) / (kFireQuad * kBlock);
    const int per = n_chunks > 1024 ? (n_chunks + 767) / 768 : 1;
    const dim3 grid_r((n_chunks + per - 1) / per), blk(kBlock);
    if (aligned16(velocities) && aligned16(forces))
        hipLaunchKernelGGL(fire_reduce_kernel<true>, grid_r, blk, 0, st, velocities, forces, batch_idx, acc, n_atoms, per,
                           ws, m, alpha, dt);
    else
        hipLaunchKernelGGL(fire_reduce_kernel<false>, grid_r, blk, 0, st, velocities, forces, batch_idx, acc, n_atoms, per,
                           ws, m, alpha, dt);
}

// The update: blocks below n_atom_blocks take one atom per thread, the blocks after them one system per thread.
//   per atom   : MD step with the time step of before the update, then the mixing with the parameter of before
//                the update (both set aside by fire_prepare_kernel) and the sums of entry
//   per system : the sums go out, n+, dt and alpha are updated in the caller's arrays
__global__ __launch_bounds__(kBlock) void fire_update_kernel(
    float* __restrict__ pos, float* __restrict__ vel, const float* __restrict__ frc,
    const float* __restrict__ masses, const float* __restrict__ maxstep, const int32_t* __restrict__ bidx,
    const uint8_t* __restrict__ active, float* __restrict__ alpha, float* __restrict__ dt,
    const float* __restrict__ alpha_start, const float* __restrict__ f_alpha, const float* __restrict__ dt_min,
    const float* __restrict__ dt_max, int32_t* __restrict__ n_pos, const int32_t* __restrict__ n_min,
    const float* __restrict__ f_dec, const float* __restrict__ f_inc, float* __restrict__ vf,
    float* __restrict__ vv, float* __restrict__ ff, FireScratch ws, int write_reductions, int n_atoms,
    int n_atom_blocks, int m) {
    if ((int)blockIdx.x >= n_atom_blocks) {
        const int s = ((int)blockIdx.x - n_atom_blocks) * kBlock + (int)threadIdx.x;
        if (s >= m) return;
        // (nobody reads flip in this kernel: the sums are taken from both slots, one of which is zero)
        if (s == 0) ws.flip[0] ^= 1;
        const double* sums = ws.acc + 6 * (size_t)s;
        const double P = sums[0] + sums[3], VV = sums[1] + sums[4], FF = sums[2] + sums[5];
        if (write_reductions) {
            vf[s] = (float)P;
            vv[s] = (float)VV;
            ff[s] = (float)FF;
        }
        if (active && !active[s]) return;
        float h = ws.dt0[s];
        if (P >= 0.0) {
            const int np = n_pos[s] + 1;
            n_pos[s] = np;
            if (np > n_min[s]) {
                const float nd = h * f_inc[s];
                const float cap = dt_max[s];
                h = nd < cap ? nd : cap;
                alpha[s] = ws.alpha0[s] * f_alpha[s];
            }
        } else {
            n_pos[s] = 0;
            const float nd = h * f_dec[s];
            const float lo = dt_min[s];
            h = nd > lo ? nd : lo;
            alpha[s] = alpha_start[s];
        }
        dt[s] = h;
        return;
    }
    const int i = (int)blockIdx.x * kBlock + (int)threadIdx.x;
    if (i >= n_atoms) return;
    const int s = bidx[i];
    if (active && !active[s]) return;
    const double* sums = ws.acc + 6 * (size_t)s;
    const double P = sums[0] + sums[3], VV = sums[1] + sums[4], FF = sums[2] + sums[5];
    const float al = ws.alpha0[s], h = ws.dt0[s], ms = maxstep[s], m_i = masses[i];
    float ma = 0.0f, mb = 0.0f;
    if (P >= 0.0) {
        ma = 1.0f - al;
        mb = (FF > 0.0) ? (float)((double)al * sqrt(VV / FF)) : 0.0f;
    }
    size_t b = 3 * (size_t)i;
    float v[3], dr[3], f[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        f[a] = frc[b + a];
        float acc = f[a] / m_i;
        v[a] = vel[b + a] + (h * acc);
        v[a] = fminf(fmaxf(v[a], -kFireVmax), kFireVmax);  // keep dr finite
        dr[a] = h * v[a];
    }
    // |dr| without overflow: scale by the largest component first
    float big = fmaxf(fmaxf(fabsf(dr[0]), fabsf(dr[1])), fabsf(dr[2]));
    float nrm = 0.0f;
    if (big > 0.0f) {
        float a0 = dr[0] / big, a1 = dr[1] / big, a2 = dr[2] / big;
        nrm = big * sqrtf((a0 * a0 + a1 * a1) + a2 * a2);
    }
    if (nrm > ms) {
        float sc = ms / nrm;
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

// ---- FIRE 2.0 -------------------------------------------------------------------------------
// Reference interface: fire2_step_coord (nvalchemi/dynamics/_ops/fire.py:467-557), called by
// FIRE2.pre_update (nvalchemi/dynamics/optimizers/fire2.py:218-251).  The reference's step is in its
// kernel library; this is FIRE 2.0 as published with its LAMMPS implementation (Guenole et al.
// 2020): semi-implicit Euler, half step back on a reset, unit masses, no initial delay:
//   P > 0 :  a = 1 - alpha, b = alpha sqrt(VV / FF); count += 1; past delaystep: dt grows, alpha decays
//   P <= 0:  count = 0; alpha = alpha0; r -= (dt/2) v; v = 0; dt shrinks while it stays >= tmin
//   v += dt F;  P > 0: v = a v + b F;  dr = dt v, the whole system's step scaled so that its
//   largest atomic displacement stays within maxstep.
struct Fire2Scratch {
    double* acc;   // (M,3): sum F.v, sum v.v, sum F.F
    float* mix_a;  // (M) factor on the kicked v
    float* mix_b;  // (M) factor on F
    float* back;   // (M) length of the step back (0: none)
    float* big;    // (M) largest |dr| of the system
    int32_t* up;   // (M) P > 0
};

struct Fire2Params {
    int delaystep;
    float dtgrow, dtshrink, alphashrink, alpha0, tmax, tmin, maxstep;
};

__global__ __launch_bounds__(kBlock) void fire2_params_kernel(float* __restrict__ alpha, float* __restrict__ dt,
                                                              int32_t* __restrict__ count, float* vf, float* vv,
                                                              float* ff, const uint8_t* __restrict__ active,
                                                              Fire2Scratch ws, Fire2Params p, int m) {
    int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    const double P = ws.acc[3 * s + 0], VV = ws.acc[3 * s + 1], FF = ws.acc[3 * s + 2];
    if (vf) vf[s] = (float)P;
    if (vv) vv[s] = (float)VV;
    if (ff) ff[s] = (float)FF;
    float ma = 1.0f, mb = 0.0f, bk = 0.0f;
    int up = 0;
    if (!active || active[s]) {
        if (P > 0.0) {
            const float al = alpha[s];
            up = 1;
            ma = 1.0f - al;
            mb = (FF > 1e-20) ? (float)((double)al * sqrt(VV / FF)) : 0.0f;
            const int c = count[s] + 1;
            count[s] = c;
            if (c > p.delaystep) {
                const float nd = dt[s] * p.dtgrow;
                dt[s] = nd < p.tmax ? nd : p.tmax;
                alpha[s] = al * p.alphashrink;
            }
        } else {
            count[s] = 0;
            alpha[s] = p.alpha0;
            bk = 0.5f * dt[s];
            const float nd = dt[s] * p.dtshrink;
            if (nd >= p.tmin) dt[s] = nd;
        }
    }
    ws.mix_a[s] = ma;
    ws.mix_b[s] = mb;
    ws.back[s] = bk;
    ws.big[s] = 0.0f;
    ws.up[s] = up;
}

// new velocities (and the step back), and the largest displacement they would give
__global__ __launch_bounds__(kBlock) void fire2_kick_kernel(float* __restrict__ pos, float* __restrict__ vel,
                                                            const float* __restrict__ frc,
                                                            const float* __restrict__ dt,
                                                            const int32_t* __restrict__ bidx,
                                                            const uint8_t* __restrict__ active, Fire2Scratch ws,
                                                            int n_atoms) {
#pragma clang fp contract(off)
    const int i = blockIdx.x * kBlock + threadIdx.x;
    int seg = -1 - (i - n_atoms);
    float nrm = 0.0f;
    bool live = false;
    if (i < n_atoms) {
        const int s = bidx[i];
        seg = s;
        live = !active || active[s];
        if (live) {
            const float h = dt[s], ma = ws.mix_a[s], mb = ws.mix_b[s], bk = ws.back[s];
            const bool up = ws.up[s] != 0;
            const size_t b = 3 * (size_t)i;
            float dr[3];
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                const float f = frc[b + a];
                float v = vel[b + a];
                if (!up) {
                    const float undo = bk * v;
                    pos[b + a] = pos[b + a] - undo;
                    v = 0.0f;
                }
                const float kick = h * f;
                v = v + kick;
                if (up) {
                    const float va = ma * v, fb = mb * f;
                    v = va + fb;
                }
                v = fminf(fmaxf(v, -kFireVmax), kFireVmax);
                vel[b + a] = v;
                dr[a] = h * v;
            }
            const float top = fmaxf(fmaxf(fabsf(dr[0]), fabsf(dr[1])), fabsf(dr[2]));
            if (top > 0.0f) {
                const float a0 = dr[0] / top, a1 = dr[1] / top, a2 = dr[2] / top;
                nrm = top * sqrtf((a0 * a0 + a1 * a1) + a2 * a2);
            } else if (top != top) {
                nrm = top;
            }
        }
    }
    const bool head = wave_segmented_max(seg, nrm);
    // norms are >= 0 or NaN: their bit patterns order like signed integers, NaN above all
    if (head && i < n_atoms && (!active || active[seg]))
        atomicMax(reinterpret_cast<int*>(ws.big) + seg, __float_as_int(nrm));
}

__global__ __launch_bounds__(kBlock) void fire2_drift_kernel(float* __restrict__ pos, const float* __restrict__ vel,
                                                             const float* __restrict__ dt,
                                                             const int32_t* __restrict__ bidx,
                                                             const uint8_t* __restrict__ active, Fire2Scratch ws,
                                                             float maxstep, float* __restrict__ max_norm, int n_atoms) {
#pragma clang fp contract(off)
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const int s = bidx[i];
    if (active && !active[s]) return;
    const float h = dt[s], big = ws.big[s];
    const float sc = big > maxstep ? maxstep / big : 1.0f;
    const size_t b = 3 * (size_t)i;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        float dr = h * vel[b + a];
        dr = dr * sc;
        pos[b + a] = pos[b + a] + dr;
    }
    if (max_norm && (i == 0 || bidx[i - 1] != s)) max_norm[s] = big;
}

// ---- status of converged systems -----------------------------------------------------------
// status[s] = target where values[s] <= threshold and status[s] == source (a NaN value is not converged)
template <typename T>
__global__ __launch_bounds__(kBlock) void status_migrate_kernel(const T* __restrict__ values, T threshold,
                                                                long long* __restrict__ status, long long source,
                                                                long long target, int m) {
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    if (values[s] <= threshold && status[s] == source) status[s] = target;
}

// ---- per-system max force norm ------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void fmax_init_kernel(float* fmax, int m) {
    int s = blockIdx.x * kBlock + threadIdx.x;
    if (s < m) fmax[s] = -INFINITY;
}

__global__ __launch_bounds__(kBlock) void fmax_kernel(const float* __restrict__ frc,
                                                      const int32_t* __restrict__ bidx,
                                                      float* __restrict__ fmax, int n_atoms) {
    int i = blockIdx.x * kBlock + threadIdx.x;
    int seg = -1 - (i - n_atoms);
    float nrm = 0.0f;
    if (i < n_atoms) {
        seg = bidx[i];
        size_t b = 3 * (size_t)i;
        float x = frc[b], y = frc[b + 1], z = frc[b + 2];
        nrm = sqrtf((x * x + y * y) + z * z);
    }
    bool head = wave_segmented_max(seg, nrm);
    if (head && i < n_atoms) {
        // norms are >= 0 (or NaN): their bit patterns order like signed integers, and the
        // bit pattern of -inf is below all of them
        atomicMax(reinterpret_cast<int*>(fmax) + seg, __float_as_int(nrm));
    }
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_vv_position_update(float* positions, float* velocities,
                                              const float* forces, const float* masses,
                                              const float* dt, const int32_t* batch_idx,
                                              const uint8_t* active, int32_t n_atoms,
                                              int32_t n_systems, void* stream) {
    (void)n_systems;
    return launch_vv<1>(positions, velocities, forces, masses, dt, batch_idx, active, n_atoms,
                        stream);
}

NVAMD_EXPORT int32_t nvamd_vv_velocity_finalize(float* velocities, const float* forces_new,
                                                const float* masses, const float* dt,
                                                const int32_t* batch_idx, const uint8_t* active,
                                                int32_t n_atoms, int32_t n_systems, void* stream) {
    (void)n_systems;
    return launch_vv<0>(nullptr, velocities, forces_new, masses, dt, batch_idx, active, n_atoms,
                        stream);
}

NVAMD_EXPORT int32_t nvamd_vv_finalize_then_update(float* positions, float* velocities, const float* forces,
                                                   const float* masses, const float* dt, const int32_t* batch_idx,
                                                   const uint8_t* active, int32_t n_atoms, int32_t n_systems,
                                                   void* stream) {
    (void)n_systems;
    return launch_vv<2>(positions, velocities, forces, masses, dt, batch_idx, active, n_atoms, stream);
}

NVAMD_EXPORT int32_t nvamd_fire_workspace_bytes(int32_t n_systems, size_t* bytes) {
    if (!bytes || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire workspace: bad argument");
    size_t m = (size_t)(n_systems > 0 ? n_systems : 1);
    *bytes = align_up(sizeof(int)) + align_up(2 * m * 3 * sizeof(double)) + 2 * align_up(m * sizeof(float));
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_fire_step(float* positions, float* velocities, const float* forces,
                                     const float* masses, float* alpha, float* dt,
                                     const float* alpha_start, const float* f_alpha,
                                     const float* dt_min, const float* dt_max, const float* maxstep,
                                     int32_t* n_steps_positive, const int32_t* n_min,
                                     const float* f_dec, const float* f_inc,
                                     const int32_t* uphill_flag, float* vf, float* vv, float* ff,
                                     const int32_t* batch_idx, int32_t compute_reductions,
                                     const uint8_t* active, int32_t n_atoms, int32_t n_systems,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    (void)uphill_flag;
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire: negative size");
    if (n_systems == 0) return NVAMD_OK;
    if (!alpha || !dt || !alpha_start || !f_alpha || !dt_min || !dt_max || !maxstep ||
        !n_steps_positive || !n_min || !f_dec || !f_inc || !vf || !vv || !ff)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire: null per-system buffer");
    if (n_atoms > 0 && (!positions || !velocities || !forces || !masses || !batch_idx))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire: null per-atom buffer");
    size_t need = 0;
    nvamd_fire_workspace_bytes(n_systems, &need);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "fire: workspace %zu < %zu bytes", workspace_bytes, need);
    size_t m = (size_t)n_systems;
    char* w = static_cast<char*>(workspace);
    FireScratch ws;
    ws.flip = reinterpret_cast<int*>(w);
    w += align_up(sizeof(int));
    ws.acc = reinterpret_cast<double*>(w);
    w += align_up(2 * m * 3 * sizeof(double));
    ws.alpha0 = reinterpret_cast<float*>(w);
    w += align_up(m * sizeof(float));
    ws.dt0 = reinterpret_cast<float*>(w);
    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 blk(kBlock);
    dim3 grid_m((n_systems + kBlock - 1) / kBlock);
    // two launches: the sums (per four atoms; its threads also clear the next call's slot and set alpha and dt
    // aside), then the update (per atom and per system).  Without atoms to sum over, or with the caller's sums,
    // a small kernel per system stands in for the first.
    if (compute_reductions && n_atoms > 0) {
        launch_fire_reduce(velocities, forces, batch_idx, nullptr, n_atoms, st, ws, n_systems, alpha, dt);
    } else {
        hipLaunchKernelGGL(fire_import_kernel, grid_m, blk, 0, st, alpha, dt, vf, vv, ff, ws, n_systems,
                           compute_reductions ? 0 : 1);
    }
    const int n_atom_blocks = (n_atoms + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(fire_update_kernel, dim3(n_atom_blocks + (n_systems + kBlock - 1) / kBlock), blk, 0, st, positions,
                       velocities, forces, masses, maxstep, batch_idx, active, alpha, dt, alpha_start, f_alpha, dt_min,
                       dt_max, n_steps_positive, n_min, f_dec, f_inc, vf, vv, ff, ws, compute_reductions ? 1 : 0,
                       n_atoms, n_atom_blocks, n_systems);
    NVAMD_LAUNCH_CHECK("fire launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_fire2_workspace_bytes(int32_t n_systems, size_t* bytes) {
    if (!bytes || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire2 workspace: bad argument");
    size_t m = (size_t)(n_systems > 0 ? n_systems : 1);
    *bytes = align_up(m * 3 * sizeof(double)) + 5 * align_up(m * sizeof(float));
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_fire2_step(float* positions, float* velocities, const float* forces,
                                      const int32_t* batch_idx, float* alpha, float* dt, int32_t* nsteps_inc,
                                      float* vf, float* v_sumsq, float* f_sumsq, float* max_norm,
                                      int32_t delaystep, double dtgrow, double dtshrink, double alphashrink,
                                      double alpha0, double tmax, double tmin, double maxstep,
                                      const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* workspace,
                                      size_t workspace_bytes, void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire2: negative size");
    if (n_systems == 0) return NVAMD_OK;
    if (!alpha || !dt || !nsteps_inc) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire2: null per-system buffer");
    if (n_atoms > 0 && (!positions || !velocities || !forces || !batch_idx))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "fire2: null per-atom buffer");
    size_t need = 0;
    nvamd_fire2_workspace_bytes(n_systems, &need);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "fire2: workspace %zu < %zu bytes", workspace_bytes, need);
    const size_t m = (size_t)n_systems;
    char* w = static_cast<char*>(workspace);
    Fire2Scratch ws;
    ws.acc = reinterpret_cast<double*>(w);
    w += align_up(m * 3 * sizeof(double));
    ws.mix_a = reinterpret_cast<float*>(w);
    w += align_up(m * sizeof(float));
    ws.mix_b = reinterpret_cast<float*>(w);
    w += align_up(m * sizeof(float));
    ws.back = reinterpret_cast<float*>(w);
    w += align_up(m * sizeof(float));
    ws.big = reinterpret_cast<float*>(w);
    w += align_up(m * sizeof(float));
    ws.up = reinterpret_cast<int32_t*>(w);
    const Fire2Params p{delaystep, (float)dtgrow, (float)dtshrink, (float)alphashrink, (float)alpha0,
                        (float)tmax, (float)tmin, (float)maxstep};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 blk(kBlock), grid_m((n_systems + kBlock - 1) / kBlock), grid_n((n_atoms + kBlock - 1) / kBlock);
    const int n3 = 3 * n_systems;
    hipLaunchKernelGGL(fire_clear_kernel, dim3((n3 + kBlock - 1) / kBlock), blk, 0, st, ws.acc, n3);
    if (n_atoms > 0) {
        launch_fire_reduce(velocities, forces, batch_idx, ws.acc, n_atoms, st);
    }
    hipLaunchKernelGGL(fire2_params_kernel, grid_m, blk, 0, st, alpha, dt, nsteps_inc, vf, v_sumsq, f_sumsq, active,
                       ws, p, n_systems);
    if (n_atoms > 0) {
        hipLaunchKernelGGL(fire2_kick_kernel, grid_n, blk, 0, st, positions, velocities, forces, dt, batch_idx,
                           active, ws, n_atoms);
        hipLaunchKernelGGL(fire2_drift_kernel, grid_n, blk, 0, st, positions, velocities, dt, batch_idx, active, ws,
                           (float)maxstep, max_norm, n_atoms);
    }
    NVAMD_LAUNCH_CHECK("fire2 launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_segment_fmax(const float* forces, const int32_t* batch_idx,
                                        int32_t n_atoms, int32_t n_systems, float* fmax,
                                        void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "fmax: negative size");
    if (n_systems == 0) return NVAMD_OK;
    if (!fmax || (n_atoms > 0 && (!forces || !batch_idx)))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "fmax: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(fmax_init_kernel, dim3((n_systems + kBlock - 1) / kBlock), dim3(kBlock), 0, st,
                       fmax, n_systems);
    if (n_atoms > 0)
        hipLaunchKernelGGL(fmax_kernel, dim3((n_atoms + kBlock - 1) / kBlock), dim3(kBlock), 0, st,
                           forces, batch_idx, fmax, n_atoms);
    NVAMD_LAUNCH_CHECK("fmax launch");
    return NVAMD_OK;
}

namespace {
template <typename T>
int32_t status_migrate(const T* values, double threshold, int64_t* status, int64_t source_status, int64_t target_status,
                       int32_t n_systems, void* stream) {
    if (n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "status migrate: negative size");
    if (n_systems == 0) return NVAMD_OK;
    if (!values || !status) return fail(NVAMD_ERR_INVALID_ARGUMENT, "status migrate: null buffer");
    hipLaunchKernelGGL(status_migrate_kernel<T>, dim3((n_systems + kBlock - 1) / kBlock), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), values, (T)threshold, reinterpret_cast<long long*>(status),
                       (long long)source_status, (long long)target_status, n_systems);
    NVAMD_LAUNCH_CHECK("status migrate launch");
    return NVAMD_OK;
}
}  // namespace

NVAMD_EXPORT int32_t nvamd_status_migrate(const float* values, double threshold, int64_t* status,
                                          int64_t source_status, int64_t target_status, int32_t n_systems,
                                          void* stream) {
    return status_migrate<float>(values, threshold, status, source_status, target_status, n_systems, stream);
}

NVAMD_EXPORT int32_t nvamd_status_migrate_f64(const double* values, double threshold, int64_t* status,
                                              int64_t source_status, int64_t target_status, int32_t n_systems,
                                              void* stream) {
    return status_migrate<double>(values, threshold, status, source_status, target_status, n_systems, stream);
}
