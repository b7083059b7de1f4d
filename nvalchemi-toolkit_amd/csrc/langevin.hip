// BAOAB Langevin half step (B-A-O-A) for gfx950.
//
// Reference interface: nvalchemi::langevin_half_step (nvalchemi/dynamics/_ops/langevin.py:52-117),
// called by NVTLangevin.pre_update (nvalchemi/dynamics/integrators/nvt_langevin.py:160-181) with
// kT in eV, the friction in 1 / internal time and random_seed + step_count as the seed.  The final
// B step, nvalchemi::langevin_finalize (:134-170), is the velocity half kick of velocity Verlet
// (nvamd_vv_velocity_finalize).
//
// Per atom, in the arrays' own type (float32, or float64 through nvamd_langevin_half_step_f64: the reference's
// op takes both, nvalchemi/dynamics/_ops/_bridge.py), one rounding per operation:
//   B   v <- v + (F/m) (dt/2)
//   A   r <- r + v (dt/2)
//   O   v <- c1 v + c2 xi,   c1 = exp(-gamma dt),  c2 = sqrt((kT/m) (1 - c1^2)),  xi ~ N(0,1)^3
//   A   r <- r + v (dt/2)
// c1 and c2 are evaluated in double and rounded once.  The three normal deviates of atom i come
// from one Philox4x32-10 block with key = the 64-bit seed and counter = (i, 0, 0, 0), through the
// Box-Muller transform in double: the stream depends on the seed and the atom index only, not on
// the launch shape.  (The reference's own generator is inside its kernel library: its random
// stream cannot be matched, only its distribution.)
//
// Bound: HBM, 68 B/atom like the first velocity-Verlet half; the generator costs about 150
// integer and 40 double-precision instructions per atom, hidden under the streams.
#include "common.h"

namespace nvamd {
namespace {

constexpr int kBlock = 256;

struct Philox {
    uint32_t c[4];
};

__device__ __forceinline__ Philox philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                uint32_t k1) {
    constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint32_t hi0 = __umulhi(M0, c0), lo0 = M0 * c0;
        const uint32_t hi1 = __umulhi(M1, c2), lo1 = M1 * c2;
        c0 = hi1 ^ c1 ^ k0;
        c1 = lo1;
        c2 = hi0 ^ c3 ^ k1;
        c3 = lo0;
        k0 += W0;
        k1 += W1;
    }
    return Philox{{c0, c1, c2, c3}};
}

// two independent standard normals from two 32-bit words: u1 in (0, 1], u2 in [0, 1)
__device__ __forceinline__ void box_muller(uint32_t a, uint32_t b, double& n0, double& n1) {
    const double u1 = ((double)a + 1.0) * (1.0 / 4294967296.0);
    const double u2 = (double)b * (1.0 / 4294967296.0);
    const double radius = sqrt(-2.0 * log(u1));
    const double angle = 6.283185307179586476925286766559 * u2;
    n0 = radius * cos(angle);
    n1 = radius * sin(angle);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void langevin_half_step_kernel(
    T* __restrict__ pos, T* __restrict__ vel, const T* __restrict__ frc,
    const T* __restrict__ masses, const T* __restrict__ dt, const T* __restrict__ kT,
    const T* __restrict__ friction, uint32_t seed_lo, uint32_t seed_hi, const int32_t* __restrict__ bidx,
    const uint8_t* __restrict__ active, int n_atoms) {
#pragma clang fp contract(off)
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const int s = bidx[i];
    if (active && !active[s]) return;
    const T m = masses[i];
    const T h = dt[s];
    const T hh = (T)0.5 * h;
    const double c1d = exp(-(double)friction[s] * (double)h);
    const T c1 = (T)c1d;
    const T c2 = (T)sqrt(((double)kT[s] / (double)m) * (1.0 - c1d * c1d));
    const Philox rnd = philox4x32_10((uint32_t)i, 0u, 0u, 0u, seed_lo, seed_hi);
    double xi[4];
    box_muller(rnd.c[0], rnd.c[1], xi[0], xi[1]);
    box_muller(rnd.c[2], rnd.c[3], xi[2], xi[3]);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        const size_t e = 3 * (size_t)i + a;
        T v = vel[e], r = pos[e];
        const T acc = frc[e] / m;
        v = v + acc * hh;
        r = r + v * hh;
        v = c1 * v + c2 * (T)xi[a];
        r = r + v * hh;
        vel[e] = v;
        pos[e] = r;
    }
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

namespace {

template <typename T>
int32_t langevin_half_step(T* positions, T* velocities, const T* forces, const T* masses, const T* dt, const T* kT,
                           const T* friction, uint64_t random_seed, const int32_t* batch_idx, const uint8_t* active,
                           int32_t n_atoms, int32_t n_systems, void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "langevin: negative size");
    if (n_atoms == 0) return NVAMD_OK;
    if (!positions || !velocities || !forces || !masses || !dt || !kT || !friction || !batch_idx)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "langevin: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(langevin_half_step_kernel<T>, dim3((n_atoms + kBlock - 1) / kBlock), dim3(kBlock), 0, st,
                       positions, velocities, forces, masses, dt, kT, friction, (uint32_t)(random_seed & 0xffffffffu),
                       (uint32_t)(random_seed >> 32), batch_idx, active, n_atoms);
    NVAMD_LAUNCH_CHECK("langevin launch");
    return NVAMD_OK;
}

}  // namespace

NVAMD_EXPORT int32_t nvamd_langevin_half_step(float* positions, float* velocities, const float* forces,
                                              const float* masses, const float* dt, const float* kT,
                                              const float* friction, uint64_t random_seed,
                                              const int32_t* batch_idx, const uint8_t* active, int32_t n_atoms,
                                              int32_t n_systems, void* stream) {
    return langevin_half_step<float>(positions, velocities, forces, masses, dt, kT, friction, random_seed, batch_idx,
                                     active, n_atoms, n_systems, stream);
}

NVAMD_EXPORT int32_t nvamd_langevin_half_step_f64(double* positions, double* velocities, const double* forces,
                                                  const double* masses, const double* dt, const double* kT,
                                                  const double* friction, uint64_t random_seed,
                                                  const int32_t* batch_idx, const uint8_t* active, int32_t n_atoms,
                                                  int32_t n_systems, void* stream) {
    return langevin_half_step<double>(positions, velocities, forces, masses, dt, kT, friction, random_seed, batch_idx,
                                      active, n_atoms, n_systems, stream);
}
