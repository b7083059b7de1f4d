// Verlet-skin displacement test and periodic wrapping for gfx950.
//
// Reference interfaces: nvalchemi::_batch_neighbor_list_rebuild_inplace
// (nvalchemi/dynamics/_ops/neighbor_list_rebuild.py:37-139) and nvalchemi_hooks::wrap_positions with
// the per-axis masking that follows it (nvalchemi/hooks/periodic.py:42-114).  Both are streaming
// passes over the atoms (24 and 24 bytes per atom); the per-system cell is inverted by every
// thread that needs it (a few dozen flops) rather than read from a second array.
#include "common.h"
#include "geom.h"

namespace nvamd {
namespace {

constexpr int kBlock = 256;

__global__ __launch_bounds__(kBlock) void clear_flags_kernel(uint8_t* flags, int n) {
    int t = blockIdx.x * kBlock + threadIdx.x;
    if (t < n) flags[t] = 0;
}

// T: the type the positions and cells are stored in; the arithmetic is double either way (float32 inputs
// convert exactly), and a float64 result is stored as it is.
template <typename T>
__global__ __launch_bounds__(kBlock) void displacement_kernel(const T* __restrict__ ref,
                                                              const T* __restrict__ cur,
                                                              const int32_t* __restrict__ bidx,
                                                              const T* __restrict__ cell,
                                                              const uint8_t* __restrict__ pbc, int n_atoms,
                                                              double thr2, uint8_t* flags) {
#pragma clang fp contract(off)
    int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const int s = bidx[i];
    double d0 = (double)cur[3 * (size_t)i + 0] - (double)ref[3 * (size_t)i + 0];
    double d1 = (double)cur[3 * (size_t)i + 1] - (double)ref[3 * (size_t)i + 1];
    double d2 = (double)cur[3 * (size_t)i + 2] - (double)ref[3 * (size_t)i + 2];
    if (cell) {
        const uint8_t* p = pbc + 3 * (size_t)s;
        if (p[0] | p[1] | p[2]) {
            double h[9], hinv[9];
#pragma unroll
            for (int k = 0; k < 9; ++k) h[k] = (double)cell[9 * (size_t)s + k];
            inv3(h, hinv);
            double f0 = (d0 * hinv[0] + d1 * hinv[3]) + d2 * hinv[6];
            double f1 = (d0 * hinv[1] + d1 * hinv[4]) + d2 * hinv[7];
            double f2 = (d0 * hinv[2] + d1 * hinv[5]) + d2 * hinv[8];
            if (p[0]) f0 -= rint(f0);
            if (p[1]) f1 -= rint(f1);
            if (p[2]) f2 -= rint(f2);
            d0 = (f0 * h[0] + f1 * h[3]) + f2 * h[6];
            d1 = (f0 * h[1] + f1 * h[4]) + f2 * h[7];
            d2 = (f0 * h[2] + f1 * h[5]) + f2 * h[8];
        }
    }
    const double r2 = (d0 * d0 + d1 * d1) + d2 * d2;
    if (r2 > thr2) flags[s] = 1;  // (every writer stores the same byte)
}

template <typename T>
__global__ __launch_bounds__(kBlock) void refresh_reference_kernel(T* __restrict__ ref,
                                                                   const T* __restrict__ cur,
                                                                   const int32_t* __restrict__ bidx,
                                                                   const uint8_t* __restrict__ flags, size_t n3) {
    size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= n3) return;
    if (flags[bidx[t / 3]]) ref[t] = cur[t];
}

template <typename T>
__global__ __launch_bounds__(kBlock) void wrap_kernel(T* __restrict__ pos, const T* __restrict__ cell,
                                                      const uint8_t* __restrict__ pbc,
                                                      const int32_t* __restrict__ bidx, int n_atoms) {
#pragma clang fp contract(off)
    int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_atoms) return;
    const int s = bidx[i];
    const uint8_t* p = pbc + 3 * (size_t)s;
    if (!(p[0] | p[1] | p[2])) return;
    double h[9], hinv[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) h[k] = (double)cell[9 * (size_t)s + k];
    inv3(h, hinv);
    T* r = pos + 3 * (size_t)i;
    const double x = (double)r[0], y = (double)r[1], z = (double)r[2];
    double f0 = (x * hinv[0] + y * hinv[3]) + z * hinv[6];
    double f1 = (x * hinv[1] + y * hinv[4]) + z * hinv[7];
    double f2 = (x * hinv[2] + y * hinv[5]) + z * hinv[8];
    f0 -= floor(f0);
    f1 -= floor(f1);
    f2 -= floor(f2);
    const double wx = (f0 * h[0] + f1 * h[3]) + f2 * h[6];
    const double wy = (f0 * h[1] + f1 * h[4]) + f2 * h[7];
    const double wz = (f0 * h[2] + f1 * h[5]) + f2 * h[8];
    // the reference keeps the old Cartesian component wherever that component's flag is clear
    if (p[0]) r[0] = (T)wx;
    if (p[1]) r[1] = (T)wy;
    if (p[2]) r[2] = (T)wz;
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

template <typename T>
static int32_t rebuild_check_impl(T* reference_positions, const T* current_positions, const int32_t* batch_idx,
                                  const T* cell, const uint8_t* pbc, int32_t n_atoms, int32_t n_systems,
                                  double threshold, int32_t update_reference, uint8_t* rebuild_flags, void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "rebuild check: negative size");
    if (!(threshold >= 0.0)) return fail(NVAMD_ERR_INVALID_ARGUMENT, "rebuild check: threshold must not be negative");
    if (n_systems == 0) return NVAMD_OK;
    if (!rebuild_flags) return fail(NVAMD_ERR_INVALID_ARGUMENT, "rebuild check: null rebuild_flags");
    if ((cell == nullptr) != (pbc == nullptr))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "rebuild check: cell and pbc must be given together");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(clear_flags_kernel, dim3((n_systems + kBlock - 1) / kBlock), dim3(kBlock), 0, st,
                       rebuild_flags, n_systems);
    if (n_atoms > 0) {
        if (!reference_positions || !current_positions || !batch_idx)
            return fail(NVAMD_ERR_INVALID_ARGUMENT, "rebuild check: null buffer");
        hipLaunchKernelGGL(displacement_kernel<T>, dim3((n_atoms + kBlock - 1) / kBlock), dim3(kBlock), 0, st,
                           reference_positions, current_positions, batch_idx, cell, pbc, n_atoms,
                           threshold * threshold, rebuild_flags);
        if (update_reference) {
            const size_t n3 = 3 * (size_t)n_atoms;
            hipLaunchKernelGGL(refresh_reference_kernel<T>, dim3((unsigned)((n3 + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                               st, reference_positions, current_positions, batch_idx, rebuild_flags, n3);
        }
    }
    NVAMD_LAUNCH_CHECK("rebuild check launch");
    return NVAMD_OK;
}

template <typename T>
static int32_t wrap_impl(T* positions, const T* cell, const uint8_t* pbc, const int32_t* batch_idx, int32_t n_atoms,
                         int32_t n_systems, void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "wrap: negative size");
    if (n_atoms == 0 || n_systems == 0) return NVAMD_OK;
    if (!positions || !cell || !pbc || !batch_idx) return fail(NVAMD_ERR_INVALID_ARGUMENT, "wrap: null buffer");
    hipLaunchKernelGGL(wrap_kernel<T>, dim3((n_atoms + kBlock - 1) / kBlock), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), positions, cell, pbc, batch_idx, n_atoms);
    NVAMD_LAUNCH_CHECK("wrap launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_rebuild_check(float* reference_positions, const float* current_positions,
                                            const int32_t* batch_idx, const float* cell, const uint8_t* pbc,
                                            int32_t n_atoms, int32_t n_systems, double threshold,
                                            int32_t update_reference, uint8_t* rebuild_flags, void* stream) {
    return rebuild_check_impl<float>(reference_positions, current_positions, batch_idx, cell, pbc, n_atoms, n_systems,
                                     threshold, update_reference, rebuild_flags, stream);
}

NVAMD_EXPORT int32_t nvamd_nl_rebuild_check_f64(double* reference_positions, const double* current_positions,
                                                const int32_t* batch_idx, const double* cell, const uint8_t* pbc,
                                                int32_t n_atoms, int32_t n_systems, double threshold,
                                                int32_t update_reference, uint8_t* rebuild_flags, void* stream) {
    return rebuild_check_impl<double>(reference_positions, current_positions, batch_idx, cell, pbc, n_atoms, n_systems,
                                      threshold, update_reference, rebuild_flags, stream);
}

NVAMD_EXPORT int32_t nvamd_wrap_positions(float* positions, const float* cell, const uint8_t* pbc,
                                          const int32_t* batch_idx, int32_t n_atoms, int32_t n_systems,
                                          void* stream) {
    return wrap_impl<float>(positions, cell, pbc, batch_idx, n_atoms, n_systems, stream);
}

NVAMD_EXPORT int32_t nvamd_wrap_positions_f64(double* positions, const double* cell, const uint8_t* pbc,
                                              const int32_t* batch_idx, int32_t n_atoms, int32_t n_systems,
                                              void* stream) {
    return wrap_impl<double>(positions, cell, pbc, batch_idx, n_atoms, n_systems, stream);
}
