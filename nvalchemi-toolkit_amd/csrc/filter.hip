// Filtering a neighbor list down to a tighter cutoff, gfx950.
//
// Reference interface: filter_neighbor_matrix (nvalchemi/models/_ops/neighbor_filter.py:43-144)
// and the distance test of filter_neighbor_list (:147-224), both in-tree Torch: an entry is kept
// iff it is not padding (index below fill_value) and |r_j - r_i + S . cell|^2 < cutoff^2; kept
// entries move to the front of their row in their order, the rest of the row becomes fill_value
// with zero shifts, and the count is the number kept.  Every slot of the row is examined
// (validity comes from the index alone, as in the reference, not from num_neighbors).
//
// The distance is the library's one expression (double on the float32 inputs, geom.h); the
// reference evaluates it in float32, so the two can differ only for pairs within float32
// rounding of the cutoff.
//
// Bound: HBM, 16 B read and up to 16 B written per slot plus one gathered position per valid
// slot.  One wavefront per row: 64 slots per step, a ballot and a prefix count give every kept
// entry its place.
#include "common.h"
#include "geom.h"

namespace nvamd {
namespace {

constexpr int kBlock = 256;

__global__ __launch_bounds__(kBlock) void filter_matrix_kernel(const float* __restrict__ pos,
                                                               const float* __restrict__ cells, int cell_stride,
                                                               const int32_t* __restrict__ nm,
                                                               const int32_t* __restrict__ shifts,
                                                               const int32_t* __restrict__ bidx, int n_atoms, int K,
                                                               int fill, double rc2, int32_t* __restrict__ out_nm,
                                                               int32_t* __restrict__ out_nn,
                                                               int32_t* __restrict__ out_shifts) {
    const int i = (int)((blockIdx.x * (size_t)kBlock + threadIdx.x) / kWave);
    if (i >= n_atoms) return;
    const int lane = lane_id();
    const float xi = pos[3 * (size_t)i], yi = pos[3 * (size_t)i + 1], zi = pos[3 * (size_t)i + 2];
    const bool shifted = cells != nullptr && shifts != nullptr;
    const float* cell = shifted ? cells + (size_t)cell_stride * (bidx ? bidx[i] : 0) : nullptr;
    const int32_t* row = nm + (size_t)i * K;
    const int32_t* srow = shifts ? shifts + (size_t)i * K * 3 : nullptr;
    int32_t* orow = out_nm + (size_t)i * K;
    int32_t* osrow = out_shifts ? out_shifts + (size_t)i * K * 3 : nullptr;
    int kept = 0;
    for (int k0 = 0; k0 < K; k0 += kWave) {
        const int k = k0 + lane;
        bool keep = false;
        int j = fill, s0 = 0, s1 = 0, s2 = 0;
        if (k < K) {
            j = row[k];
            if (srow) {
                s0 = srow[3 * k + 0];
                s1 = srow[3 * k + 1];
                s2 = srow[3 * k + 2];
            }
            if (j < fill) {
                // (the reference clamps the index into range before the gather)
                const int js = j < 0 ? 0 : (j >= n_atoms ? n_atoms - 1 : j);
                const float* pj = pos + 3 * (size_t)js;
                double tx = 0.0, ty = 0.0, tz = 0.0, d0, d1, d2;
                if (shifted) shift_vector(cell, s0, s1, s2, tx, ty, tz);
                keep = pair_d2_shifted(xi, yi, zi, pj[0], pj[1], pj[2], tx, ty, tz, d0, d1, d2) < rc2;
            }
        }
        const unsigned long long m = __ballot(keep);
        if (keep) {
            const int at = kept + __popcll(m & ((1ull << lane) - 1ull));
            orow[at] = j;
            if (osrow) {
                osrow[3 * at + 0] = s0;
                osrow[3 * at + 1] = s1;
                osrow[3 * at + 2] = s2;
            }
        }
        kept += __popcll(m);
    }
    // the rest of the row is padding
    for (int k = kept + lane; k < K; k += kWave) {
        orow[k] = fill;
        if (osrow) {
            osrow[3 * k + 0] = 0;
            osrow[3 * k + 1] = 0;
            osrow[3 * k + 2] = 0;
        }
    }
    if (lane == 0) out_nn[i] = kept;
}

__global__ __launch_bounds__(kBlock) void filter_coo_flags_kernel(const float* __restrict__ pos,
                                                                  const float* __restrict__ cells, int cell_stride,
                                                                  const int32_t* __restrict__ nl,
                                                                  const int32_t* __restrict__ nl_shifts,
                                                                  const int32_t* __restrict__ bidx, long long n_edges,
                                                                  double rc2, uint8_t* __restrict__ keep) {
    const long long e = blockIdx.x * (long long)kBlock + threadIdx.x;
    if (e >= n_edges) return;
    const int i = nl[2 * e], j = nl[2 * e + 1];
    const float* pi = pos + 3 * (size_t)i;
    const float* pj = pos + 3 * (size_t)j;
    double tx = 0.0, ty = 0.0, tz = 0.0, d0, d1, d2;
    if (cells && nl_shifts) {
        // (per-system cells are looked up by the source atom's system)
        const float* cell = cells + (size_t)cell_stride * (bidx ? bidx[i] : 0);
        shift_vector(cell, nl_shifts[3 * e], nl_shifts[3 * e + 1], nl_shifts[3 * e + 2], tx, ty, tz);
    }
    keep[e] = pair_d2_shifted(pi[0], pi[1], pi[2], pj[0], pj[1], pj[2], tx, ty, tz, d0, d1, d2) < rc2 ? 1 : 0;
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_nl_filter_matrix(const float* positions, const float* cells, int32_t per_system_cells,
                                            const int32_t* neighbor_matrix, const int32_t* neighbor_matrix_shifts,
                                            const int32_t* batch_idx, int32_t n_atoms, int32_t max_neighbors,
                                            int32_t fill_value, double cutoff, int32_t* out_neighbor_matrix,
                                            int32_t* out_num_neighbors, int32_t* out_shifts, void* stream) {
    if (n_atoms < 0 || max_neighbors < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: negative size");
    if (!(cutoff >= 0.0)) return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: cutoff must be non-negative");
    if (n_atoms == 0) return NVAMD_OK;
    if (!positions || !out_num_neighbors || (max_neighbors > 0 && (!neighbor_matrix || !out_neighbor_matrix)))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: null buffer");
    if (neighbor_matrix_shifts && !out_shifts) return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: shifts without output");
    if (per_system_cells && cells && neighbor_matrix_shifts && !batch_idx)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: batch_idx is required with per-system cells");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t threads = (size_t)n_atoms * kWave;
    hipLaunchKernelGGL(filter_matrix_kernel, dim3((unsigned)((threads + kBlock - 1) / kBlock)), dim3(kBlock), 0, st,
                       positions, cells, per_system_cells ? 9 : 0, neighbor_matrix, neighbor_matrix_shifts,
                       per_system_cells ? batch_idx : nullptr, n_atoms, max_neighbors, fill_value, cutoff * cutoff,
                       out_neighbor_matrix, out_num_neighbors, neighbor_matrix_shifts ? out_shifts : nullptr);
    NVAMD_LAUNCH_CHECK("filter launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_filter_coo_flags(const float* positions, const float* cells, int32_t per_system_cells,
                                               const int32_t* neighbor_list, const int32_t* neighbor_list_shifts,
                                               const int32_t* batch_idx, int64_t n_edges, double cutoff,
                                               uint8_t* keep, void* stream) {
    if (n_edges < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: negative size");
    if (!(cutoff >= 0.0)) return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: cutoff must be non-negative");
    if (n_edges == 0) return NVAMD_OK;
    if (!positions || !neighbor_list || !keep) return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: null buffer");
    if (per_system_cells && cells && neighbor_list_shifts && !batch_idx)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "filter: batch_idx is required with per-system cells");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(filter_coo_flags_kernel, dim3((unsigned)((n_edges + kBlock - 1) / kBlock)), dim3(kBlock), 0, st,
                       positions, cells, per_system_cells ? 9 : 0, neighbor_list, neighbor_list_shifts,
                       per_system_cells ? batch_idx : nullptr, (long long)n_edges, cutoff * cutoff, keep);
    NVAMD_LAUNCH_CHECK("filter launch");
    return NVAMD_OK;
}
