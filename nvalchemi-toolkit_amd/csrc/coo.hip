// Dense neighbor matrix -> COO edge list (row-major order: atom ascending, slot ascending).
//
// Reference interface: get_neighbor_list_from_neighbor_matrix as called at
// nvalchemi/neighbors.py:92-103; the in-tree statement of its result is
// nvalchemi/models/_ops/neighbor_filter.py:255-283 (edges (E,2) rows [i, j], CSR pointer
// from the cumulative counts, shifts (E,3)).  Bound: HBM (16 B read + 20 B written per edge).
#include "common.h"
#include "scan.h"

namespace nvamd {
namespace {

constexpr int kBlock = 256;
constexpr int kLanesPerRow = 16;

__global__ __launch_bounds__(kBlock) void coo_fill_kernel(const int32_t* __restrict__ nm,
                                                          const int32_t* __restrict__ shifts,
                                                          const int32_t* __restrict__ edge_ptr,
                                                          int n_atoms, int K, long long cap,
                                                          int32_t* __restrict__ nl,
                                                          int32_t* __restrict__ nl_shifts) {
    int i = (int)((blockIdx.x * (size_t)kBlock + threadIdx.x) / kLanesPerRow);
    int sub = threadIdx.x % kLanesPerRow;
    if (i >= n_atoms) return;
    long long e0 = edge_ptr[i];
    int cnt = edge_ptr[i + 1] - (int)e0;
    const int32_t* row = nm + (size_t)i * K;
    const int32_t* srow = shifts ? shifts + (size_t)i * K * 3 : nullptr;
    for (int k = sub; k < cnt; k += kLanesPerRow) {
        long long e = e0 + k;
        if (e >= cap) break;
        nl[2 * e + 0] = i;
        nl[2 * e + 1] = row[k];
        if (nl_shifts) {
            nl_shifts[3 * e + 0] = srow ? srow[3 * k + 0] : 0;
            nl_shifts[3 * e + 1] = srow ? srow[3 * k + 1] : 0;
            nl_shifts[3 * e + 2] = srow ? srow[3 * k + 2] : 0;
        }
    }
}

// total number of edges and whether it exceeds what the caller's buffers hold
__global__ void coo_count_kernel(const int32_t* __restrict__ edge_ptr, int n_atoms, long long cap,
                                 int32_t* __restrict__ counts) {
    const int e = edge_ptr[n_atoms];
    counts[0] = e;
    counts[1] = (long long)e > cap ? 1 : 0;
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_coo_workspace_bytes(int32_t n_atoms, size_t* bytes) {
    if (!bytes || n_atoms < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "coo workspace: bad argument");
    *bytes = align_up(((size_t)scan::tiles_for((size_t)(n_atoms > 0 ? n_atoms : 1)) + 1) * sizeof(int));
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_edge_ptr(const int32_t* num_neighbors, int32_t n_atoms,
                                       int32_t max_neighbors, int32_t* edge_ptr, void* workspace,
                                       size_t workspace_bytes, void* stream) {
    if (n_atoms < 0 || max_neighbors < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "edge_ptr: negative size");
    if (!edge_ptr || (n_atoms > 0 && !num_neighbors))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "edge_ptr: null buffer");
    size_t need = 0;
    nvamd_coo_workspace_bytes(n_atoms, &need);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "edge_ptr: workspace %zu < %zu bytes", workspace_bytes, need);
    if ((long long)n_atoms * max_neighbors > 0x7fffffffLL)
        return fail(NVAMD_ERR_UNSUPPORTED, "edge_ptr: N*K exceeds int32 edge offsets");
    hipStream_t st = static_cast<hipStream_t>(stream);
    scan::exclusive(scan::LoadClamped{num_neighbors, max_neighbors}, nullptr, n_atoms,
                    scan::tiles_for((size_t)n_atoms), static_cast<int*>(workspace), edge_ptr, st);
    NVAMD_LAUNCH_CHECK("edge_ptr launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_matrix_to_coo(const int32_t* neighbor_matrix,
                                            const int32_t* neighbor_matrix_shifts,
                                            const int32_t* edge_ptr, int32_t n_atoms,
                                            int32_t max_neighbors, int64_t edge_capacity,
                                            int32_t* neighbor_list, int32_t* neighbor_list_shifts,
                                            void* stream) {
    if (n_atoms < 0 || max_neighbors < 0 || edge_capacity < 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "coo: negative size");
    if (n_atoms == 0 || edge_capacity == 0 || max_neighbors == 0) return NVAMD_OK;
    if (!neighbor_matrix || !edge_ptr || !neighbor_list)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "coo: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    size_t threads = (size_t)n_atoms * kLanesPerRow;
    hipLaunchKernelGGL(coo_fill_kernel, dim3((unsigned)((threads + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       st, neighbor_matrix, neighbor_matrix_shifts, edge_ptr, n_atoms, max_neighbors,
                       (long long)edge_capacity, neighbor_list, neighbor_list_shifts);
    NVAMD_LAUNCH_CHECK("coo launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_coo_from_matrix(const int32_t* neighbor_matrix, const int32_t* neighbor_matrix_shifts,
                                              const int32_t* num_neighbors, int32_t n_atoms, int32_t max_neighbors,
                                              int64_t edge_capacity, int32_t* edge_ptr, int32_t* neighbor_list,
                                              int32_t* neighbor_list_shifts, int32_t* counts, void* workspace,
                                              size_t workspace_bytes, void* stream) {
    if (!counts) return fail(NVAMD_ERR_INVALID_ARGUMENT, "coo: null counts");
    int32_t rc = nvamd_nl_edge_ptr(num_neighbors, n_atoms, max_neighbors, edge_ptr, workspace, workspace_bytes, stream);
    if (rc != NVAMD_OK) return rc;
    rc = nvamd_nl_matrix_to_coo(neighbor_matrix, neighbor_matrix_shifts, edge_ptr, n_atoms, max_neighbors,
                                edge_capacity, neighbor_list, neighbor_list_shifts, stream);
    if (rc != NVAMD_OK) return rc;
    hipLaunchKernelGGL(coo_count_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), edge_ptr, n_atoms,
                       (long long)edge_capacity, counts);
    NVAMD_LAUNCH_CHECK("coo count launch");
    return NVAMD_OK;
}
