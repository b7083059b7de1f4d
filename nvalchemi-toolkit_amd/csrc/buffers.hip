// Masked copy and in-place compaction of per-system rows and of per-system segments, gfx950.
//
// Reference interfaces (nvalchemi/data/buffer_kernels.py): put_masked_per_system (:1171-1220),
// compute_put_fit_mask_per_system (:1139-1169), defrag_per_system (:1294-1333),
// put_masked_segmented (:1442-1527), compute_put_fit_mask_segmented (:558-610) and
// defrag_segmented (:1700-1741) -- the data movement under Batch.put / Batch.defrag
// (nvalchemi/data/batch.py:876-985), i.e. the refill of finished systems during a run.
//
// Rows are opaque: a row is row_bytes bytes, whatever the element type (the reference has one
// overload per dtype; source and destination always share it).  Every operation is a plan kernel
// -- one workgroup that scans the masks and lengths of the systems, a few thousand at most -- and
// a data kernel over the rows in 16-, 4- or 1-byte units, whichever the row size and the
// pointers allow.  Bound: HBM; a put reads and writes the moved rows once, a compaction moves
// the kept rows to scratch and back (the kept rows cannot be moved in place by independent
// workgroups: a destination may still hold rows that another workgroup has yet to read).
#include "common.h"

namespace nvamd {
namespace {

constexpr int kPlanBlock = 1024;
constexpr int kBlock = 256;

struct Plan {
    int32_t count;      // masked (put) or kept (defrag) systems
    int32_t max_copy;   // rows a per-system put may move
    int32_t first_empty;
    int32_t base;       // first free element of a segmented destination
    int32_t n_fit;      // segments a segmented put moves
    int32_t total_kept; // elements a segmented compaction keeps
};

struct Scratch {
    Plan* plan;
    int32_t* a;    // (n + 1) scan of the mask / element offset of a segment in its destination
    int32_t* b;    // (n + 1) fits flag / new segment boundaries
    char* temp;    // staging copy of the data for the compactions
};

size_t carve(Scratch* s, char* base, size_t n, size_t data_bytes) {
    size_t off = 0;
    if (s) s->plan = reinterpret_cast<Plan*>(base + off);
    off += align_up(sizeof(Plan));
    if (s) s->a = reinterpret_cast<int32_t*>(base + off);
    off += align_up((n + 1) * sizeof(int32_t));
    if (s) s->b = reinterpret_cast<int32_t*>(base + off);
    off += align_up((n + 1) * sizeof(int32_t));
    if (s) s->temp = base + off;
    off += align_up(data_bytes > 0 ? data_bytes : 1);
    return off;
}

// exclusive scan of one value per thread over the workgroup; returns the total through `total`
__device__ __forceinline__ int block_scan(int v, int& total) {
    __shared__ int wave_sums[kPlanBlock / kWave];
    const int lane = lane_id(), wave = threadIdx.x / kWave;
    int inc = v;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        int t = __shfl_up(inc, o, kWave);
        if (lane >= o) inc += t;
    }
    __syncthreads();  // (the previous round's readers are done with wave_sums)
    if (lane == kWave - 1) wave_sums[wave] = inc;
    __syncthreads();
    int before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kPlanBlock / kWave; ++w) {
        const int s = wave_sums[w];
        if (w < wave) before += s;
        all += s;
    }
    total = all;
    return before + inc - v;
}

// out[i] = exclusive prefix sum of value(i) over 0..n-1, out[n] = the total; one workgroup
template <class F>
__device__ __forceinline__ int scan_all(int n, int32_t* out, F value) {
    int carry = 0;
    for (int i0 = 0; i0 < n; i0 += kPlanBlock) {
        const int i = i0 + (int)threadIdx.x;
        const int v = i < n ? value(i) : 0;
        int total;
        const int ex = block_scan(v, total);
        if (i < n) out[i] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) out[n] = carry;
    return carry;
}

// ---- rows (one per system) ----------------------------------------------------------------

__global__ __launch_bounds__(kPlanBlock) void put_rows_plan_kernel(const uint8_t* __restrict__ src_mask, int n_src,
                                                                   const uint8_t* __restrict__ dest_mask, int n_dest,
                                                                   Scratch s) {
    __shared__ int sh_empty, sh_first;
    if (threadIdx.x == 0) {
        sh_empty = 0;
        sh_first = n_dest;
    }
    const int masked = scan_all(n_src, s.a, [&](int i) { return src_mask[i] ? 1 : 0; });
    int empty = 0, first = n_dest;
    for (int i = threadIdx.x; i < n_dest; i += kPlanBlock)
        if (!dest_mask[i]) {
            ++empty;
            first = first < i ? first : i;
        }
    __syncthreads();
    if (empty) {
        atomicAdd(&sh_empty, empty);
        atomicMin(&sh_first, first);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        s.plan->count = masked;
        s.plan->max_copy = masked < sh_empty ? masked : sh_empty;
        s.plan->first_empty = sh_first;
    }
}

// the masked rows that fit go to consecutive slots from the first empty one
template <class U>
__global__ __launch_bounds__(kBlock) void put_rows_copy_kernel(const U* __restrict__ src,
                                                               const uint8_t* __restrict__ src_mask, U* __restrict__ dest,
                                                               uint8_t* __restrict__ dest_mask,
                                                               uint8_t* __restrict__ copied, int n_src, int upr,
                                                               Scratch s) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t i = t / (size_t)upr;
    if (i >= (size_t)n_src) return;
    const int u = (int)(t - i * upr);
    const int rank = s.a[i];
    if (!src_mask[i] || rank >= s.plan->max_copy) return;
    const size_t slot = (size_t)s.plan->first_empty + rank;
    dest[slot * upr + u] = src[i * upr + u];
    if (u == 0) {
        dest_mask[slot] = 1;
        copied[i] = 1;
    }
}

__global__ __launch_bounds__(kBlock) void fit_rows_kernel(const uint8_t* __restrict__ src_mask,
                                                          uint8_t* __restrict__ fit, int n_src, Scratch s) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_src) return;
    fit[i] = (src_mask[i] && s.a[i] < s.plan->max_copy) ? 1 : 0;
}

__global__ __launch_bounds__(kPlanBlock) void defrag_rows_plan_kernel(const uint8_t* __restrict__ copied, int n,
                                                                      Scratch s) {
    const int kept = scan_all(n, s.a, [&](int i) { return copied[i] ? 0 : 1; });
    if (threadIdx.x == 0) s.plan->count = kept;
}

template <class U>
__global__ __launch_bounds__(kBlock) void defrag_rows_scatter_kernel(const U* __restrict__ src,
                                                                     const uint8_t* __restrict__ copied, int n, int upr,
                                                                     Scratch s) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t i = t / (size_t)upr;
    if (i >= (size_t)n || copied[i]) return;
    const int u = (int)(t - i * upr);
    reinterpret_cast<U*>(s.temp)[(size_t)s.a[i] * upr + u] = src[i * upr + u];
}

// kept rows back to the front, zeros behind them, and the flags say which rows are now free
template <class U>
__global__ __launch_bounds__(kBlock) void defrag_rows_back_kernel(U* __restrict__ src, uint8_t* __restrict__ copied,
                                                                  int n, int upr, Scratch s) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t i = t / (size_t)upr;
    if (i >= (size_t)n) return;
    const int u = (int)(t - i * upr);
    const bool live = (int)i < s.plan->count;
    U zero;
    __builtin_memset(&zero, 0, sizeof(U));
    src[i * upr + u] = live ? reinterpret_cast<const U*>(s.temp)[i * upr + u] : zero;
    if (u == 0) copied[i] = live ? 0 : 1;
}

// ---- segments (a run of rows per system) --------------------------------------------------

// system of element r: the last i with ptr[i] <= r (empty segments are skipped over)
__device__ __forceinline__ int segment_of(const int32_t* __restrict__ ptr, int n, int r) {
    int lo = 0, hi = n;  // invariant: ptr[lo] <= r < ptr[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (ptr[mid] <= r) lo = mid;
        else hi = mid;
    }
    return lo;
}

// Offsets of the masked segments behind the destination's last one, which of them fit, and --
// with `commit` -- the destination's new boundaries and the flags of the moved segments.
__global__ __launch_bounds__(kPlanBlock) void put_segments_plan_kernel(const int32_t* __restrict__ src_ptr,
                                                                       const uint8_t* __restrict__ src_mask, int n,
                                                                       int32_t* __restrict__ dest_ptr, int n_dest_segments,
                                                                       int dest_capacity, uint8_t* __restrict__ copied,
                                                                       uint8_t* __restrict__ fit_mask,
                                                                       int32_t* __restrict__ new_num_dest, int commit,
                                                                       Scratch s) {
    scan_all(n, s.a, [&](int i) { return src_mask[i] ? src_ptr[i + 1] - src_ptr[i] : 0; });
    __syncthreads();
    const int base = dest_ptr[n_dest_segments];
    auto fits = [&](int i) {
        return (src_mask[i] && base + s.a[i] + (src_ptr[i + 1] - src_ptr[i]) <= dest_capacity) ? 1 : 0;
    };
    // rank of a fitting segment among the fitting ones (they are a prefix of the masked ones)
    __shared__ int sh_nfit;
    int carry = 0;
    for (int i0 = 0; i0 < n; i0 += kPlanBlock) {
        const int i = i0 + (int)threadIdx.x;
        const int f = i < n ? fits(i) : 0;
        int total;
        const int rank = carry + block_scan(f, total);
        carry += total;
        if (i < n) {
            s.b[i] = f;
            if (fit_mask) fit_mask[i] = (uint8_t)f;
            if (f && commit) {
                copied[i] = 1;
                dest_ptr[n_dest_segments + 1 + rank] = base + s.a[i] + (src_ptr[i + 1] - src_ptr[i]);
            }
        }
    }
    if (threadIdx.x == 0) sh_nfit = carry;
    __syncthreads();
    const int n_fit = sh_nfit;
    if (threadIdx.x == 0) {
        s.plan->base = base;
        s.plan->n_fit = n_fit;
        if (new_num_dest) *new_num_dest = n_dest_segments + n_fit;
        // (the reference leaves one more copy of the last boundary behind the new ones)
        if (commit && n_fit > 0) dest_ptr[n_dest_segments + 1 + n_fit] = dest_ptr[n_dest_segments + n_fit];
    }
}

template <class U>
__global__ __launch_bounds__(kBlock) void put_segments_copy_kernel(const U* __restrict__ src,
                                                                   const int32_t* __restrict__ src_ptr, int n,
                                                                   int total_rows, U* __restrict__ dest, int upr,
                                                                   int upt, Scratch s) {
    // a thread moves upt units of a row: the whole of a narrow row (one search per row), one unit
    // of a wide one (coalesced)
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const int tpr = upr / upt;
    const size_t r = t / (size_t)tpr;
    if (r >= (size_t)total_rows) return;
    const int u0 = (int)(t - r * tpr) * upt;
    if ((int)r < src_ptr[0] || (int)r >= src_ptr[n]) return;  // rows outside every segment
    const int i = segment_of(src_ptr, n, (int)r);
    if (!s.b[i]) return;
    const size_t out = (size_t)s.plan->base + s.a[i] + ((int)r - src_ptr[i]);
    for (int u = u0; u < u0 + upt; ++u) dest[out * upr + u] = src[r * upr + u];
}

__global__ __launch_bounds__(kPlanBlock) void defrag_segments_plan_kernel(const int32_t* __restrict__ src_ptr,
                                                                          const uint8_t* __restrict__ copied, int n,
                                                                          int32_t* __restrict__ num_kept, Scratch s) {
    // a: where each kept segment starts after the compaction; b: the boundaries of the kept ones
    const int total = scan_all(n, s.a, [&](int i) { return copied[i] ? 0 : src_ptr[i + 1] - src_ptr[i]; });
    __syncthreads();
    int carry = 0;
    for (int i0 = 0; i0 < n; i0 += kPlanBlock) {
        const int i = i0 + (int)threadIdx.x;
        const int k = (i < n && !copied[i]) ? 1 : 0;
        int tot;
        const int rank = carry + block_scan(k, tot);
        carry += tot;
        if (k) s.b[rank] = s.a[i];
    }
    __syncthreads();
    for (int k = carry + (int)threadIdx.x; k <= n; k += kPlanBlock) s.b[k] = total;
    if (threadIdx.x == 0) {
        s.plan->count = carry;
        s.plan->total_kept = total;
        *num_kept = carry;
    }
}

template <class U>
__global__ __launch_bounds__(kBlock) void defrag_segments_scatter_kernel(const U* __restrict__ src,
                                                                         const int32_t* __restrict__ src_ptr,
                                                                         const uint8_t* __restrict__ copied, int n,
                                                                         int total_rows, int upr, int upt,
                                                                         Scratch s) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const int tpr = upr / upt;
    const size_t r = t / (size_t)tpr;
    if (r >= (size_t)total_rows) return;
    const int u0 = (int)(t - r * tpr) * upt;
    if ((int)r < src_ptr[0] || (int)r >= src_ptr[n]) return;  // rows outside every segment
    const int i = segment_of(src_ptr, n, (int)r);
    if (copied[i]) return;
    const size_t out = (size_t)s.a[i] + ((int)r - src_ptr[i]);
    for (int u = u0; u < u0 + upt; ++u) reinterpret_cast<U*>(s.temp)[out * upr + u] = src[r * upr + u];
}

template <class U>
__global__ __launch_bounds__(kBlock) void defrag_segments_back_kernel(U* __restrict__ src, int total_rows, int upr,
                                                                      Scratch s) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t r = t / (size_t)upr;
    if (r >= (size_t)total_rows) return;
    const int u = (int)(t - r * upr);
    U zero;
    __builtin_memset(&zero, 0, sizeof(U));
    src[r * upr + u] = (int)r < s.plan->total_kept ? reinterpret_cast<const U*>(s.temp)[r * upr + u] : zero;
}

__global__ __launch_bounds__(kBlock) void write_ptr_kernel(int32_t* __restrict__ ptr, int n, Scratch s) {
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k <= n) ptr[k] = s.b[k];
}

__global__ void empty_segments_kernel(int32_t* ptr, int32_t* num_kept) {
    ptr[0] = 0;
    *num_kept = 0;
}

// 16-, 4- or 1-byte units: the widest that divides the row and suits every pointer
int unit_bytes(size_t row_bytes, const void* p, const void* q, const void* r = nullptr) {
    auto ok = [&](size_t a) {
        auto al = [&](const void* x) { return x == nullptr || (reinterpret_cast<uintptr_t>(x) % a) == 0; };
        return row_bytes % a == 0 && al(p) && al(q) && al(r);
    };
    return ok(16) ? 16 : ok(4) ? 4 : 1;
}

inline unsigned blocks_for(size_t n) { return (unsigned)((n + kBlock - 1) / kBlock); }

#define NVAMD_UNIT_DISPATCH(UB, CALL)              \
    do {                                           \
        if ((UB) == 16) { using U = uint4; CALL; } \
        else if ((UB) == 4) { using U = uint32_t; CALL; } \
        else { using U = uint8_t; CALL; }          \
    } while (0)

constexpr size_t kMaxBytes = (size_t)1 << 38;  // keeps every grid below 2^31 workgroups

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_buffer_workspace_bytes(int64_t n_systems, int64_t data_bytes, size_t* bytes) {
    if (!bytes || n_systems < 0 || data_bytes < 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "buffer workspace: bad argument");
    *bytes = carve(nullptr, nullptr, (size_t)n_systems, (size_t)data_bytes);
    return NVAMD_OK;
}

static int32_t check_common(const char* what, int64_t n, int64_t row_bytes, void* workspace, size_t ws_bytes,
                            size_t data_bytes, Scratch* s) {
    if (n < 0 || n > INT32_MAX - 1 || row_bytes < 0 || row_bytes > INT32_MAX)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "%s: bad size", what);
    if (data_bytes > kMaxBytes) return fail(NVAMD_ERR_INVALID_ARGUMENT, "%s: more than 2^38 bytes", what);
    const size_t need = carve(nullptr, nullptr, (size_t)n, data_bytes);
    if (!workspace || ws_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "%s: workspace %zu < %zu bytes", what, ws_bytes, need);
    carve(s, static_cast<char*>(workspace), (size_t)n, data_bytes);
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_put_masked_per_system(const void* source, const uint8_t* source_mask, void* dest,
                                                 uint8_t* dest_mask, uint8_t* source_data_copied, int32_t num_src,
                                                 int32_t num_dest, int64_t row_bytes, void* workspace,
                                                 size_t workspace_bytes, void* stream) {
    Scratch s;
    if (row_bytes <= 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_masked_per_system: rows of zero bytes");
    int32_t rc = check_common("put_masked_per_system", num_src, row_bytes, workspace, workspace_bytes, 0, &s);
    if (rc != NVAMD_OK) return rc;
    if (num_dest < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_masked_per_system: negative num_dest");
    if ((size_t)num_src * (size_t)row_bytes > kMaxBytes)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_masked_per_system: more than 2^38 bytes");
    if (num_src == 0) return NVAMD_OK;
    if (!source_mask || !source_data_copied || (num_dest > 0 && !dest_mask) ||
        (row_bytes > 0 && (!source || (num_dest > 0 && !dest))))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_masked_per_system: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(put_rows_plan_kernel, dim3(1), dim3(kPlanBlock), 0, st, source_mask, num_src, dest_mask,
                       num_dest, s);
    const int ub = unit_bytes((size_t)row_bytes, source, dest);
    const int upr = (int)(row_bytes / ub);
    const size_t units = (size_t)num_src * upr;
    NVAMD_UNIT_DISPATCH(ub, hipLaunchKernelGGL((put_rows_copy_kernel<U>), dim3(blocks_for(units)), dim3(kBlock), 0, st,
                                               static_cast<const U*>(source), source_mask, static_cast<U*>(dest),
                                               dest_mask, source_data_copied, num_src, upr, s));
    NVAMD_LAUNCH_CHECK("put_masked_per_system launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_put_fit_mask_per_system(const uint8_t* source_mask, const uint8_t* dest_mask,
                                                   uint8_t* fit_mask, int32_t num_src, int32_t num_dest,
                                                   void* workspace, size_t workspace_bytes, void* stream) {
    Scratch s;
    int32_t rc = check_common("put_fit_mask_per_system", num_src, 0, workspace, workspace_bytes, 0, &s);
    if (rc != NVAMD_OK) return rc;
    if (num_dest < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_fit_mask_per_system: negative num_dest");
    if (num_src == 0) return NVAMD_OK;
    if (!source_mask || !fit_mask || (num_dest > 0 && !dest_mask))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_fit_mask_per_system: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(put_rows_plan_kernel, dim3(1), dim3(kPlanBlock), 0, st, source_mask, num_src, dest_mask,
                       num_dest, s);
    hipLaunchKernelGGL(fit_rows_kernel, dim3(blocks_for(num_src)), dim3(kBlock), 0, st, source_mask, fit_mask, num_src,
                       s);
    NVAMD_LAUNCH_CHECK("put_fit_mask_per_system launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_defrag_per_system(void* source, uint8_t* source_data_copied, int32_t num_src,
                                             int64_t row_bytes, void* workspace, size_t workspace_bytes,
                                             void* stream) {
    Scratch s;
    if (row_bytes <= 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "defrag_per_system: rows of zero bytes");
    int32_t rc = check_common("defrag_per_system", num_src, row_bytes, workspace, workspace_bytes,
                              (size_t)(num_src > 0 ? num_src : 0) * (size_t)row_bytes, &s);
    if (rc != NVAMD_OK) return rc;
    if (num_src == 0) return NVAMD_OK;
    if (!source || !source_data_copied) return fail(NVAMD_ERR_INVALID_ARGUMENT, "defrag_per_system: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(defrag_rows_plan_kernel, dim3(1), dim3(kPlanBlock), 0, st, source_data_copied, num_src, s);
    const int ub = unit_bytes((size_t)row_bytes, source, s.temp);
    const int upr = (int)(row_bytes / ub);
    const size_t units = (size_t)num_src * upr;
    NVAMD_UNIT_DISPATCH(ub, {
        hipLaunchKernelGGL((defrag_rows_scatter_kernel<U>), dim3(blocks_for(units)), dim3(kBlock), 0, st,
                           static_cast<const U*>(source), source_data_copied, num_src, upr, s);
        hipLaunchKernelGGL((defrag_rows_back_kernel<U>), dim3(blocks_for(units)), dim3(kBlock), 0, st,
                           static_cast<U*>(source), source_data_copied, num_src, upr, s);
    });
    NVAMD_LAUNCH_CHECK("defrag_per_system launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_put_masked_segmented(const void* source, const int32_t* source_batch_ptr,
                                                const uint8_t* source_mask, void* dest, int32_t* dest_batch_ptr,
                                                int32_t num_dest_segments, int32_t dest_capacity,
                                                uint8_t* source_data_copied, int32_t* new_num_dest,
                                                int32_t num_systems, int32_t total_rows, int64_t row_bytes,
                                                void* workspace, size_t workspace_bytes, void* stream) {
    Scratch s;
    int32_t rc = check_common("put_masked_segmented", num_systems, row_bytes, workspace, workspace_bytes, 0, &s);
    if (rc != NVAMD_OK) return rc;
    if (num_dest_segments < 0 || dest_capacity < 0 || total_rows < 0 || row_bytes <= 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_masked_segmented: bad size");
    if ((size_t)total_rows * (size_t)row_bytes > kMaxBytes)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_masked_segmented: more than 2^38 bytes");
    if (num_systems == 0) return NVAMD_OK;
    if (!source_batch_ptr || !source_mask || !dest_batch_ptr || !source_data_copied || !new_num_dest ||
        (total_rows > 0 && !source) || (dest_capacity > 0 && !dest))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_masked_segmented: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(put_segments_plan_kernel, dim3(1), dim3(kPlanBlock), 0, st, source_batch_ptr, source_mask,
                       num_systems, dest_batch_ptr, num_dest_segments, dest_capacity, source_data_copied,
                       (uint8_t*)nullptr, new_num_dest, 1, s);
    if (total_rows > 0) {
        const int ub = unit_bytes((size_t)row_bytes, source, dest);
        const int upr = (int)(row_bytes / ub);
        const int upt = upr <= 4 ? upr : 1;
        const size_t threads = (size_t)total_rows * (upr / upt);
        NVAMD_UNIT_DISPATCH(ub, hipLaunchKernelGGL((put_segments_copy_kernel<U>), dim3(blocks_for(threads)),
                                                   dim3(kBlock), 0, st, static_cast<const U*>(source), source_batch_ptr,
                                                   num_systems, total_rows, static_cast<U*>(dest), upr, upt, s));
    }
    NVAMD_LAUNCH_CHECK("put_masked_segmented launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_put_fit_mask_segmented(const int32_t* source_batch_ptr, const uint8_t* source_mask,
                                                  const int32_t* dest_batch_ptr, int32_t num_dest_segments,
                                                  int32_t dest_capacity, uint8_t* fit_mask, int32_t num_systems,
                                                  void* workspace, size_t workspace_bytes, void* stream) {
    Scratch s;
    int32_t rc = check_common("put_fit_mask_segmented", num_systems, 0, workspace, workspace_bytes, 0, &s);
    if (rc != NVAMD_OK) return rc;
    if (num_dest_segments < 0 || dest_capacity < 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_fit_mask_segmented: bad size");
    if (num_systems == 0) return NVAMD_OK;
    if (!source_batch_ptr || !source_mask || !dest_batch_ptr || !fit_mask)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "put_fit_mask_segmented: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(put_segments_plan_kernel, dim3(1), dim3(kPlanBlock), 0, st, source_batch_ptr, source_mask,
                       num_systems, const_cast<int32_t*>(dest_batch_ptr), num_dest_segments, dest_capacity,
                       (uint8_t*)nullptr, fit_mask, (int32_t*)nullptr, 0, s);
    NVAMD_LAUNCH_CHECK("put_fit_mask_segmented launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_defrag_segmented(void* source, int32_t* source_batch_ptr,
                                            const uint8_t* source_data_copied, int32_t* num_kept,
                                            int32_t num_systems, int32_t total_rows, int64_t row_bytes,
                                            void* workspace, size_t workspace_bytes, void* stream) {
    Scratch s;
    if (row_bytes <= 0 || total_rows < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "defrag_segmented: bad size");
    int32_t rc = check_common("defrag_segmented", num_systems, row_bytes, workspace, workspace_bytes,
                              (size_t)total_rows * (size_t)row_bytes, &s);
    if (rc != NVAMD_OK) return rc;
    if (!source_batch_ptr || !num_kept) return fail(NVAMD_ERR_INVALID_ARGUMENT, "defrag_segmented: null buffer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (num_systems == 0) {
        hipLaunchKernelGGL(empty_segments_kernel, dim3(1), dim3(1), 0, st, source_batch_ptr, num_kept);
        NVAMD_LAUNCH_CHECK("defrag_segmented launch");
        return NVAMD_OK;
    }
    if (!source_data_copied || (total_rows > 0 && !source))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "defrag_segmented: null buffer");
    hipLaunchKernelGGL(defrag_segments_plan_kernel, dim3(1), dim3(kPlanBlock), 0, st, source_batch_ptr,
                       source_data_copied, num_systems, num_kept, s);
    if (total_rows > 0) {
        const int ub = unit_bytes((size_t)row_bytes, source, s.temp);
        const int upr = (int)(row_bytes / ub);
        const int upt = upr <= 4 ? upr : 1;
        const size_t units = (size_t)total_rows * upr;
        NVAMD_UNIT_DISPATCH(ub, {
            hipLaunchKernelGGL((defrag_segments_scatter_kernel<U>), dim3(blocks_for(units / upt)), dim3(kBlock), 0, st,
                               static_cast<const U*>(source), source_batch_ptr, source_data_copied, num_systems,
                               total_rows, upr, upt, s);
            hipLaunchKernelGGL((defrag_segments_back_kernel<U>), dim3(blocks_for(units)), dim3(kBlock), 0, st,
                               static_cast<U*>(source), total_rows, upr, s);
        });
    }
    hipLaunchKernelGGL(write_ptr_kernel, dim3(blocks_for((size_t)num_systems + 1)), dim3(kBlock), 0, st,
                       source_batch_ptr, num_systems, s);
    NVAMD_LAUNCH_CHECK("defrag_segmented launch");
    return NVAMD_OK;
}
