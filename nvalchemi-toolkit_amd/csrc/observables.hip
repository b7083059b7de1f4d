// Per-system reductions of per-atom quantities for gfx950: sum, max, min, mean of a float32 vector
// over the segments given by a sorted batch index, and the kinetic energy per system.
//
// Reference interfaces: the custom ops nvalchemi_hooks::segmented_sum / _max / _min / _mean and
// nvalchemi_hooks::compute_kinetic_energy (nvalchemi/dynamics/hooks/_utils.py:58-170), behind
// scatter_reduce_per_graph, kinetic_energy_per_graph and temperature_per_graph (:172-290).
// One streaming pass (8 B/atom; 20 B/atom for the kinetic energy): a segmented reduction inside
// each wavefront (the batch index is sorted, so a system is one run of lanes), then one atomic
// per wavefront and system -- sums in float64, extrema on order-preserving integer keys -- and a
// pass over the systems that writes the float32 results.
#include "common.h"

namespace nvamd {
namespace {

constexpr int kBlock = 256;
enum { kOpSum = 0, kOpMax = 1, kOpMin = 2, kOpMean = 3, kOpKinetic = 4 };

struct SegScratch {
    double* sum;     // (M)
    uint32_t* key;   // (M) extremum as an order key, or the element count for the mean
};

size_t seg_carve(SegScratch* s, char* base, int m) {
    size_t M = (size_t)(m > 0 ? m : 1);
    size_t off = 0;
    if (s) s->sum = reinterpret_cast<double*>(base + off);
    off += align_up(M * sizeof(double));
    if (s) s->key = reinterpret_cast<uint32_t*>(base + off);
    off += align_up(M * sizeof(uint32_t));
    return off;
}

__global__ __launch_bounds__(kBlock) void seg_init_kernel(SegScratch sc, int m, int op) {
    int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    sc.sum[s] = 0.0;
    sc.key[s] = (op == kOpMax) ? float_order_key(-INFINITY) : (op == kOpMin) ? float_order_key(INFINITY) : 0u;
}

template <int OP>
__global__ __launch_bounds__(kBlock) void seg_reduce_kernel(const float* __restrict__ values,
                                                            const float* __restrict__ masses,
                                                            const int32_t* __restrict__ bidx, int n,
                                                            SegScratch sc) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    const int lane = lane_id();
    int seg = -1 - (i - n);  // lanes past the end: each its own (negative) segment
    double v = 0.0;
    float x = 0.f;
    int cnt = 0;
    if (i < n) {
        seg = bidx[i];
        cnt = 1;
        if (OP == kOpKinetic) {
            const size_t b = 3 * (size_t)i;
            const double vx = values[b], vy = values[b + 1], vz = values[b + 2];
            v = 0.5 * (double)masses[i] * ((vx * vx + vy * vy) + vz * vz);
        } else {
            x = values[i];
            v = (double)x;
        }
    }
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const int seg_up = __shfl_down(seg, o, kWave);
        const bool take = (lane + o < kWave) && (seg_up == seg);
        if (OP == kOpMax || OP == kOpMin) {
            const float up = __shfl_down(x, o, kWave);
            if (take) x = (OP == kOpMax) ? fmaxf(x, up) : fminf(x, up);
        } else {
            const double up = __shfl_down(v, o, kWave);
            if (take) v += up;
            if (OP == kOpMean) {
                const int cu = __shfl_down(cnt, o, kWave);
                if (take) cnt += cu;
            }
        }
    }
    const int seg_prev = __shfl_up(seg, 1, kWave);
    const bool head = (lane == 0 || seg_prev != seg) && i < n;
    if (!head) return;
    if (OP == kOpMax) atomicMax(sc.key + seg, float_order_key(x));
    else if (OP == kOpMin) atomicMin(sc.key + seg, float_order_key(x));
    else {
        atomic_add_f64(sc.sum + seg, v);
        if (OP == kOpMean) atomicAdd(sc.key + seg, (uint32_t)cnt);
    }
}

__global__ __launch_bounds__(kBlock) void seg_finish_kernel(SegScratch sc, int m, int op, float* __restrict__ out) {
    int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= m) return;
    float r;
    if (op == kOpMax || op == kOpMin) r = float_from_order_key(sc.key[s]);
    else if (op == kOpMean) r = sc.key[s] ? (float)(sc.sum[s] / (double)sc.key[s]) : 0.0f;
    else r = (float)sc.sum[s];
    out[s] = r;
}

int32_t run(const float* values, const float* masses, const int32_t* bidx, int32_t n, int32_t m, int op,
            float* out, void* workspace, size_t workspace_bytes, void* stream, const char* what) {
    if (n < 0 || m < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "%s: negative size", what);
    if (m == 0) return NVAMD_OK;
    if (!out || (n > 0 && (!values || !bidx))) return fail(NVAMD_ERR_INVALID_ARGUMENT, "%s: null buffer", what);
    const size_t need = seg_carve(nullptr, nullptr, m);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "%s: workspace %zu < %zu bytes", what, workspace_bytes, need);
    SegScratch sc;
    seg_carve(&sc, static_cast<char*>(workspace), m);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 gm((m + kBlock - 1) / kBlock), gn((n + kBlock - 1) / kBlock), blk(kBlock);
    hipLaunchKernelGGL(seg_init_kernel, gm, blk, 0, st, sc, m, op);
    if (n > 0) {
        switch (op) {
            case kOpSum: hipLaunchKernelGGL(seg_reduce_kernel<kOpSum>, gn, blk, 0, st, values, masses, bidx, n, sc); break;
            case kOpMax: hipLaunchKernelGGL(seg_reduce_kernel<kOpMax>, gn, blk, 0, st, values, masses, bidx, n, sc); break;
            case kOpMin: hipLaunchKernelGGL(seg_reduce_kernel<kOpMin>, gn, blk, 0, st, values, masses, bidx, n, sc); break;
            case kOpMean: hipLaunchKernelGGL(seg_reduce_kernel<kOpMean>, gn, blk, 0, st, values, masses, bidx, n, sc); break;
            default: hipLaunchKernelGGL(seg_reduce_kernel<kOpKinetic>, gn, blk, 0, st, values, masses, bidx, n, sc); break;
        }
    }
    hipLaunchKernelGGL(seg_finish_kernel, gm, blk, 0, st, sc, m, op, out);
    NVAMD_LAUNCH_CHECK(what);
    return NVAMD_OK;
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_segment_workspace_bytes(int32_t n_segments, size_t* bytes) {
    if (!bytes || n_segments < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "segment workspace: bad argument");
    *bytes = seg_carve(nullptr, nullptr, n_segments);
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_segment_reduce(const float* values, const int32_t* batch_idx, int32_t n_values,
                                          int32_t n_segments, int32_t op, float* out, void* workspace,
                                          size_t workspace_bytes, void* stream) {
    if (op < kOpSum || op > kOpMean) return fail(NVAMD_ERR_INVALID_ARGUMENT, "segment reduce: unknown operation %d", op);
    return run(values, nullptr, batch_idx, n_values, n_segments, op, out, workspace, workspace_bytes, stream,
               "segment reduce");
}

NVAMD_EXPORT int32_t nvamd_kinetic_energy(const float* velocities, const float* masses, const int32_t* batch_idx,
                                          int32_t n_atoms, int32_t n_systems, float* kinetic_energy,
                                          void* workspace, size_t workspace_bytes, void* stream) {
    if (n_atoms > 0 && !masses) return fail(NVAMD_ERR_INVALID_ARGUMENT, "kinetic energy: null masses");
    return run(velocities, masses, batch_idx, n_atoms, n_systems, kOpKinetic, kinetic_energy, workspace,
               workspace_bytes, stream, "kinetic energy");
}
