// Device-wide exclusive scan of int32 in three small kernels (tile sums, scan of the tile
// sums by one workgroup, tile-local scan plus offset).  The element count may live on the
// device (n_dev != nullptr), so callers need no host synchronisation to size the scan.
#pragma once

#include "common.h"

namespace nvamd {
namespace scan {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;
constexpr int kItems = 8;
constexpr int kTile = kBlock * kItems;

inline int tiles_for(size_t n) { return (int)((n + kTile - 1) / kTile); }

// exclusive scan of one value per thread across the workgroup; `total` = workgroup sum
__device__ __forceinline__ int block_exclusive(int v, int* s_wave, int& total) {
    int lane = lane_id(), wave = (int)threadIdx.x / kWave;
    int incl = v;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        int up = __shfl_up(incl, o, kWave);
        if (lane >= o) incl += up;
    }
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    int before = 0;
    total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        int sw = s_wave[w];
        if (w < wave) before += sw;
        total += sw;
    }
    __syncthreads();
    return before + incl - v;
}

// Load: int operator()(int index) const
template <class Load>
__global__ __launch_bounds__(kBlock) void partial_kernel(Load load, const int* n_dev, int n_host,
                                                         int* __restrict__ tile_sums) {
    __shared__ int s_wave[kWaves];
    const int n = n_dev ? *n_dev : n_host;
    const int tile0 = (int)blockIdx.x * kTile;
    int sum = 0;
    if (tile0 < n) {
        int base = tile0 + (int)threadIdx.x * kItems;
#pragma unroll
        for (int k = 0; k < kItems; ++k)
            if (base + k < n) sum += load(base + k);
    }
    int tot;
    block_exclusive(sum, s_wave, tot);
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = tot;
}

template <int kUnused = 0>
__global__ __launch_bounds__(kBlock) void top_kernel(const int* n_dev, int n_host,
                                                     int* __restrict__ tile_sums) {
    __shared__ int s_wave[kWaves];
    __shared__ int s_carry;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    const int n = n_dev ? *n_dev : n_host;
    const int nb = (n + kTile - 1) / kTile;
    for (int base = 0; base < nb; base += kBlock) {
        int t = base + (int)threadIdx.x;
        int v = t < nb ? tile_sums[t] : 0;
        int tot;
        int ex = block_exclusive(v, s_wave, tot);
        int carry = s_carry;
        if (t < nb) tile_sums[t] = carry + ex;
        __syncthreads();
        if (threadIdx.x == 0) s_carry = carry + tot;
        __syncthreads();
    }
}

// writes out[0..n] (n+1 entries: the last one is the grand total)
template <class Load>
__global__ __launch_bounds__(kBlock) void final_kernel(Load load, const int* n_dev, int n_host,
                                                       const int* __restrict__ tile_sums,
                                                       int* __restrict__ out) {
    __shared__ int s_wave[kWaves];
    const int n = n_dev ? *n_dev : n_host;
    const int tile0 = (int)blockIdx.x * kTile;
    if (tile0 >= n) {
        if (n == 0 && blockIdx.x == 0 && threadIdx.x == 0) out[0] = 0;
        return;
    }
    int base = tile0 + (int)threadIdx.x * kItems;
    int v[kItems];
    int sum = 0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        v[k] = (base + k < n) ? load(base + k) : 0;
        sum += v[k];
    }
    int tot;
    int ex = block_exclusive(sum, s_wave, tot) + tile_sums[blockIdx.x];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (base + k < n) out[base + k] = ex;
        ex += v[k];
    }
    if (base <= n - 1 && n - 1 < base + kItems) out[n] = ex;
}

// n_tiles must cover the largest n the device value can take
template <class Load>
inline void exclusive(Load load, const int* n_dev, int n_host, int n_tiles, int* tile_sums, int* out,
                      hipStream_t st) {
    if (n_tiles < 1) n_tiles = 1;
    hipLaunchKernelGGL((partial_kernel<Load>), dim3(n_tiles), dim3(kBlock), 0, st, load, n_dev, n_host,
                       tile_sums);
    hipLaunchKernelGGL((top_kernel<0>), dim3(1), dim3(kBlock), 0, st, n_dev, n_host, tile_sums);
    hipLaunchKernelGGL((final_kernel<Load>), dim3(n_tiles), dim3(kBlock), 0, st, load, n_dev, n_host,
                       tile_sums, out);
}

struct LoadArray {
    const int* p;
    __device__ __forceinline__ int operator()(int i) const { return p[i]; }
};

struct LoadClamped {
    const int* p;
    int cap;
    __device__ __forceinline__ int operator()(int i) const {
        int v = p[i];
        return v < cap ? v : cap;
    }
};

}  // namespace scan
}  // namespace nvamd
