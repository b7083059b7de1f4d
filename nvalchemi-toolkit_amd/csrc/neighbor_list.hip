// Batched periodic cell-list neighbor build for gfx950.
//
// Reference interface: nvalchemiops.torch.neighbors.neighbor_list as called at
// nvalchemi/neighbors.py:253-266 and nvalchemi/hooks/neighbor_list.py:328-343 (dense
// (N,K) matrix + counts + (N,K,3) integer shifts written in place, counting past K as the
// overflow signal), including the stale-slot masking the hook performs afterwards
// (nvalchemi/hooks/neighbor_list.py:377-380).
//
// Pipeline (all on the caller's stream, no host synchronisation, no allocation):
//   1 prepare   per system: cell, inverse, periodic flags; clear histogram and bounds
//   2 bounds    fractional bounding box on non-periodic axes (skipped work for periodic ones)
//   3 grid      per system: cells per axis (width >= cutoff), stencil radius, cell offsets
//   4 bin       per atom: wrapped fractional coordinate -> cell, rank inside the cell
//   5 scan      exclusive scan of the histogram (three small kernels)
//   6 scatter   counting-sort the atoms into cell order: cell-local coordinates + wrap
//   7 search    one workgroup per run of cells along z: stage the stencil's atoms in LDS, one
//               wavefront per centre atom, 64 candidates per step, ballot + prefix-popcount
//               compaction into a hit list, the list written out into the atom's row
// (batches of many small systems take 1-6 in one workgroup per system: nl_system_sort_kernel).
// What the search writes (rows, shifts) goes out with non-temporal stores.  For batches of large systems it can
// also leave a description of its tiles for the pair kernel and skip the stores of zero shifts over zeros
// (nvamd_nl_build_extras).  The unit counter and the status bits live in the workspace's header, in two slots taken
// in turn, so that a build needs no launch to reset them.
//
// Which pairs are neighbors is decided in double on the original positions (geom.h).  The search
// classifies candidates with float32 distances on cell-local coordinates whose rounding error is
// bounded by per-system tolerances (a wider one for the three-instruction form of the scan, the
// usual one for the direct form of the write-out); only candidates inside the band around the
// cutoff are re-evaluated exactly, so the list is independent of the order of float32
// operations in the fast path.
#include "common.h"
#include "geom.h"
#include "scan.h"

namespace nvamd {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
#ifndef NVAMD_NL_TILE
#define NVAMD_NL_TILE 1088
#endif
constexpr int kTile = NVAMD_NL_TILE;  // candidates staged in LDS at a time
constexpr int kStencilBatch = 64; // stencil cells enumerated at a time (one per lane of a wave)
#ifndef NVAMD_NL_MAXCHUNK
#define NVAMD_NL_MAXCHUNK 72
#endif
constexpr int kCenterChunk = NVAMD_NL_MAXCHUNK;  // centre atoms of a run of cells handled per pass
#ifndef NVAMD_NL_CHUNK
#define NVAMD_NL_CHUNK(n) center_chunk_for(n)
#endif
// Centre atoms per unit of work for a batch of n_atoms: kCenterChunk from 58 000 atoms on, 16 below 19 000 (measured
// on batches of 500-atom FCC boxes and of 3900-atom liquid boxes of 4 000 to 250 000 atoms: smaller units fill the
// chip sooner, larger ones stage their tile for more centre atoms; 40, whole cells of the FCC boxes, is the best
// at 32 000 atoms for both)
inline int center_chunk_for(int n_atoms) {
    int c = n_atoms / 800 / 8 * 8;
    return c < 16 ? 16 : (c > kCenterChunk ? kCenterChunk : c);
}
constexpr int kMaxRun = 4;        // a workgroup's unit of work: up to this many cells in a row along z
#ifndef NVAMD_NL_HITCAP
#define NVAMD_NL_HITCAP 256
#endif
constexpr int kHitCap = NVAMD_NL_HITCAP;      // per-wave list of accepted candidates before it is written out
constexpr int kPackOverflow = 1 << 15;
static_assert(kMaxRun <= 4, "a centre atom's place in its run is kept in two bits");
constexpr int kMaxCellsPerAxis = 1024;
static_assert(kMaxCellsPerAxis <= 1024, "a search unit's cell coordinates are packed 10 bits each");
constexpr int kMinCellCap = 8;    // a system may use at least this many cells
constexpr int kMaxStencilRadius = 32;  // cells searched per axis and direction, at most
constexpr int kTileRecord = NVAMD_NL_TILE_RECORD_INTS / 2;  // 8-byte words of a unit's record for the pair kernel
static_assert(kTileRecord == 2 + kStencilBatch, "two words of header, then one word per stencil cell");
static_assert(kTile <= NVAMD_NL_TILE_ATOMS, "a tile index must stay below what the header promises");

struct NlSys {
    double h[9];       // rows = lattice vectors (identity without a cell)
    double hinv[9];    // frac = r . hinv
    double width[3];   // perpendicular width of the cell along each lattice direction
    double lo[3];      // lower end of the binned fractional interval
    double ext[3];     // its length (1 on periodic axes)
    double step[9];    // row d = (ext[d]/nc[d]) * h[d,:] : one cell step along axis d
    float tol;         // relative half-width of the float32 uncertainty band on d^2
    float tol_scan;    // the same for the expanded form |q|^2 - 2 p.q + |p|^2 that the candidate scan evaluates
    int nc[3];
    int R[3];
    int per[3];
    int cell_offset;
    int n_cells;
    int zr;            // cells per run along axis 2 (the search's unit of work)
    int n_units;       // runs in this system
    int error;         // bit 0: cell degenerate or narrower than cutoff/kMaxStencilRadius
    int atom_begin, atom_end;
};

// What the search kernel needs per system, in 32-bit words (read through scalar loads).
struct NlSearchSys {
    float step[9];  // cell step vectors, row d = one cell along axis d
    float tol;      // relative half-width of the float32 uncertainty band on d^2
    float tol_scan; // the same for the expanded form of the candidate scan (wider: its terms are as large as reach^2)
    int nc[3];
    int R[3];
    int per[3];
    int cell_offset;
    int zr;
    float half_diag;  // half of the longest body diagonal of one cell
    float cull_far;   // distance of the farthest stencil cell centre from its run's nearest cell centre
};

// One unit of search work: a run of cells along axis 2, with what the enumeration of its
// stencil needs from its system, so that the search kernel reaches the cell table with one
// round trip to memory less.
struct __attribute__((aligned(32))) NlUnit {
    int c0;           // first cell of the run (global id)
    int sidx;         // system
    int cxyz;         // that cell's coordinates, 10 bits each: cx << 20 | cy << 10 | cz
    int run_len;      // cells in the run
    int nc_pack;      // cells per axis minus one, 10 bits each: (nc0-1) | (nc1-1) << 10 | (nc2-1) << 20
    int rper_pack;    // stencil radii, 6 bits each, then the periodic flags: R0 | R1 << 6 | R2 << 12 | per << 18
    int cell_offset;  // first cell of the system
    int first_centre; // -1: the unit covers all centre atoms of the run; else count << 24 | first: `count` of them from `first`
};
static_assert(sizeof(NlUnit) == 32, "read as two 16-byte words");
static_assert(kMaxStencilRadius < 64, "stencil radii are packed 6 bits each");

struct NlHeader {
    // The unit counter and the flags of a build live in one of two slots, taken in turn (flip), so that no build
    // needs a launch that resets them: the kernels that sort (which run before any other kernel of a build reads
    // the slot in hand) clear the other slot, the one of the build before, after moving its flags to `sticky`; the
    // search kernel reads the sum of both counters (the other one is zero by then) and its first workgroup turns
    // flip over for the next build (nobody else reads flip while the search runs).  A new workspace starts with a
    // zeroed header.
    int total_cells;
    int flip;       // the slot of the next build (of the build in hand, until its search kernel runs)
    int units[2];   // search units of the build that used the slot
    int error[2];   // its NVAMD_NL_STATUS_* bits
    int sticky;     // the bits of all builds before the last one since they were last cleared
    int pad[9];
};
static_assert(sizeof(NlHeader) == 64, "inside the 256 bytes that a new workspace starts with as zeros");

// First thing in a build, by one thread of a kernel that runs before the build's counters are read by anyone else:
// the slot of the build before is folded away and cleared.
__device__ __forceinline__ void retire_other_slot(NlHeader* hdr) {
    const int other = hdr->flip ^ 1;
    hdr->sticky |= hdr->error[other];
    hdr->error[other] = 0;
    hdr->units[other] = 0;
}

struct NlWorkspace {
    NlHeader* hdr;
    NlSys* sys;
    uint32_t* bounds;    // (B,6) order keys: min x,y,z then max x,y,z
    NlSearchSys* ssys;   // (B)
    int* cell_offset;    // (B+1)
    int* unit_offset;    // (B+1) first unit of each system
    NlUnit* units;       // (C) the search's units of work
    int* atom_rank;      // (N)
    int* cell_count;     // (C)
    int* cell_start;     // (C+1)
    int* block_sums;     // scan partials
    float4* sorted_pos;  // (N) cell-local xyz + original index bits
    int4* sorted_aux;    // (N) wrap integers
    int max_cells;
    int n_scan_blocks;
};

size_t max_cells_for(int n_atoms, int n_systems) {
    // (one more per system: the per-system path gives every system its own end-of-cells entry)
    return (size_t)n_atoms + (size_t)(kMinCellCap + 1) * (size_t)n_systems + 1;
}

size_t carve(NlWorkspace* ws, char* base, int n_atoms, int n_systems) {
    size_t N = (size_t)(n_atoms > 0 ? n_atoms : 1), B = (size_t)(n_systems > 0 ? n_systems : 1);
    size_t C = max_cells_for(n_atoms, n_systems);
    size_t nsb = (size_t)scan::tiles_for(C);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        size_t o = off;
        off += align_up(bytes);
        return base ? base + o : nullptr;
    };
    char* p;
    p = take(sizeof(NlHeader)); if (ws) ws->hdr = reinterpret_cast<NlHeader*>(p);
    p = take(B * sizeof(NlSys)); if (ws) ws->sys = reinterpret_cast<NlSys*>(p);
    p = take(B * 6 * sizeof(uint32_t)); if (ws) ws->bounds = reinterpret_cast<uint32_t*>(p);
    p = take(B * sizeof(NlSearchSys)); if (ws) ws->ssys = reinterpret_cast<NlSearchSys*>(p);
    p = take((B + 1) * sizeof(int)); if (ws) ws->cell_offset = reinterpret_cast<int*>(p);
    p = take((B + 1) * sizeof(int)); if (ws) ws->unit_offset = reinterpret_cast<int*>(p);
    p = take(C * sizeof(NlUnit)); if (ws) ws->units = reinterpret_cast<NlUnit*>(p);
    p = take(N * sizeof(int)); if (ws) ws->atom_rank = reinterpret_cast<int*>(p);
    p = take(C * sizeof(int)); if (ws) ws->cell_count = reinterpret_cast<int*>(p);
    p = take((C + 1) * sizeof(int)); if (ws) ws->cell_start = reinterpret_cast<int*>(p);
    p = take((nsb + 1) * sizeof(int)); if (ws) ws->block_sums = reinterpret_cast<int*>(p);
    p = take(N * sizeof(float4)); if (ws) ws->sorted_pos = reinterpret_cast<float4*>(p);
    p = take(N * sizeof(int4)); if (ws) ws->sorted_aux = reinterpret_cast<int4*>(p);
    if (ws) {
        ws->max_cells = (int)C;
        ws->n_scan_blocks = (int)nsb;
    }
    return off;
}

struct NlArgs {
    const float* pos;      // float32 positions and cells ...
    const float* cell;
    const double* pos64;   // ... or float64 ones (then pos and cell are null)
    const double* cell64;
    const uint8_t* pbc;
    const int32_t* ptr;
    const int32_t* bidx;
    const uint8_t* rebuild;
    int n_atoms, n_systems, K, half, tail_mode;
    int unit_group;  // units are dealt to the XCDs in groups of this many (a power of two)
    int center_chunk;  // centre atoms per unit of work at most (<= kCenterChunk; smaller for small batches: more units)
    // What a pair kernel needs to walk the search's own tiles again (all null unless asked for):
    uint16_t* tile_index;  // (N, K) per listed pair: where the neighbor stood in the tile of the centre atom's unit
    float4* tile_xyz;      // (N) the atoms' own float32 coordinates + original index bits, in cell order
    int2* tile_records;    // (max cells, kTileRecord) per unit: (first row, rows), (system, atoms in the tile or -1),
                           // then per stencil cell (first slot of the cell order, offset in the tile)
    int32_t* tile_count;   // (1) units of this build
    // Shifts written only where they have to be (null: every listed pair's shift is written).  Bit g of a row's
    // word says that slots [g << group_shift, (g + 1) << group_shift) of the row may hold a shift that is not zero;
    // everywhere else the shifts in memory are zero and a zero shift need not be written again.
    uint32_t* shift_groups;  // (N)
    int group_shift;
    double rc, rc2, rcb;
    int32_t* nm;
    int32_t* nn;
    int32_t* shifts;
};

// position of atom i in double, whichever type it is stored in
struct Pos3 {
    double x, y, z;
};
__device__ __forceinline__ Pos3 load_pos(const NlArgs& a, size_t i) {
    Pos3 p;
    if (a.pos64) {
        p.x = a.pos64[3 * i + 0];
        p.y = a.pos64[3 * i + 1];
        p.z = a.pos64[3 * i + 2];
    } else {
        p.x = (double)a.pos[3 * i + 0];
        p.y = (double)a.pos[3 * i + 1];
        p.z = (double)a.pos[3 * i + 2];
    }
    return p;
}

__device__ __forceinline__ void frac_of(const NlSys& s, const Pos3& r, double* f) {
    double x = r.x, y = r.y, z = r.z;
    f[0] = x * s.hinv[0] + y * s.hinv[3] + z * s.hinv[6];
    f[1] = x * s.hinv[1] + y * s.hinv[4] + z * s.hinv[7];
    f[2] = x * s.hinv[2] + y * s.hinv[5] + z * s.hinv[8];
}

// ---- 1 prepare ------------------------------------------------------------------------------
// Per-system constants that do not depend on the atoms: cell, inverse, widths, periodic flags.
__device__ __forceinline__ void system_setup(NlSys& s, const NlArgs& a, int t) {
    const bool has_cell = a.cell != nullptr || a.cell64 != nullptr;
#pragma unroll
    for (int k = 0; k < 9; ++k)
        s.h[k] = a.cell64 ? a.cell64[9 * (size_t)t + k]
                          : (a.cell ? (double)a.cell[9 * (size_t)t + k] : ((k % 4 == 0) ? 1.0 : 0.0));
    inv3(s.h, s.hinv);
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        double nx = s.hinv[d], ny = s.hinv[3 + d], nz = s.hinv[6 + d];
        s.width[d] = 1.0 / sqrt(nx * nx + ny * ny + nz * nz);
        s.per[d] = (has_cell && a.pbc) ? (a.pbc[3 * (size_t)t + d] != 0) : 0;
        s.lo[d] = 0.0;
        s.ext[d] = 1.0;
        s.nc[d] = 1;
        s.R[d] = 0;
    }
#pragma unroll
    for (int k = 0; k < 9; ++k) s.step[k] = s.h[k];
    s.tol = 0.f;
    s.cell_offset = 0;
    s.n_cells = 1;
    s.zr = 1;
    s.n_units = 0;
    s.error = 0;
    s.atom_begin = a.ptr[t];
    s.atom_end = a.ptr[t + 1];
}

__global__ __launch_bounds__(kBlock) void nl_prepare_kernel(NlArgs a, NlWorkspace ws) {
    int t = blockIdx.x * kBlock + threadIdx.x;
    if (t < ws.max_cells) ws.cell_count[t] = 0;
    if (t == 0) retire_other_slot(ws.hdr);
    if (t >= a.n_systems) return;
    NlSys s;
    system_setup(s, a, t);
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        ws.bounds[6 * (size_t)t + d] = 0xffffffffu;      // min key
        ws.bounds[6 * (size_t)t + 3 + d] = 0u;           // max key
    }
    ws.sys[t] = s;
}

// ---- 2 bounds -------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void nl_bounds_kernel(NlArgs a, NlWorkspace ws) {
    int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.n_atoms) return;
    int sidx = a.bidx[i];
    const NlSys& s = ws.sys[sidx];
    if (s.per[0] && s.per[1] && s.per[2]) return;
    double f[3];
    frac_of(s, load_pos(a, (size_t)i), f);
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        if (s.per[d]) continue;
        float lo = __double2float_rd(f[d]), hi = __double2float_ru(f[d]);
        atomicMin(ws.bounds + 6 * (size_t)sidx + d, float_order_key(lo));
        atomicMax(ws.bounds + 6 * (size_t)sidx + 3 + d, float_order_key(hi));
    }
}

// Cells per axis (width >= cutoff), stencil radius, run length, cell steps and the float32
// tolerance of one system; bounds6 holds the order keys of the fractional bounding box
// (min x,y,z then max x,y,z), read on non-periodic axes only.
__device__ __forceinline__ void choose_grid(NlSys& s, const NlArgs& a, const uint32_t* bounds6, int* error_flag) {
    const int n_at = s.atom_end - s.atom_begin;
    for (int d = 0; d < 3; ++d) {
        if (!s.per[d]) {
            uint32_t kmin = bounds6[d], kmax = bounds6[3 + d];
            if (kmin <= kmax && n_at > 0) {
                double lo = (double)float_from_order_key(kmin), hi = (double)float_from_order_key(kmax);
                s.lo[d] = lo;
                s.ext[d] = hi - lo;
            }
            if (!(s.ext[d] > 1e-30)) s.ext[d] = 1e-30;
        }
        double span = s.ext[d] * s.width[d];
        double q = floor(span / a.rcb);
        int c = (q >= 1.0) ? (q > (double)kMaxCellsPerAxis ? kMaxCellsPerAxis : (int)q) : 1;
        s.nc[d] = c;
    }
    int cap = n_at > kMinCellCap ? n_at : kMinCellCap;
    while ((long long)s.nc[0] * s.nc[1] * s.nc[2] > (long long)cap) {
        int m = 0;
        if (s.nc[1] > s.nc[m]) m = 1;
        if (s.nc[2] > s.nc[m]) m = 2;
        if (s.nc[m] == 1) break;
        s.nc[m] = (s.nc[m] + 1) / 2;
    }
    double len[3];
    for (int d = 0; d < 3; ++d) {
        double cw = s.ext[d] * s.width[d] / s.nc[d];
        int R;
        if (!s.per[d] && s.nc[d] == 1) R = 0;
        else {
            double r = ceil(a.rcb / cw);
            if (r >= 1.0 && r <= (double)kMaxStencilRadius) R = (int)r;
            else {
                R = (r > (double)kMaxStencilRadius) ? kMaxStencilRadius : 1;
                if (n_at > 0) atomicOr(error_flag, NVAMD_NL_STATUS_CELL_TOO_THIN);
            }
            if (!s.per[d] && R > s.nc[d] - 1) R = s.nc[d] - 1;
        }
        s.R[d] = R;
        double sc = s.ext[d] / s.nc[d];
        double l2 = 0.0;
        for (int k = 0; k < 3; ++k) {
            s.step[3 * d + k] = sc * s.h[3 * d + k];
            l2 += s.step[3 * d + k] * s.step[3 * d + k];
        }
        len[d] = sqrt(l2);
    }
    s.n_cells = n_at > 0 ? s.nc[0] * s.nc[1] * s.nc[2] : 0;
    // Run length along axis 2: as long as the run's whole stencil is expected to fit one
    // batch of stencil cells and one LDS tile, and its centre atoms one pass.
    int zr = 1;
    if (s.n_cells > 0) {
        const double per_cell = 1.2 * (double)n_at / (double)s.n_cells;
        const int e01 = (2 * s.R[0] + 1) * (2 * s.R[1] + 1);
        for (int cand = 2; cand <= kMaxRun && cand <= s.nc[2]; ++cand) {
            const int entries = (cand + 2 * s.R[2]) * e01;
            if (entries > kStencilBatch) break;
            if (entries * per_cell + kWave > (double)kTile) break;
            if (cand * per_cell > (double)a.center_chunk) break;
            zr = cand;
        }
        const int runs = (s.nc[2] + zr - 1) / zr;
        zr = (s.nc[2] + runs - 1) / runs;  // same number of runs, evened out
    }
    s.zr = zr;
    s.n_units = s.n_cells > 0 ? s.nc[0] * s.nc[1] * ((s.nc[2] + zr - 1) / zr) : 0;
    // largest cell-local coordinate the search can meet
    const double reach = (s.R[0] + 1) * len[0] + (s.R[1] + 1) * len[1] + (s.R[2] + zr) * len[2];
    s.tol = (float)(2.0e-6 * (reach / a.rc + 1.0));
    // |q|^2 - 2 p.q against rc^2 - |p|^2 in float32, |p| and |q| at most reach: |q|^2 takes three roundings of
    // values up to reach^2, the three fused multiply-adds round values up to 3 reach^2 (|q|^2 + 2 |p.q|), the
    // threshold takes four roundings of values up to reach^2: (3 + 9 + 4) 2^-24 reach^2 = 0.96e-6 reach^2 in
    // all; the constant leaves nearly a factor of two
    s.tol_scan = (float)((double)s.tol + 1.8e-6 * (reach / a.rc) * (reach / a.rc));
}

__device__ __forceinline__ NlSearchSys search_view(const NlSys& s) {
    NlSearchSys q;
    for (int k = 0; k < 9; ++k) q.step[k] = (float)s.step[k];
    q.tol = s.tol;
    q.tol_scan = s.tol_scan;
    for (int d = 0; d < 3; ++d) {
        q.nc[d] = s.nc[d];
        q.R[d] = s.R[d];
        q.per[d] = s.per[d];
    }
    q.cell_offset = s.cell_offset;
    q.zr = s.zr;
    float d2max = 0.f;
    for (int sg = 0; sg < 4; ++sg) {
        const float a = (sg & 1) ? -1.f : 1.f, b = (sg & 2) ? -1.f : 1.f;
        float d2 = 0.f;
        for (int k = 0; k < 3; ++k) {
            const float v = q.step[k] + a * q.step[3 + k] + b * q.step[6 + k];
            d2 += v * v;
        }
        d2max = d2 > d2max ? d2 : d2max;
    }
    q.half_diag = 0.5f * sqrtf(d2max) * 1.0001f;
    // the stencil cell furthest from a run's nearest cell is a corner of the stencil
    float far2 = 0.f;
    for (int sg = 0; sg < 4; ++sg) {
        const float a = (sg & 1) ? -1.f : 1.f, b = (sg & 2) ? -1.f : 1.f;
        float d2 = 0.f;
        for (int k = 0; k < 3; ++k) {
            const float v = (float)q.R[0] * q.step[k] + a * (float)q.R[1] * q.step[3 + k] + b * (float)q.R[2] * q.step[6 + k];
            d2 += v * v;
        }
        far2 = d2 > far2 ? d2 : far2;
    }
    q.cull_far = sqrtf(far2) * 1.0001f;
    return q;
}

// ---- 3 grid ---------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void nl_grid_kernel(NlArgs a, NlWorkspace ws) {
    // low word: cells, high word: search units (both totals stay below 2^31, so the packed
    // sums never carry into each other)
    __shared__ unsigned long long s_scan[1024];
    __shared__ unsigned long long s_carry;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    for (int base = 0; base < a.n_systems; base += 1024) {
        int t = base + threadIdx.x;
        int ncell = 0, nunit = 0;
        if (t < a.n_systems) {
            NlSys s = ws.sys[t];
            choose_grid(s, a, ws.bounds + 6 * (size_t)t, &ws.hdr->error[ws.hdr->flip]);
            ncell = s.n_cells;
            nunit = s.n_units;
            ws.sys[t] = s;
        }
        // exclusive scan of both counts over the 1024 systems of this pass
        const unsigned long long mine = (unsigned long long)(unsigned)ncell | ((unsigned long long)(unsigned)nunit << 32);
        s_scan[threadIdx.x] = mine;
        __syncthreads();
        for (int o = 1; o < 1024; o <<= 1) {
            unsigned long long v = (int)threadIdx.x >= o ? s_scan[threadIdx.x - o] : 0ull;
            __syncthreads();
            s_scan[threadIdx.x] += v;
            __syncthreads();
        }
        const unsigned long long incl = s_scan[threadIdx.x];
        const unsigned long long carry = s_carry;
        if (t < a.n_systems) {
            const unsigned long long excl = carry + incl - mine;
            const int off = (int)(unsigned)(excl & 0xffffffffull);
            ws.sys[t].cell_offset = off;
            ws.cell_offset[t] = off;
            ws.unit_offset[t] = (int)(unsigned)(excl >> 32);
            ws.ssys[t] = search_view(ws.sys[t]);
        }
        __syncthreads();
        if (threadIdx.x == 1023) s_carry = carry + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const unsigned long long tot = s_carry;
        ws.cell_offset[a.n_systems] = (int)(unsigned)(tot & 0xffffffffull);
        ws.unit_offset[a.n_systems] = (int)(unsigned)(tot >> 32);
        ws.hdr->total_cells = (int)(unsigned)(tot & 0xffffffffull);
        ws.hdr->units[ws.hdr->flip] = (int)(unsigned)(tot >> 32);
    }
}

// ---- 4 bin / 6 scatter ----------------------------------------------------------------------
struct Binned {
    int cell;      // global cell id
    int w[3];      // wrap integers (periodic axes)
    float u[3];    // cartesian offset from the cell's corner
};

__device__ __forceinline__ Binned bin_atom(const NlSys& s, const Pos3& r) {
    Binned b;
    double f[3], g[3];
    frac_of(s, r, f);
    int c[3];
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        double fd = f[d];
        int w = 0;
        if (s.per[d]) {
            double fl = floor(fd);
            fl = fl > 2.0e9 ? 2.0e9 : (fl < -2.0e9 ? -2.0e9 : fl);
            w = (int)fl;
            fd -= fl;
        }
        b.w[d] = w;
        double x = (fd - s.lo[d]) / s.ext[d] * (double)s.nc[d];
        double fx = floor(x);
        int ci = fx < 0.0 ? 0 : (fx > (double)(s.nc[d] - 1) ? s.nc[d] - 1 : (int)fx);
        c[d] = ci;
        g[d] = x - (double)ci;
    }
    b.cell = s.cell_offset + (c[0] * s.nc[1] + c[1]) * s.nc[2] + c[2];
#pragma unroll
    for (int k = 0; k < 3; ++k)
        b.u[k] = (float)(g[0] * s.step[k] + g[1] * s.step[3 + k] + g[2] * s.step[6 + k]);
    return b;
}

// Unit lu of a system: the run-th run of cells along axis 2 in column (cx, cy).
__device__ __forceinline__ NlUnit make_unit(const NlSearchSys& q, int lu, int runs, int sys) {
    const int column = lu / runs, run = lu - column * runs;
    const int cx = column / q.nc[1], cy = column - cx * q.nc[1], cz0 = run * q.zr;
    NlUnit u;
    u.c0 = q.cell_offset + column * q.nc[2] + cz0;
    u.sidx = sys;
    u.cxyz = (cx << 20) | (cy << 10) | cz0;
    u.run_len = (q.nc[2] - cz0) < q.zr ? (q.nc[2] - cz0) : q.zr;
    u.nc_pack = (q.nc[0] - 1) | ((q.nc[1] - 1) << 10) | ((q.nc[2] - 1) << 20);
    u.rper_pack = q.R[0] | (q.R[1] << 6) | (q.R[2] << 12) | ((q.per[0] ? 1 : 0) << 18) | ((q.per[1] ? 1 : 0) << 19) |
                  ((q.per[2] ? 1 : 0) << 20);
    u.cell_offset = q.cell_offset;
    u.first_centre = -1;
    return u;
}

// Launched over max(atoms, cell bound) threads: thread t bins atom t and describes search unit t.
__global__ __launch_bounds__(kBlock) void nl_bin_kernel(NlArgs a, NlWorkspace ws) {
    int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < ws.hdr->units[ws.hdr->flip]) {
        // the system that owns unit i: the last one whose first unit is <= i
        int lo = 0, hi = a.n_systems;
        while (hi - lo > 1) {
            int mid = (lo + hi) >> 1;
            if (ws.unit_offset[mid] <= i) lo = mid; else hi = mid;
        }
        const NlSearchSys& q = ws.ssys[lo];
        const int lu = i - ws.unit_offset[lo];
        const int runs = (q.nc[2] + q.zr - 1) / q.zr;
        ws.units[i] = make_unit(q, lu, runs, lo);
    }
    if (i >= a.n_atoms) return;
    const NlSys& s = ws.sys[a.bidx[i]];
    Binned b = bin_atom(s, load_pos(a, (size_t)i));
    ws.atom_rank[i] = atomicAdd(ws.cell_count + b.cell, 1);
}

__global__ __launch_bounds__(kBlock) void nl_scatter_kernel(NlArgs a, NlWorkspace ws) {
    int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.n_atoms) return;
    const NlSys& s = ws.sys[a.bidx[i]];
    Binned b = bin_atom(s, load_pos(a, (size_t)i));
    int slot = ws.cell_start[b.cell] + ws.atom_rank[i];
    ws.sorted_pos[slot] = make_float4(b.u[0], b.u[1], b.u[2], __int_as_float(i));
    ws.sorted_aux[slot] = make_int4(b.w[0], b.w[1], b.w[2], 0);
    if (a.tile_xyz) {
        const Pos3 r = load_pos(a, (size_t)i);
        a.tile_xyz[slot] = make_float4((float)r.x, (float)r.y, (float)r.z, __int_as_float(i));
    }
}

// ---- per-system path: 1-6 in one workgroup per system -----------------------------------------
// For batches of many small systems.  One workgroup takes one system through set-up, bounds,
// grid choice, histogram (in LDS), scan and scatter; no global histogram, no global scan.
// Every system owns the cell ids [atom_begin + 9 s, ... + n_cells] (cells <= max(atoms, 8), plus
// one end entry), so cell ids need no prefix sum over the systems either.  A system with more
// cells than the LDS histogram holds is still handled, slowly, through global memory.
constexpr int kSortBlock = 512;   // (four workgroups per CU: a system's set-up is a chain of dependent steps that others hide)
constexpr int kSortCells = 8192;         // cells of a system whose histogram fits in LDS
constexpr int kPerSystemMeanAtoms = 8192;  // the path is taken up to this many atoms per system on average

__device__ __forceinline__ int block_exclusive_scan(int v, int* s_part, int* total) {
    // kSortBlock threads; s_part holds one partial per wave
    const int lane = lane_id(), wave = (int)threadIdx.x / kWave;
    int incl = v;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        int up = __shfl_up(incl, o, kWave);
        if (lane >= o) incl += up;
    }
    __syncthreads();  // s_part may still be read from a previous call
    if (lane == kWave - 1) s_part[wave] = incl;
    __syncthreads();
    int before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kSortBlock / kWave; ++w) {
        const int p = s_part[w];
        before += (w < wave) ? p : 0;
        all += p;
    }
    *total = all;
    return before + incl - v;
}

// kKeep: atoms per thread whose positions and bins stay in registers from the histogram to the scatter (systems of
// up to kKeep * kSortBlock atoms are binned once): four, or eight when the mean system has more than 2048 atoms.
// kWaves: waves per SIMD the kernel is built for.  With more systems than CUs the instance of four atoms is held to
// 128 registers (four waves per SIMD, two workgroups per CU: one system's chain of dependent steps then runs
// beside another's, 6 % off the build of 2048 mixed systems for 19 spilled words); with fewer systems than that
// nothing would run beside it, and it keeps its 152 registers (the spills cost 64 boxes of 500 atoms 2 %).
template <int kKeep, int kWaves>
__global__ __launch_bounds__(kSortBlock, kWaves) void nl_system_sort_kernel(NlArgs a, NlWorkspace ws) {
    __shared__ NlSys s_sys;
    __shared__ uint32_t s_bounds[6];
    __shared__ int s_err;
    __shared__ int s_unit0;
    __shared__ NlSearchSys s_view;
    __shared__ int s_hist[kSortCells + 1];  // counts, then first atoms (and the end of the last cell)
    __shared__ int s_part[kSortBlock / kWave];
    const int t = blockIdx.x;
    const int tid = threadIdx.x;
    // (which slot of the header this build counts in: asked for now, used when the units are reserved)
    const int slot = __builtin_amdgcn_readfirstlane(ws.hdr->flip);
    if (t == 0 && tid == 0) retire_other_slot(ws.hdr);
    const int begin = a.ptr[t], end = a.ptr[t + 1];
    // up to kKeep atoms per thread stay in registers from here to the scatter; their positions
    // are requested now, so that they arrive while thread 0 works out the system's grid
    const bool kept = !a.pos64 && (end - begin) <= kKeep * kSortBlock;
    float my_pos[kKeep][3];
    if (kept) {
#pragma unroll
        for (int k = 0; k < kKeep; ++k) {
            const int i = begin + tid + k * kSortBlock;
            const float* r = a.pos + 3 * (size_t)(i < end ? i : (end > begin ? begin : 0));
            my_pos[k][0] = r[0];
            my_pos[k][1] = r[1];
            my_pos[k][2] = r[2];
        }
    }
    if (tid < 6) s_bounds[tid] = tid < 3 ? 0xffffffffu : 0u;
    if (tid == 0) {
        s_err = 0;
        system_setup(s_sys, a, t);  // (worked on in place, in LDS)
    }
    __syncthreads();
    const int cell_base = begin + (kMinCellCap + 1) * t;
    const bool idle = end <= begin || (a.rebuild && !a.rebuild[t]);  // nothing to search: no cells, no units
    // ---- bounds on non-periodic axes
    if (!idle && !(s_sys.per[0] && s_sys.per[1] && s_sys.per[2])) {
        for (int i = begin + tid; i < end; i += kSortBlock) {
            double f[3];
            frac_of(s_sys, load_pos(a, (size_t)i), f);
#pragma unroll
            for (int d = 0; d < 3; ++d) {
                if (s_sys.per[d]) continue;
                float lo = __double2float_rd(f[d]), hi = __double2float_ru(f[d]);
                atomicMin(&s_bounds[d], float_order_key(lo));
                atomicMax(&s_bounds[3 + d], float_order_key(hi));
            }
        }
        __syncthreads();
    }
    // ---- grid
    if (tid == 0) {
        if (idle) {
            s_sys.n_cells = 0;
            s_sys.n_units = 0;
        } else {
            choose_grid(s_sys, a, s_bounds, &s_err);
        }
        s_sys.error = s_err;
        s_sys.cell_offset = cell_base;
        ws.cell_offset[t] = cell_base;
        if (s_err) atomicOr(&ws.hdr->error[slot], s_err);
    }
    __syncthreads();
    {
        // the system's record leaves LDS word by word
        const int* src = reinterpret_cast<const int*>(&s_sys);
        int* dst = reinterpret_cast<int*>(ws.sys + t);
        for (int w = tid; w < (int)(sizeof(NlSys) / sizeof(int)); w += kSortBlock) dst[w] = src[w];
        const NlSearchSys q = search_view(s_sys);
        if (tid == 0) {
            ws.ssys[t] = q;
            s_view = q;
        }
    }
    if (idle) return;
    const int n_cells = s_sys.n_cells;
    const bool in_lds = n_cells <= kSortCells;
    int* g_hist = ws.cell_count + cell_base;
    int* g_start = ws.cell_start + cell_base;
    // ---- histogram: rank of every atom inside its cell
    for (int c = tid; c < n_cells; c += kSortBlock) {
        if (in_lds) s_hist[c] = 0;
        else g_hist[c] = 0;
    }
    __syncthreads();
    Binned mine[kKeep];
    int my_rank[kKeep];
    if (kept) {
#pragma unroll
        for (int k = 0; k < kKeep; ++k) {
            const int i = begin + tid + k * kSortBlock;
            if (i < end) {
                mine[k] = bin_atom(s_sys, Pos3{(double)my_pos[k][0], (double)my_pos[k][1], (double)my_pos[k][2]});
                const int lc = mine[k].cell - cell_base;
                my_rank[k] = in_lds ? atomicAdd(&s_hist[lc], 1) : atomicAdd(&g_hist[lc], 1);
            }
        }
    } else {
        for (int i = begin + tid; i < end; i += kSortBlock) {
            const Binned b = bin_atom(s_sys, load_pos(a, (size_t)i));
            const int lc = b.cell - cell_base;
            ws.atom_rank[i] = in_lds ? atomicAdd(&s_hist[lc], 1) : atomicAdd(&g_hist[lc], 1);
        }
    }
    __syncthreads();
    // ---- scan: thread t owns a contiguous chunk of cells
    {
        const int chunk = (n_cells + kSortBlock - 1) / kSortBlock;
        const int c_lo = tid * chunk < n_cells ? tid * chunk : n_cells;
        const int c_hi = (c_lo + chunk) < n_cells ? (c_lo + chunk) : n_cells;
        int sum = 0;
        for (int c = c_lo; c < c_hi; ++c)
            sum += in_lds ? s_hist[c] : __hip_atomic_load(&g_hist[c], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int total;
        int running = begin + block_exclusive_scan(sum, s_part, &total);
        for (int c = c_lo; c < c_hi; ++c) {
            const int n = in_lds ? s_hist[c] : __hip_atomic_load(&g_hist[c], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (in_lds) {
                s_hist[c] = running;
                g_start[c] = running;
            } else {
                __hip_atomic_store(&g_start[c], running, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            running += n;
        }
        if (tid == 0) {
            g_start[n_cells] = end;
            if (in_lds) s_hist[n_cells] = end;
        }
    }
    __syncthreads();
    // ---- scatter into cell order
    auto place = [&](const Binned& b, int i, int rank) {
        const int lc = b.cell - cell_base;
        const int start = in_lds ? s_hist[lc] : __hip_atomic_load(&g_start[lc], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int slot = start + rank;
        ws.sorted_pos[slot] = make_float4(b.u[0], b.u[1], b.u[2], __int_as_float(i));
        ws.sorted_aux[slot] = make_int4(b.w[0], b.w[1], b.w[2], 0);
        if (a.tile_xyz) {
            const Pos3 r = load_pos(a, (size_t)i);
            a.tile_xyz[slot] = make_float4((float)r.x, (float)r.y, (float)r.z, __int_as_float(i));
        }
    };
    if (kept) {
#pragma unroll
        for (int k = 0; k < kKeep; ++k) {
            const int i = begin + tid + k * kSortBlock;
            if (i < end) place(mine[k], i, my_rank[k]);
        }
    } else {
        for (int i = begin + tid; i < end; i += kSortBlock) place(bin_atom(s_sys, load_pos(a, (size_t)i)), i, ws.atom_rank[i]);
    }
    __syncthreads();
    // ---- the system's units of search work.  A run of cells with more centre atoms than one
    //      pass of the search takes is split into one unit per pass (so that a system that is one
    //      crowded cell does not end up on a single workgroup); empty runs get none.
    {
        const NlSearchSys& q = s_view;
        const int n_runs = s_sys.n_units;
        const int runs = (q.nc[2] + q.zr - 1) / q.zr;
        auto first_atom = [&](int lc) {
            return in_lds ? s_hist[lc] : __hip_atomic_load(&g_start[lc], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        };
        auto centres_of = [&](const NlUnit& u) {
            const int lc0 = u.c0 - cell_base;
            const int n_centre = first_atom(lc0 + u.run_len) - first_atom(lc0);
            return n_centre;
        };
        auto passes_for = [&](int n_centre) { return (n_centre + a.center_chunk - 1) / a.center_chunk; };
        int mine_units = 0;
        for (int lu = tid; lu < n_runs; lu += kSortBlock) mine_units += passes_for(centres_of(make_unit(q, lu, runs, t)));
        int total;
        const int before = block_exclusive_scan(mine_units, s_part, &total);
        // a contiguous piece of the unit list, wherever the counter stands (the order of the
        // systems in the list is of no consequence)
        if (tid == 0) s_unit0 = total > 0 ? atomicAdd(&ws.hdr->units[slot], total) : 0;
        __syncthreads();
        NlUnit* out = ws.units + s_unit0 + before;
        for (int lu = tid; lu < n_runs; lu += kSortBlock) {
            NlUnit u = make_unit(q, lu, runs, t);
            const int n_centre = centres_of(u);
            const int passes = passes_for(n_centre);
            const int share = passes > 0 ? (n_centre + passes - 1) / passes : 0;  // equal shares, not full chunks and a rest
            for (int k = 0; k < passes; ++k) {
                u.first_centre = passes > 1 ? ((share << 24) | (k * share)) : -1;
                *out++ = u;
            }
        }
    }
}

// ---- 7 search -------------------------------------------------------------------------------
__device__ __forceinline__ int floordiv(int x, int n) {
    int q = x / n, r = x - q * n;
    return (r < 0) ? q - 1 : q;
}

__device__ __forceinline__ bool half_keep(int i, int j, int s0, int s1, int s2) {
    if (i != j) return i < j;
    if (s0 != 0) return s0 > 0;
    if (s1 != 0) return s1 > 0;
    return s2 > 0;
}

__device__ __forceinline__ int pack_shift(int x, int y, int z) {
    // three signed 5-bit fields; anything wider is flagged and recovered from global memory
    if ((unsigned)(x + 16) > 31u || (unsigned)(y + 16) > 31u || (unsigned)(z + 16) > 31u)
        return kPackOverflow;
    return (x + 16) | ((y + 16) << 5) | ((z + 16) << 10);
}

__device__ __forceinline__ float uniform_f(float v) {
    return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}

// Shift of candidate k relative to the centre atom: packed fast path, or (wide shifts) recovered
// from the sorted arrays through the stencil tables of the current batch.
struct ShiftSource {
    const unsigned short* c_pk;
    const int* st_prefix;
    const int* st_start;
    const int (*st_q)[3];
    const int4* sorted_aux;
    int t0;
};

__device__ __forceinline__ void candidate_shift(const ShiftSource& src, int k, int wi0, int wi1, int wi2,
                                                int& s0, int& s1, int& s2) {
    const int pk = src.c_pk[k];
    if (pk & kPackOverflow) {
        int flat = src.t0 + k, lo = 0, hi = kStencilBatch;
        for (int it = 0; it < 6; ++it) {
            int mid = (lo + hi) >> 1;
            if (src.st_prefix[mid] <= flat) lo = mid; else hi = mid;
        }
        int4 w = src.sorted_aux[src.st_start[lo] + (flat - src.st_prefix[lo])];
        s0 = src.st_q[lo][0] - w.x + wi0;
        s1 = src.st_q[lo][1] - w.y + wi1;
        s2 = src.st_q[lo][2] - w.z + wi2;
    } else {
        s0 = (pk & 31) - 16 + wi0;
        s1 = ((pk >> 5) & 31) - 16 + wi1;
        s2 = ((pk >> 10) & 31) - 16 + wi2;
    }
}

// A workgroup's unit of work is a run of up to kMaxRun cells that follow each other along
// axis 2 (they are consecutive cell ids, so their atoms are one contiguous slice of the
// sorted arrays).  The run's stencil is enumerated layer by layer along axis 2, so the
// candidates a centre cell of the run has to look at are one contiguous range of the LDS tile;
// what a range picks up beyond its own layers (ranges are widened to multiples of 64) lies
// further than the stencil radius away and can never pass the distance test.
template <bool HALF, bool F64, bool TILES, bool SPARSE>
// The tables that every lane of a workgroup reads at the same address (unit records, the per-system
// constants, the run's cell ranges) come in as read-only arguments of their own besides the workspace:
// nothing in the kernel can be seen to write them, so they are fetched through the scalar cache, which
// answers sooner than the vector path and keeps these loads out of the order of the row stores.
__global__ __launch_bounds__(kBlock, 5) void nl_search_kernel(NlArgs a, NlWorkspace ws,
                                                              const NlUnit* __restrict__ units_ro,
                                                              const NlSearchSys* __restrict__ ssys_ro,
                                                              const int* __restrict__ cell_start_ro) {
    __shared__ float4 c_pos[kTile];           // candidate: xyz relative to the run's first cell, and |xyz|^2
    __shared__ int c_j[kTile];                // its atom index
    __shared__ unsigned short c_pk[kTile];    // packed (image of its cell - its own wrap)
    __shared__ float4 ca_pos[kCenterChunk];   // centre atoms of this pass: same frame + atom index
    __shared__ int4 ca_w[kCenterChunk];       // their wrap integers; .w = place of their cell in the run
    __shared__ int ca_pad[kCenterChunk];      // slot up to which their row has to be padded afterwards
    __shared__ int4 ca_meta[kCenterChunk];    // per batch of stencil cells: flat slot of the centre itself, first and
                                              // last candidate to scan; .w = running row length
    __shared__ int st_start[kStencilBatch];
    __shared__ int st_prefix[kStencilBatch + 1];
    __shared__ int st_q[kStencilBatch][3];
    __shared__ float st_off[kStencilBatch][3];
    __shared__ unsigned short hits[kWavesPerBlock][kHitCap + 2];

    // (the counter of the slot that this build did not use is zero: see NlHeader)
    const int total_units = ws.hdr->units[0] + ws.hdr->units[1];
    if (blockIdx.x == 0 && threadIdx.x == 0) ws.hdr->flip ^= 1;
    if (TILES && blockIdx.x == 0 && threadIdx.x == 0) *a.tile_count = total_units;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x / kWave);
    const float rc2f = (float)a.rc2;
    const float cull_reach = (float)a.rcb * 1.001f;
    // Consecutive workgroups go to the 8 XCDs round-robin; the units are dealt to the XCDs in
    // groups of consecutive units, so the stencil data an XCD re-reads stays in its own L2.  The
    // dealing does not depend on the number of units: a workgroup asks for its first unit and
    // for that number at the same time.
    const int xcd = blockIdx.x % 8, slot0 = blockIdx.x / 8, stride = gridDim.x / 8;
    const int group = a.unit_group;  // a power of two
    const int last_unit = ws.max_cells - 1;

    for (int li = slot0;; li += stride) {
        // NOTE: every thread of the workgroup takes the same path through this loop body
        const int round0 = (li / group) * 8 * group;  // first unit of this round of 8 groups
        const int u = round0 + xcd * group + li % group;
        const int4* rec = reinterpret_cast<const int4*>(units_ro + (u < last_unit ? u : last_unit));
        const int4 unit = rec[0], grid = rec[1];  // (asked for before u is known to exist)
        if (round0 >= total_units) break;
        if (u >= total_units) continue;
        const int c0 = __builtin_amdgcn_readfirstlane(unit.x);
        const int sidx = __builtin_amdgcn_readfirstlane(unit.y);
        const int cxyz = __builtin_amdgcn_readfirstlane(unit.z);
        const int run_len = __builtin_amdgcn_readfirstlane(unit.w);
        const int nc_pack = __builtin_amdgcn_readfirstlane(grid.x);
        const int rper = __builtin_amdgcn_readfirstlane(grid.y);
        const int cell_offset = __builtin_amdgcn_readfirstlane(grid.z);
        if (a.rebuild && !a.rebuild[sidx]) continue;
        const NlSearchSys S = ssys_ro[sidx];  // (the cell steps and the tolerance are taken from here)
        const int nc0 = (nc_pack & 1023) + 1, nc1 = ((nc_pack >> 10) & 1023) + 1, nc2 = ((nc_pack >> 20) & 1023) + 1;
        const int per0 = (rper >> 18) & 1, per1 = (rper >> 19) & 1, per2 = (rper >> 20) & 1;
        const int cz0 = cxyz & 1023, cy = (cxyz >> 10) & 1023, cx = cxyz >> 20;
        const int c_begin = cell_start_ro[c0];
        // first centre atom (relative to c_begin) of the run's cells 1, 2, 3 and the run's end
        int run_off[kMaxRun + 1];
        run_off[0] = 0;
#pragma unroll
        for (int r = 1; r <= kMaxRun; ++r) run_off[r] = cell_start_ro[c0 + (r < run_len ? r : run_len)] - c_begin;
        const int R0 = rper & 63, R1 = (rper >> 6) & 63, R2 = (rper >> 12) & 63;
        const int e1 = 2 * R1 + 1, e01 = (2 * R0 + 1) * e1;
        const int n_layers = run_len + 2 * R2;
        const int n_stencil = n_layers * e01;
        // one batch of stencil cells and (checked below) one tile: rows are finished in place and
        // every centre atom scans only the layers of its own cell's stencil
        const bool one_batch = n_stencil <= kStencilBatch;
        const float rc2_lo = rc2f * (1.0f - S.tol), rc2_hi = rc2f * (1.0f + S.tol), rc2_scan = rc2f * (1.0f + S.tol_scan);
        // (square cells never have a stencil cell out of reach: the test is skipped for them)
        const bool may_cull = S.cull_far > cull_reach + 2.0f * S.half_diag;
        // One batch of stencil cells: the last wave enumerates up to 64 of them, one per lane, and scans
        // their sizes.  (The other waves load centre atoms meanwhile: the round trips to memory run
        // side by side.)  The cells' ranges need nothing but the unit record.
        auto enumerate_stencil = [&](const int sb, const bool first) {
            const int si = sb + lane;
            int start = 0, count = 0, q0 = 0, q1 = 0, q2 = 0;
            float o0 = 0.f, o1 = 0.f, o2 = 0.f;
            if (si < n_stencil) {
                const int layer = si / e01, in_layer = si - layer * e01;
                const int oz = layer - R2, oy = in_layer % e1 - R1, ox = in_layer / e1 - R0;
                int gx = cx + ox, gy = cy + oy, gz = cz0 + oz;
                bool ok = true;
                if (per0) { q0 = floordiv(gx, nc0); gx -= q0 * nc0; } else ok = ok && gx >= 0 && gx < nc0;
                if (per1) { q1 = floordiv(gy, nc1); gy -= q1 * nc1; } else ok = ok && gy >= 0 && gy < nc1;
                if (per2) { q2 = floordiv(gz, nc2); gz -= q2 * nc2; } else ok = ok && gz >= 0 && gz < nc2;
                if (ok) {
                    // the cell's range is asked for first: it needs nothing but the unit record,
                    // so it does not wait for the system's constants
                    const int c2 = cell_offset + (gx * nc1 + gy) * nc2 + gz;
                    start = ws.cell_start[c2];
                    const int end = ws.cell_start[c2 + 1];
                    float fx = (float)ox, fy = (float)oy, fz = (float)oz;
                    o0 = fx * S.step[0] + fy * S.step[3] + fz * S.step[6];
                    o1 = fx * S.step[1] + fy * S.step[4] + fz * S.step[7];
                    o2 = fx * S.step[2] + fy * S.step[5] + fz * S.step[8];
                    // Skewed cells put far-away images into the stencil.  A cell whose centre is
                    // further than the search radius plus two half-diagonals from the centre of
                    // every cell of the run holds no neighbor (no two points of two cells are
                    // closer than their centres minus the half-diagonals): it is left empty.
                    float best = 0.f;
                    if (may_cull) best = 3.0e38f;
                    for (int r = 0; may_cull && r < run_len; ++r) {
                        const float dx = o0 - (float)r * S.step[6], dy = o1 - (float)r * S.step[7],
                                    dz = o2 - (float)r * S.step[8];
                        const float d2 = dx * dx + dy * dy + dz * dz;
                        best = d2 < best ? d2 : best;
                    }
                    const float lim = cull_reach + 2.0f * S.half_diag;
                    count = (best <= lim * lim) ? end - start : 0;
                    if (count == 0) start = 0;
                }
            }
            int incl = count;
#pragma unroll
            for (int o = 1; o < kWave; o <<= 1) {
                int up = __shfl_up(incl, o, kWave);
                if (lane >= o) incl += up;
            }
            st_start[lane] = start;
            st_prefix[lane] = incl - count;
            if (lane == kWave - 1) st_prefix[kStencilBatch] = incl;
            st_q[lane][0] = q0; st_q[lane][1] = q1; st_q[lane][2] = q2;
            st_off[lane][0] = o0; st_off[lane][1] = o1; st_off[lane][2] = o2;
            if (TILES && first) {
                // the unit's record for the pair kernel: the tile is laid out by these numbers alone, the same for
                // all passes of a unit; "no tile" unless the whole stencil is one batch and one tile
                int2* const record = a.tile_records + (size_t)u * kTileRecord;
                const int total = __shfl(incl, kWave - 1, kWave);
                record[2 + lane] = make_int2(start, incl - count);
                if (lane == 0) record[1] = make_int2(sidx, (one_batch && total <= kTile) ? total : -1);
            }
        };
        // The first batch is enumerated before the run's own cell ranges have arrived.  (Nobody reads
        // the tables of the previous unit any more: its last pass ended with a barrier.)
        if (wave == kWavesPerBlock - 1) enumerate_stencil(0, true);
        const int n_center = run_off[kMaxRun];
        // the run's centre atoms, one pass at a time; or the one pass this unit stands for
        const int first_centre = __builtin_amdgcn_readfirstlane(grid.w);
        const int cc_begin = first_centre >= 0 ? (first_centre & 0xffffff) : 0;
        const int cc_share = first_centre >= 0 ? (first_centre >> 24) : n_center;
        const int cc_end = (cc_begin + cc_share) < n_center ? (cc_begin + cc_share) : n_center;
        // the unit's rows for the pair kernel (slots of the cell order); the rest of its record is written with the
        // stencil tables
        if (TILES && threadIdx.x == 0)
            a.tile_records[(size_t)u * kTileRecord] = make_int2(c_begin + cc_begin, cc_end > cc_begin ? cc_end - cc_begin : 0);
        if (n_center == 0) continue;
        for (int cc0 = cc_begin; cc0 < cc_end; cc0 += kCenterChunk) {
            const int n_cc = (cc_end - cc0) < kCenterChunk ? (cc_end - cc0) : kCenterChunk;
            int pad_end = 0;
            if ((int)threadIdx.x < n_cc) {
                const int ca_abs = cc0 + (int)threadIdx.x;
                int r = 0;
#pragma unroll
                for (int q = 1; q < kMaxRun; ++q) r += (ca_abs >= run_off[q]) ? 1 : 0;
                float4 p = ws.sorted_pos[c_begin + ca_abs];
                int4 w = ws.sorted_aux[c_begin + ca_abs];
                const float fr = (float)r;
                p.x += fr * S.step[6];
                p.y += fr * S.step[7];
                p.z += fr * S.step[8];
                // what the row must be padded up to afterwards: all of it, or what the previous build
                // left.  That count is a gather two loads deep; it is asked for here and stored to LDS
                // only after the tile has been staged, so nothing before that waits for it.
                pad_end = a.tail_mode ? a.K : a.nn[__float_as_int(p.w)];
                w.w = r;
                ca_pos[threadIdx.x] = p;
                ca_w[threadIdx.x] = w;
                ca_meta[threadIdx.x].w = 0;
            }

            for (int sb = 0; sb < n_stencil; sb += kStencilBatch) {
                if (wave == kWavesPerBlock - 1 && !(sb == 0 && cc0 == cc_begin)) enumerate_stencil(sb, false);
                __syncthreads();
                const int batch_total = st_prefix[kStencilBatch];
                const int n_entries = (n_stencil - sb) < kStencilBatch ? (n_stencil - sb) : kStencilBatch;
                const bool fused = one_batch && batch_total <= kTile;
                if ((int)threadIdx.x < n_cc) {
                    // The centre atom meets itself (shift 0) at exactly one slot of the flattened
                    // stencil: in its own cell, i.e. layer r + R2, at the middle of that layer.
                    const int r = ca_w[threadIdx.x].w;
                    const int e_self = (r + R2) * e01 + R0 * e1 + R1;
                    int self_flat = -1;
                    if (e_self >= sb && e_self < sb + kStencilBatch) {
                        int first_of_cell = 0;  // run_off[r] without dynamic indexing
#pragma unroll
                        for (int q = 1; q < kMaxRun; ++q) first_of_cell = (r == q) ? run_off[q] : first_of_cell;
                        self_flat = st_prefix[e_self - sb] + (cc0 + (int)threadIdx.x - first_of_cell);
                    }
                    // candidates to scan: the centre's own layers when rows are finished in place
                    int lo = 0, hi = 0x7fffffff;
                    if (fused) {
                        lo = st_prefix[r * e01] & ~(kWave - 1);
                        hi = (st_prefix[(r + 2 * R2 + 1) * e01] + kWave - 1) & ~(kWave - 1);
                    }
                    ca_meta[threadIdx.x].x = self_flat;
                    ca_meta[threadIdx.x].y = lo;
                    ca_meta[threadIdx.x].z = hi;
                }

                for (int t0 = 0; t0 < batch_total; t0 += kTile) {
                    const int tile_n = (batch_total - t0) < kTile ? (batch_total - t0) : kTile;
                    const int tile_pad = (tile_n + kWave - 1) & ~(kWave - 1);
                    // ---- stage the tile: thread t takes flat candidates t, t + 256, ...; all of a
                    //      thread's global loads are in flight together (indices are clamped rather
                    //      than branched over), then shifted by the stencil cell's offset
                    {
                        constexpr int kPer = (kTile + kBlock - 1) / kBlock;
                        float4 sp[kPer];
                        int4 sw[kPer];
                        int se[kPer];
#pragma unroll
                        for (int i = 0; i < kPer; ++i) {
                            const int f = (int)threadIdx.x + i * kBlock;
                            const int flat = t0 + (f < tile_n ? f : tile_n - 1);
                            int e = 0;  // the stencil cell this candidate belongs to
#pragma unroll
                            for (int step = kStencilBatch / 2; step > 0; step >>= 1)
                                if (st_prefix[e + step] <= flat) e += step;
                            const int src = st_start[e] + (flat - st_prefix[e]);
                            se[i] = e;
                            sp[i] = ws.sorted_pos[src];
                            sw[i] = ws.sorted_aux[src];
                        }
#pragma unroll
                        for (int i = 0; i < kPer; ++i) {
                            const int f = (int)threadIdx.x + i * kBlock;
                            if (f < tile_n) {
                                const int e = se[i];
                                float4 p = sp[i];
                                p.x += st_off[e][0];
                                p.y += st_off[e][1];
                                p.z += st_off[e][2];
                                c_j[f] = __float_as_int(p.w);
                                p.w = p.x * p.x + p.y * p.y + p.z * p.z;
                                c_pos[f] = p;
                                c_pk[f] = (unsigned short)pack_shift(st_q[e][0] - sw[i].x, st_q[e][1] - sw[i].y, st_q[e][2] - sw[i].z);
                            }
                        }
                    }
                    // padding up to a multiple of 64: candidates that no centre atom can reach
                    if ((int)threadIdx.x < tile_pad - tile_n)
                        c_pos[tile_n + threadIdx.x] = make_float4(0.f, 0.f, 0.f, 3.0e38f);
                    // Every load above has landed before the centre loop starts (vmcnt(0)): otherwise
                    // the loop would begin each turn with a wait on "the loads that may still be in
                    // flight", which, the counter being in-order, waits for the previous centre
                    // atom's row stores instead.
                    if ((int)threadIdx.x < n_cc) ca_pad[threadIdx.x] = pad_end < a.K ? pad_end : a.K;
                    __builtin_amdgcn_s_waitcnt(0x0F70);
                    __syncthreads();

                    const ShiftSource shifts{c_pk, st_prefix, st_start, st_q, ws.sorted_aux, t0};

                    // ---- each wave: its centre atoms against the tile, 64 candidates a step
                    for (int ca = wave; ca < n_cc; ca += kWavesPerBlock) {
                        const float4 ci = ca_pos[ca];
                        const int4 wa = ca_w[ca];
                        // The scan evaluates |q|^2 - 2 p.q against rc^2 - |p|^2: three fused multiply-adds and a
                        // comparison per candidate, with |q|^2 staged beside q.  (-2 p is kept; p = -0.5 (-2 p) exactly.)
                        float m2x = -2.0f * ci.x, m2y = -2.0f * ci.y, m2z = -2.0f * ci.z;
                        asm volatile("" : "+v"(m2x), "+v"(m2y), "+v"(m2z));  // (so that the products, not ci, go to scalar registers)
                        const float mx = uniform_f(m2x), my = uniform_f(m2y), mz = uniform_f(m2z);
                        const float scan_lim = uniform_f(rc2_scan - (ci.x * ci.x + ci.y * ci.y + ci.z * ci.z));
                        const int i_atom = __builtin_amdgcn_readfirstlane(__float_as_int(ci.w));
                        const int wi0 = __builtin_amdgcn_readfirstlane(wa.x);
                        const int wi1 = __builtin_amdgcn_readfirstlane(wa.y);
                        const int wi2 = __builtin_amdgcn_readfirstlane(wa.z);
                        const int hi_slot = __builtin_amdgcn_readfirstlane(ca_pad[ca]);
                        const int4 meta = ca_meta[ca];
                        const int self_flat = __builtin_amdgcn_readfirstlane(meta.x);
                        const int k_self = self_flat >= 0 ? self_flat - t0 : -1;
                        const int k_lo = __builtin_amdgcn_readfirstlane(meta.y);
                        const int k_hi_all = __builtin_amdgcn_readfirstlane(meta.z);
                        const int k_hi = k_hi_all < tile_pad ? k_hi_all : tile_pad;
                        int base = __builtin_amdgcn_readfirstlane(meta.w);  // found before this tile
                        int32_t* row = a.nm + (size_t)i_atom * a.K;
                        int32_t* srow = a.shifts ? a.shifts + (size_t)i_atom * a.K * 3 : nullptr;
                        // which groups of the row's slots may hold a shift that is not zero (rows that are not finished
                        // in one piece write every shift and come out as dirty all over); asked for here, used at the
                        // first write of the row
                        const unsigned was_dirty = (SPARSE && fused && a.shifts) ? a.shift_groups[i_atom] : 0xffffffffu;
                        unsigned now_dirty = 0;                             // (the same in every lane)
                        int nh = 0;                                         // entries in the hit list
                        unsigned short* my_hits = hits[wave];

                        // One step: 64 candidates against the centre atom, one comparison each: whatever
                        // is inside the outer edge of the float32 uncertainty band goes to the wave's hit
                        // list.  The list is a superset: it still holds the centre atom itself (distance 0)
                        // and the few candidates inside the band.
                        auto scan_form = [&](const float4& p) { return fmaf(p.z, mz, fmaf(p.y, my, fmaf(p.x, mx, p.w))); };
                        auto dist2 = [&](const float4& p) {
                            const float dx = fmaf(mx, 0.5f, p.x), dy = fmaf(my, 0.5f, p.y), dz = fmaf(mz, 0.5f, p.z);
                            return dx * dx + dy * dy + dz * dz;
                        };
                        auto accept = [&](const int k, const float4& p, const float t) {
                            const bool take = t < scan_lim;
                            const unsigned long long m = __builtin_amdgcn_ballot_w64(take);
                            // (no branch around the store: lanes without a hit write to a slot past the list)
                            const int before = __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32),
                                                                         __builtin_amdgcn_mbcnt_lo((unsigned)m, 0));
                            my_hits[take ? nh + before : kHitCap] = (unsigned short)k;
                            nh += __popcll(m);
                        };
                        // Writing the list out, 64 entries a step: the self entry is dropped, an entry
                        // inside the band is decided by the exact expression (rare), the rest get their
                        // shift and their slot.  This keeps everything but one comparison out of the
                        // per-candidate loop.
                        auto flush = [&]() {
                            // (straight-line code: every lane reads some candidate, the lanes without an
                            // entry read candidate 0 and drop out at the ballot; the two rare cases, a shift
                            // too wide for its packed form and a candidate inside the band, share one branch)
                            for (int l0 = 0; l0 < nh; l0 += kWave) {
                                const int l = l0 + lane;
                                const int k_read = my_hits[l < nh ? l : 0];
                                bool in = l < nh && k_read != k_self;
                                const int k = in ? k_read : 0;
                                const float4 p = c_pos[k];
                                const int pk = c_pk[k];
                                const int j = c_j[k];
                                int s0 = (pk & 31) - 16 + wi0;
                                int s1 = ((pk >> 5) & 31) - 16 + wi1;
                                int s2 = ((pk >> 10) & 31) - 16 + wi2;
                                const bool wide = (pk & kPackOverflow) != 0;
                                const float d2 = dist2(p);
                                in = in && d2 < rc2_hi;  // (the scan's form lets a few more through than this one)
                                const bool band = !(d2 < rc2_lo);
                                if (__builtin_expect(__builtin_amdgcn_ballot_w64(in && (wide || band)) != 0, 0)) {
                                    if (in && wide) candidate_shift(shifts, k, wi0, wi1, wi2, s0, s1, s2);
                                    if (in && band) {  // inside the band: decide exactly
                                        // (the type of the positions is a compile-time matter here: looking at it
                                        // at run time costs the float32 kernel registers it does not have)
                                        Pos3 pi, pj;
                                        if (F64) {
                                            pi = Pos3{a.pos64[3 * (size_t)i_atom], a.pos64[3 * (size_t)i_atom + 1], a.pos64[3 * (size_t)i_atom + 2]};
                                            pj = Pos3{a.pos64[3 * (size_t)j], a.pos64[3 * (size_t)j + 1], a.pos64[3 * (size_t)j + 2]};
                                        } else {
                                            const float* fi = a.pos + 3 * (size_t)i_atom;
                                            const float* fj = a.pos + 3 * (size_t)j;
                                            pi = Pos3{(double)fi[0], (double)fi[1], (double)fi[2]};
                                            pj = Pos3{(double)fj[0], (double)fj[1], (double)fj[2]};
                                        }
                                        double e0, e1d, e2d;
                                        in = pair_d2_exact(pi.x, pi.y, pi.z, pj.x, pj.y, pj.z, s0, s1, s2,
                                                           ws.sys[sidx].h, e0, e1d, e2d) < a.rc2;
                                    }
                                }
                                if (HALF) in = in && half_keep(i_atom, j, s0, s1, s2);
                                const unsigned long long m = __builtin_amdgcn_ballot_w64(in);
                                const int slot = base + __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32),
                                                                                  __builtin_amdgcn_mbcnt_lo((unsigned)m, 0));
                                bool store_shift = srow != nullptr;
                                if (SPARSE && m != 0) {
                                    // These entries go to slots [base, base + n): their shifts are left unwritten if all
                                    // of them are zero and the groups they fall into held nothing but zeros; one
                                    // decision for the whole step, taken on scalar registers.
                                    const int s_hi = base + __popcll(m) - 1;
                                    const int g_lo = (base < a.K - 1 ? base : a.K - 1) >> a.group_shift;
                                    const int g_hi = (s_hi < a.K - 1 ? s_hi : a.K - 1) >> a.group_shift;
                                    const unsigned groups = (2u << g_hi) - (1u << g_lo);
                                    const bool any_shift = __builtin_amdgcn_ballot_w64(in && (s0 | s1 | s2) != 0) != 0;
                                    if (any_shift) now_dirty |= groups;
                                    store_shift = store_shift && (any_shift || (was_dirty & groups) != 0);
                                }
                                if (in && slot < a.K) {
                                    // (the rows are written past the caches' retention, like the shifts below: what the
                                    // search re-reads, the sorted atoms of neighboring units, keeps its place in L2)
                                    __builtin_nontemporal_store(j, &row[slot]);
                                    if (TILES) __builtin_nontemporal_store((uint16_t)k, &a.tile_index[(size_t)i_atom * a.K + slot]);
                                    if (store_shift) {
                                        __builtin_nontemporal_store(s0, &srow[3 * slot + 0]);
                                        __builtin_nontemporal_store(s1, &srow[3 * slot + 1]);
                                        __builtin_nontemporal_store(s2, &srow[3 * slot + 2]);
                                    }
                                }
                                base += __popcll(m);
                            }
                            nh = 0;
                        };
                        int k0 = k_lo;
                        // four steps' candidates are in flight at once (the registers are there: the
                        // kernel's register count is set by its set-up phases, not by this loop)
                        for (; k0 + 3 * kWave < k_hi; k0 += 4 * kWave) {
                            const int k = k0 + lane;
                            const float4 pa = c_pos[k], pb = c_pos[k + kWave], pc = c_pos[k + 2 * kWave],
                                         pd = c_pos[k + 3 * kWave];
                            const float da = scan_form(pa), db = scan_form(pb), dc = scan_form(pc), dd = scan_form(pd);
                            accept(k, pa, da);
                            accept(k + kWave, pb, db);
                            if (__builtin_expect(nh > kHitCap - 2 * kWave, 0)) flush();
                            accept(k + 2 * kWave, pc, dc);
                            accept(k + 3 * kWave, pd, dd);
                            if (__builtin_expect(nh > kHitCap - 2 * kWave, 0)) flush();
                        }
                        for (; k0 + kWave < k_hi; k0 += 2 * kWave) {
                            const int k = k0 + lane;
                            const float4 pa = c_pos[k], pb = c_pos[k + kWave];
                            const float da = scan_form(pa), db = scan_form(pb);
                            accept(k, pa, da);
                            accept(k + kWave, pb, db);
                            if (__builtin_expect(nh > kHitCap - 2 * kWave, 0)) flush();
                        }
                        if (k0 < k_hi) {
                            const int k = k0 + lane;
                            const float4 pa = c_pos[k];
                            accept(k, pa, scan_form(pa));
                        }
                        flush();
                        if (fused) {
                            // ---- count, and padding over what the previous build left beyond it
                            for (int k = base + lane; k < hi_slot; k += kWave) {
                                row[k] = a.n_atoms;
                                if (srow && (!SPARSE || ((was_dirty >> (k >> a.group_shift)) & 1u))) {
                                    srow[3 * k + 0] = 0;
                                    srow[3 * k + 1] = 0;
                                    srow[3 * k + 2] = 0;
                                }
                            }
                            if (lane == 0) {
                                a.nn[i_atom] = base;
                                if (SPARSE && srow) a.shift_groups[i_atom] = now_dirty;
                                if (base > a.K) atomicOr(&ws.hdr->error[ws.hdr->units[1] > 0 ? 1 : 0], NVAMD_NL_STATUS_ROW_OVERFLOW);
                            }
                        } else if (lane == 0) {
                            ca_meta[ca].w = base;
                        }
                    }
                    __syncthreads();
                }
                __syncthreads();  // everyone has read this batch's tables before wave 0 rewrites them
            }

            if (!(one_batch && st_prefix[kStencilBatch] <= kTile)) {
                // several batches or tiles: counts were carried in LDS, finish the rows now
                for (int ca = wave; ca < n_cc; ca += kWavesPerBlock) {
                    const int i_atom = __builtin_amdgcn_readfirstlane(__float_as_int(ca_pos[ca].w));
                    const int cnt = __builtin_amdgcn_readfirstlane(ca_meta[ca].w);
                    const int hi_slot = __builtin_amdgcn_readfirstlane(ca_pad[ca]);
                    int32_t* row = a.nm + (size_t)i_atom * a.K;
                    int32_t* srow = a.shifts ? a.shifts + (size_t)i_atom * a.K * 3 : nullptr;
                    for (int k = cnt + lane; k < hi_slot; k += kWave) {
                        row[k] = a.n_atoms;
                        if (srow) {
                            srow[3 * k + 0] = 0;
                            srow[3 * k + 1] = 0;
                            srow[3 * k + 2] = 0;
                        }
                    }
                    if (lane == 0) {
                        a.nn[i_atom] = cnt;
                        if (SPARSE && srow) a.shift_groups[i_atom] = 0xffffffffu;
                        if (cnt > a.K) atomicOr(&ws.hdr->error[ws.hdr->units[1] > 0 ? 1 : 0], NVAMD_NL_STATUS_ROW_OVERFLOW);
                    }
                }
            }
            __syncthreads();
        }
    }
}

__global__ void nl_status_kernel(NlHeader* hdr, int32_t* out, int clear) {
    // (between builds flip names the slot of the next build: the last one used the other)
    const int now = hdr->error[hdr->flip ^ 1], all = hdr->sticky | hdr->error[0] | hdr->error[1];
    out[0] = now;
    out[1] = all;
    if (clear) {
        hdr->sticky = 0;
        hdr->error[0] = 0;
        hdr->error[1] = 0;
    }
}

__global__ __launch_bounds__(kBlock) void nl_atom_order_kernel(const float4* __restrict__ sorted_pos,
                                                               const int32_t* __restrict__ bidx,
                                                               const uint8_t* __restrict__ flags, int n_atoms,
                                                               int32_t* __restrict__ order) {
    int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= n_atoms) return;
    // slot k of the sorted arrays belongs to the system atom k belongs to (both are laid out by batch_ptr)
    if (flags && !flags[bidx[k]]) return;
    order[k] = __float_as_int(sorted_pos[k].w);
}

}  // namespace
}  // namespace nvamd

using namespace nvamd;

NVAMD_EXPORT int32_t nvamd_nl_atom_order(const void* workspace, size_t workspace_bytes, const int32_t* batch_idx,
                                         const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                                         int32_t* atom_order, void* stream) {
    if (n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "atom order: negative size");
    if (n_atoms == 0 || n_systems == 0) return NVAMD_OK;
    if (!atom_order || !batch_idx) return fail(NVAMD_ERR_INVALID_ARGUMENT, "atom order: null buffer");
    size_t need = carve(nullptr, nullptr, n_atoms, n_systems);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "atom order: workspace %zu < %zu bytes", workspace_bytes, need);
    NlWorkspace ws;
    carve(&ws, static_cast<char*>(const_cast<void*>(workspace)), n_atoms, n_systems);
    hipLaunchKernelGGL(nl_atom_order_kernel, dim3((n_atoms + kBlock - 1) / kBlock), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), ws.sorted_pos, batch_idx, rebuild_flags, n_atoms, atom_order);
    NVAMD_LAUNCH_CHECK("atom order launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_status(void* workspace, size_t workspace_bytes, int32_t n_atoms, int32_t n_systems,
                                     int32_t* status, int32_t clear, void* stream) {
    if (n_atoms < 0 || n_systems < 0 || !status) return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl status: bad argument");
    size_t need = carve(nullptr, nullptr, n_atoms, n_systems);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "nl status: workspace %zu < %zu bytes", workspace_bytes, need);
    NlWorkspace ws;
    carve(&ws, static_cast<char*>(workspace), n_atoms, n_systems);
    hipLaunchKernelGGL(nl_status_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), ws.hdr, status,
                       clear ? 1 : 0);
    NVAMD_LAUNCH_CHECK("nl status launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_workspace_bytes(int32_t n_atoms, int32_t n_systems, size_t* bytes) {
    if (!bytes || n_atoms < 0 || n_systems < 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl workspace: bad argument");
    *bytes = carve(nullptr, nullptr, n_atoms, n_systems);
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_build(const float* positions, const float* cell, const uint8_t* pbc,
                                    const int32_t* batch_ptr, const int32_t* batch_idx,
                                    const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                                    double cutoff, int32_t max_neighbors, int32_t half_fill,
                                    int32_t tail_mode, int32_t* neighbor_matrix, int32_t* num_neighbors,
                                    int32_t* neighbor_matrix_shifts, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    return nvamd_nl_build_path(positions, cell, pbc, batch_ptr, batch_idx, rebuild_flags, n_atoms, n_systems, cutoff,
                               max_neighbors, half_fill, tail_mode, NVAMD_NL_SORT_AUTO, neighbor_matrix, num_neighbors,
                               neighbor_matrix_shifts, workspace, workspace_bytes, stream);
}

static int32_t nl_build_impl(const float* positions, const float* cell, const double* positions64, const double* cell64,
                             const uint8_t* pbc, const int32_t* batch_ptr, const int32_t* batch_idx,
                             const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems, double cutoff,
                             int32_t max_neighbors, int32_t half_fill, int32_t tail_mode, int32_t sort_path,
                             int32_t* neighbor_matrix, int32_t* num_neighbors, int32_t* neighbor_matrix_shifts,
                             void* workspace, size_t workspace_bytes, void* stream, uint16_t* tile_index = nullptr,
                             float* ordered_positions = nullptr, int32_t* tile_records = nullptr,
                             int32_t* tile_count = nullptr, uint32_t* shift_groups = nullptr) {
    if (sort_path != NVAMD_NL_SORT_AUTO && sort_path != NVAMD_NL_SORT_PER_SYSTEM && sort_path != NVAMD_NL_SORT_GLOBAL)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl: unknown sort_path %d", (int)sort_path);
    if (n_atoms < 0 || n_systems < 0 || max_neighbors < 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl: negative size");
    if (!(cutoff > 0.0)) return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl: cutoff must be positive");
    if (n_atoms == 0 || n_systems == 0) return NVAMD_OK;
    if ((!positions && !positions64) || !batch_ptr || !batch_idx || !num_neighbors ||
        (max_neighbors > 0 && !neighbor_matrix))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl: null buffer");
    const bool has_cell = cell != nullptr || cell64 != nullptr;
    if (has_cell != (pbc != nullptr))
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl: cell and pbc must be given together");
    if (has_cell && !neighbor_matrix_shifts && max_neighbors > 0)
        return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl: periodic build needs neighbor_matrix_shifts");
    size_t need = carve(nullptr, nullptr, n_atoms, n_systems);
    if (!workspace || workspace_bytes < need)
        return fail(NVAMD_ERR_WORKSPACE_TOO_SMALL, "nl: workspace %zu < %zu bytes", workspace_bytes, need);
    if (max_cells_for(n_atoms, n_systems) > 0x7fffffffull)
        return fail(NVAMD_ERR_UNSUPPORTED, "nl: too many cells");
    if (shift_groups && (!positions || tail_mode))
        return fail(NVAMD_ERR_UNSUPPORTED,
                    "nl: shift_groups go with float32 positions and tail_mode 0 (buffers that only this function writes)");
    if (tile_index) {
        if (!ordered_positions || !tile_records || !tile_count)
            return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl: the tile outputs come together");
        if (!positions || half_fill || rebuild_flags || max_neighbors % 8 != 0)
            return fail(NVAMD_ERR_UNSUPPORTED,
                        "nl: tiles are written for float32 positions, a full list, a build of every system and "
                        "max_neighbors a multiple of 8");
    }

    NlWorkspace ws;
    carve(&ws, static_cast<char*>(workspace), n_atoms, n_systems);
    NlArgs a;
    a.pos = positions;
    a.cell = cell;
    a.pos64 = positions64;
    a.cell64 = cell64;
    a.pbc = pbc;
    a.ptr = batch_ptr;
    a.bidx = batch_idx;
    a.rebuild = rebuild_flags;
    a.n_atoms = n_atoms;
    a.n_systems = n_systems;
    a.K = max_neighbors;
    a.half = half_fill ? 1 : 0;
    a.tail_mode = tail_mode ? 1 : 0;
    a.unit_group = 1;
    while (a.unit_group < 64 && (long long)a.unit_group * 8192 <= (long long)n_atoms) a.unit_group *= 2;
    // A small batch does not fill the chip with units of kCenterChunk centre atoms: smaller units
    a.center_chunk = NVAMD_NL_CHUNK(n_atoms);
    a.tile_index = tile_index;
    a.tile_xyz = reinterpret_cast<float4*>(ordered_positions);
    a.tile_records = reinterpret_cast<int2*>(tile_records);
    a.tile_count = tile_count;
    // (no shifts, nothing to keep track of)
    a.shift_groups = neighbor_matrix_shifts ? shift_groups : nullptr;
    a.group_shift = 0;
    while ((max_neighbors - 1) >> a.group_shift > 31) ++a.group_shift;
    a.rc = cutoff;
    a.rc2 = cutoff * cutoff;
    a.rcb = cutoff * (1.0 + 1.0 / 1024.0);
    a.nm = neighbor_matrix;
    a.nn = num_neighbors;
    a.shifts = neighbor_matrix_shifts;

    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 blk(kBlock);
    auto blocks = [](size_t n) { return dim3((unsigned)((n + kBlock - 1) / kBlock)); };
    const bool per_system = sort_path == NVAMD_NL_SORT_AUTO ? (n_atoms / n_systems <= kPerSystemMeanAtoms)
                                                            : (sort_path == NVAMD_NL_SORT_PER_SYSTEM);
    if (per_system) {
        // many small systems: set-up to scatter in one workgroup per system
        if (!a.pos64 && n_atoms / n_systems > 4 * kSortBlock && n_atoms / n_systems <= 8 * kSortBlock)
            hipLaunchKernelGGL((nl_system_sort_kernel<8, 2>), dim3(n_systems), dim3(kSortBlock), 0, st, a, ws);
        else if (n_systems > 256)
            hipLaunchKernelGGL((nl_system_sort_kernel<4, 4>), dim3(n_systems), dim3(kSortBlock), 0, st, a, ws);
        else
            hipLaunchKernelGGL((nl_system_sort_kernel<4, 2>), dim3(n_systems), dim3(kSortBlock), 0, st, a, ws);
    } else {
        size_t n_prep = (size_t)ws.max_cells > (size_t)n_systems ? (size_t)ws.max_cells : (size_t)n_systems;
        hipLaunchKernelGGL(nl_prepare_kernel, blocks(n_prep), blk, 0, st, a, ws);
        hipLaunchKernelGGL(nl_bounds_kernel, blocks(n_atoms), blk, 0, st, a, ws);
        hipLaunchKernelGGL(nl_grid_kernel, dim3(1), dim3(1024), 0, st, a, ws);
        hipLaunchKernelGGL(nl_bin_kernel, blocks(n_prep > (size_t)n_atoms ? n_prep : (size_t)n_atoms), blk, 0, st, a, ws);
        scan::exclusive(scan::LoadArray{ws.cell_count}, &ws.hdr->total_cells, 0, ws.n_scan_blocks,
                        ws.block_sums, ws.cell_start, st);
        hipLaunchKernelGGL(nl_scatter_kernel, blocks(n_atoms), blk, 0, st, a, ws);
    }
    // one workgroup per cell; the grid is a fixed size (the cell count lives on the device)
    // and strides over the cells
    unsigned n_search = 8u * 2048u;
    size_t cells_bound = max_cells_for(n_atoms, n_systems);
    if (cells_bound < n_search) n_search = (unsigned)((cells_bound + 7) / 8 * 8);
#define NVAMD_NL_SEARCH(H, D, T, S) \
    hipLaunchKernelGGL((nl_search_kernel<H, D, T, S>), dim3(n_search), blk, 0, st, a, ws, ws.units, ws.ssys, ws.cell_start)
    if (a.tile_index) {
        if (a.shift_groups) NVAMD_NL_SEARCH(false, false, true, true);
        else NVAMD_NL_SEARCH(false, false, true, false);
    } else if (a.shift_groups) {
        if (a.half) NVAMD_NL_SEARCH(true, false, false, true);
        else NVAMD_NL_SEARCH(false, false, false, true);
    } else if (a.pos64) {
        if (a.half) NVAMD_NL_SEARCH(true, true, false, false);
        else NVAMD_NL_SEARCH(false, true, false, false);
    } else {
        if (a.half) NVAMD_NL_SEARCH(true, false, false, false);
        else NVAMD_NL_SEARCH(false, false, false, false);
    }
#undef NVAMD_NL_SEARCH
    NVAMD_LAUNCH_CHECK("neighbor list launch");
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_build_path(const float* positions, const float* cell, const uint8_t* pbc,
                                         const int32_t* batch_ptr, const int32_t* batch_idx,
                                         const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                                         double cutoff, int32_t max_neighbors, int32_t half_fill,
                                         int32_t tail_mode, int32_t sort_path, int32_t* neighbor_matrix,
                                         int32_t* num_neighbors, int32_t* neighbor_matrix_shifts, void* workspace,
                                         size_t workspace_bytes, void* stream) {
    return nl_build_impl(positions, cell, nullptr, nullptr, pbc, batch_ptr, batch_idx, rebuild_flags, n_atoms, n_systems,
                         cutoff, max_neighbors, half_fill, tail_mode, sort_path, neighbor_matrix, num_neighbors,
                         neighbor_matrix_shifts, workspace, workspace_bytes, stream);
}

NVAMD_EXPORT int32_t nvamd_nl_build_extras(const float* positions, const float* cell, const uint8_t* pbc,
                                           const int32_t* batch_ptr, const int32_t* batch_idx,
                                           const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                                           double cutoff, int32_t max_neighbors, int32_t half_fill, int32_t tail_mode,
                                           int32_t sort_path, int32_t* neighbor_matrix, int32_t* num_neighbors,
                                           int32_t* neighbor_matrix_shifts, uint16_t* tile_index,
                                           float* ordered_positions, int32_t* tile_records, int32_t* tile_count,
                                           uint32_t* shift_groups, void* workspace, size_t workspace_bytes,
                                           void* stream) {
    const int given = (tile_index ? 1 : 0) + (ordered_positions ? 1 : 0) + (tile_records ? 1 : 0) + (tile_count ? 1 : 0);
    if (given != 0 && given != 4) return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl: the four tile outputs come together");
    return nl_build_impl(positions, cell, nullptr, nullptr, pbc, batch_ptr, batch_idx, rebuild_flags, n_atoms, n_systems,
                         cutoff, max_neighbors, half_fill, tail_mode, sort_path, neighbor_matrix, num_neighbors,
                         neighbor_matrix_shifts, workspace, workspace_bytes, stream, tile_index, ordered_positions,
                         tile_records, tile_count, shift_groups);
}

NVAMD_EXPORT int32_t nvamd_nl_tile_records(int32_t n_atoms, int32_t n_systems, size_t* records) {
    if (!records || n_atoms < 0 || n_systems < 0) return fail(NVAMD_ERR_INVALID_ARGUMENT, "nl tile records: bad argument");
    *records = max_cells_for(n_atoms, n_systems);
    return NVAMD_OK;
}

NVAMD_EXPORT int32_t nvamd_nl_build_f64(const double* positions, const double* cell, const uint8_t* pbc,
                                        const int32_t* batch_ptr, const int32_t* batch_idx,
                                        const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                                        double cutoff, int32_t max_neighbors, int32_t half_fill,
                                        int32_t tail_mode, int32_t sort_path, int32_t* neighbor_matrix,
                                        int32_t* num_neighbors, int32_t* neighbor_matrix_shifts, void* workspace,
                                        size_t workspace_bytes, void* stream) {
    return nl_build_impl(nullptr, nullptr, positions, cell, pbc, batch_ptr, batch_idx, rebuild_flags, n_atoms, n_systems,
                         cutoff, max_neighbors, half_fill, tail_mode, sort_path, neighbor_matrix, num_neighbors,
                         neighbor_matrix_shifts, workspace, workspace_bytes, stream);
}
