/*
 * nvalchemi_amd.h -- C ABI of the MI355X (gfx950) batched-MD inner loop.
 *
 * One shared library, libnvalchemi_amd.so, exports these entry points.  They are what the
 * reference's Python binds for this path: the reference reaches its kernels through
 * torch custom ops and plain calls into an ops wheel; each declaration cites the reference
 * interface it replaces.  All pointers are DEVICE pointers unless stated otherwise; every
 * buffer is allocated and owned by the caller; outputs are written in place; work is
 * enqueued on `stream` (a hipStream_t, NULL = the default stream) and no entry point
 * synchronises.  Every function returns NVAMD_OK or an error code; nvamd_last_error()
 * holds a message for the calling thread.  Nothing throws across this boundary.
 *
 * Layouts (reference: nvalchemi/neighbors.py:239-266, nvalchemi/models/_ops/lj.py:135-151):
 *   positions (N,3) f32 | cell (B,3,3) f32, rows = lattice vectors | pbc (B,3) u8 (bool)
 *   batch_ptr (B+1) i32 | batch_idx (N) i32, non-decreasing
 *   neighbor_matrix (N,K) i32 padded with N | num_neighbors (N) i32
 *   neighbor_matrix_shifts (N,K,3) i32, zero in the padding
 * Pair geometry: r_ij = r_j - r_i + S . cell ; neighbor iff |r_ij|^2 < cutoff^2 (strict),
 * evaluated in double on the float32 inputs.
 */
#ifndef NVALCHEMI_AMD_H
#define NVALCHEMI_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NVAMD_OK 0
#define NVAMD_ERR_INVALID_ARGUMENT 1
#define NVAMD_ERR_WORKSPACE_TOO_SMALL 2
#define NVAMD_ERR_HIP 3
#define NVAMD_ERR_UNSUPPORTED 4

#define NVAMD_ABI_VERSION 1

/* Library identification and the last error message of the calling thread. */
int32_t nvamd_abi_version(void);
const char* nvamd_last_error(void);

/* ------------------------------------------------------------------------------------------
 * Neighbor list.  Replaces nvalchemiops.torch.neighbors.neighbor_list(...) as called at
 * nvalchemi/neighbors.py:253-266 and nvalchemi/hooks/neighbor_list.py:328-343, together with
 * its scratch allocators (allocate_cell_list / estimate_batch_cell_list_sizes,
 * nvalchemi/hooks/neighbor_list.py:682-704) and the hook's stale-slot masking (:377-380).
 *
 * nvamd_nl_workspace_bytes: size of the scratch buffer nvamd_nl_build needs for at most
 *   n_atoms atoms in n_systems systems (host-only computation, no device access).
 *
 * nvamd_nl_build:
 *   cell, pbc            NULL together = non-periodic (positions are never wrapped).
 *   rebuild_flags        (B) u8 or NULL; systems with 0 keep their rows and counts.
 *   max_neighbors        K.  Counting continues past K, nothing is written past K; the
 *                        caller treats max(num_neighbors) >= K as overflow and retries.
 *   half_fill            0 = both directions; 1 = each pair once (i<j; self images by the
 *                        lexicographically positive shift).
 *   tail_mode            what to do with slots k >= num_neighbors[i] of a rebuilt row:
 *                        0 = trust that slots beyond the PREVIOUS count already hold the
 *                            padding (reset only [new, old)); valid for buffers that were
 *                            prefilled once and are only ever written by this function;
 *                        1 = write the padding over the whole tail [new, K).
 *                        num_neighbors must hold the previous counts (zeros at first use).
 *   neighbor_matrix_shifts may be NULL when cell is NULL.
 * ---------------------------------------------------------------------------------------- */
/* The workspace: device memory of at least this many bytes whose first 256 bytes (the header) are ZERO when it is
 * first used (hipMemsetAsync of 256 bytes, once).  The header keeps the unit counter and the status bits of a build
 * in one of two slots, taken in turn, and every build clears the slot of the build before it (no reset launch), so
 * builds through one workspace must not overlap; apart from the header nothing in it outlives a call except what
 * nvamd_nl_atom_order and nvamd_nl_status read. */
int32_t nvamd_nl_workspace_bytes(int32_t n_atoms, int32_t n_systems, size_t* bytes);

int32_t nvamd_nl_build(const float* positions, const float* cell, const uint8_t* pbc,
                       const int32_t* batch_ptr, const int32_t* batch_idx,
                       const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                       double cutoff, int32_t max_neighbors, int32_t half_fill,
                       int32_t tail_mode, int32_t* neighbor_matrix, int32_t* num_neighbors,
                       int32_t* neighbor_matrix_shifts, void* workspace, size_t workspace_bytes,
                       void* stream);

/* nvamd_nl_build with the way the atoms are brought into cell order chosen by the caller instead
 * of by the library (no counterpart in the reference; the lists are the same sets either way):
 *   NVAMD_NL_SORT_AUTO        what nvamd_nl_build does: per system up to 8192 atoms per system
 *                             on average, global above
 *   NVAMD_NL_SORT_PER_SYSTEM  one workgroup sorts one system (batches of many small systems)
 *   NVAMD_NL_SORT_GLOBAL      one counting sort over all atoms (few, large systems)
 * Either path handles any input; the choice only matters for speed.  The tests use it to run
 * every case on both. */
#define NVAMD_NL_SORT_AUTO 0
#define NVAMD_NL_SORT_PER_SYSTEM 1
#define NVAMD_NL_SORT_GLOBAL 2
int32_t nvamd_nl_build_path(const float* positions, const float* cell, const uint8_t* pbc,
                            const int32_t* batch_ptr, const int32_t* batch_idx,
                            const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                            double cutoff, int32_t max_neighbors, int32_t half_fill,
                            int32_t tail_mode, int32_t sort_path, int32_t* neighbor_matrix,
                            int32_t* num_neighbors, int32_t* neighbor_matrix_shifts, void* workspace,
                            size_t workspace_bytes, void* stream);

/* Dense -> COO compaction in row-major order (atom ascending, slot ascending).  Replaces
 * nvalchemiops.torch.neighbors.neighbor_utils.get_neighbor_list_from_neighbor_matrix as
 * called at nvalchemi/neighbors.py:92-103, in two steps so the caller can size the output:
 *   nvamd_nl_edge_ptr       edge_ptr (N+1) i32 = exclusive scan of min(num_neighbors, K);
 *                           edge_ptr[N] = E.  workspace: nvamd_coo_workspace_bytes(n_atoms).
 *   nvamd_nl_matrix_to_coo  neighbor_list (E_cap,2) i32 rows [i, j]; neighbor_list_shifts
 *                           (E_cap,3) i32 or NULL; edges at or beyond E_cap are not written.
 */
int32_t nvamd_coo_workspace_bytes(int32_t n_atoms, size_t* bytes);
int32_t nvamd_nl_edge_ptr(const int32_t* num_neighbors, int32_t n_atoms, int32_t max_neighbors,
                          int32_t* edge_ptr, void* workspace, size_t workspace_bytes,
                          void* stream);
int32_t nvamd_nl_matrix_to_coo(const int32_t* neighbor_matrix,
                               const int32_t* neighbor_matrix_shifts, const int32_t* edge_ptr,
                               int32_t n_atoms, int32_t max_neighbors, int64_t edge_capacity,
                               int32_t* neighbor_list, int32_t* neighbor_list_shifts,
                               void* stream);
/* Both steps in one call, for callers that bring buffers of a capacity of their choice and do not want to
 * wait for the edge count in between (the same call site, nvalchemi/neighbors.py:92-103): the edge pointer
 * is scanned on the device, edges below edge_capacity are written, and counts (2) i32 on the device receives
 * the number of edges E and 1 if E exceeds edge_capacity (then the caller grows its buffers and calls again;
 * the overflow protocol of the matrix build, for edges).  No host synchronisation.
 * workspace: nvamd_coo_workspace_bytes(n_atoms). */
int32_t nvamd_nl_coo_from_matrix(const int32_t* neighbor_matrix, const int32_t* neighbor_matrix_shifts,
                                 const int32_t* num_neighbors, int32_t n_atoms, int32_t max_neighbors,
                                 int64_t edge_capacity, int32_t* edge_ptr, int32_t* neighbor_list,
                                 int32_t* neighbor_list_shifts, int32_t* counts, void* workspace,
                                 size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Lennard-Jones pair kernel over the neighbor matrix.  Replaces the Warp launches inside
 * nvalchemi::lj_energy_forces_batch and nvalchemi::lj_energy_forces_virial_batch
 * (nvalchemi/models/_ops/lj.py:116-216, 246-321) and fuses the per-system fp64 energy
 * scatter of nvalchemi/models/lj.py:467-477.
 *   neighbor_matrix_shifts NULL = all shifts zero.
 *   atomic_energies (N) f32, forces (N,3) f32: overwritten.
 *   virials (B,9) f32 or NULL: W = -sum r_ij (x) F_ij, row-major, overwritten.
 *   system_energies (B) f32 or NULL: fp64 sum of the float32 atomic energies, overwritten.
 *   switch_width in [0, cutoff]: 0 is plain truncation; otherwise the pair energy is multiplied by
 *     S(t) = 1 - t^3 (10 - 15 t + 6 t^2), t = (r - (cutoff - switch_width)) / switch_width, between
 *     cutoff - switch_width and cutoff (the least-degree polynomial that keeps energy, force and force
 *     gradient continuous; the reference's own polynomial is inside its absent kernel library).
 *   workspace: nvamd_lj_workspace_bytes(n_atoms, n_systems, half_list); always required.
 * ---------------------------------------------------------------------------------------- */
int32_t nvamd_lj_workspace_bytes(int32_t n_atoms, int32_t n_systems, int32_t half_list,
                                 size_t* bytes);

int32_t nvamd_lj_energy_forces(const float* positions, const float* cells,
                               const int32_t* neighbor_matrix,
                               const int32_t* neighbor_matrix_shifts,
                               const int32_t* num_neighbors, const int32_t* batch_idx,
                               int32_t n_atoms, int32_t max_neighbors, int32_t n_systems,
                               int32_t fill_value, double epsilon, double sigma, double cutoff,
                               double switch_width, int32_t half_list, float* atomic_energies,
                               float* forces, float* virials, float* system_energies,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Velocity Verlet halves.  Replace nvalchemi::vv_position_update and
 * nvalchemi::vv_velocity_finalize (nvalchemi/dynamics/_ops/velocity_verlet.py:50-92,102-138).
 *   dt (M) f32 per system; `active` (M) u8 or NULL: systems with 0 are left untouched (the
 *   in-kernel form of the save/restore masking of nvalchemi/dynamics/base.py:1849-1891).
 * ---------------------------------------------------------------------------------------- */
int32_t nvamd_vv_position_update(float* positions, float* velocities, const float* forces,
                                 const float* masses, const float* dt, const int32_t* batch_idx,
                                 const uint8_t* active, int32_t n_atoms, int32_t n_systems,
                                 void* stream);

int32_t nvamd_vv_velocity_finalize(float* velocities, const float* forces_new,
                                   const float* masses, const float* dt,
                                   const int32_t* batch_idx, const uint8_t* active,
                                   int32_t n_atoms, int32_t n_systems, void* stream);

/* nvamd_vv_velocity_finalize followed by nvamd_vv_position_update with the same forces, in one launch: the closing
 * half kick of one step and the opening half kick and drift of the next, which the reference launches back to back
 * when nothing is registered between two steps (nvalchemi/dynamics/base.py:1875-1883 for consecutive steps).  No
 * counterpart in the reference; the results are those of the two calls in a row, bit for bit (the same operations
 * in the same order per element).  float32 only. */
int32_t nvamd_vv_finalize_then_update(float* positions, float* velocities, const float* forces,
                                      const float* masses, const float* dt, const int32_t* batch_idx,
                                      const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* stream);

/* ------------------------------------------------------------------------------------------
 * FIRE step.  Replaces nvalchemi::_fire_step_op (nvalchemi/dynamics/_ops/fire.py:79-140).
 *   All per-system arrays have M entries; alpha, dt, n_steps_positive, vf, vv, ff and
 *   positions, velocities are updated.  compute_reductions = 0 consumes vf/vv/ff as given.
 *   Order (nvalchemi/dynamics/_ops/fire.py:270-272): reductions over the arrays as passed in,
 *   then the MD integration with the stored dt (kick, drift limited to maxstep per atom), then
 *   the mixing with the stored alpha (sum F.v >= 0) or the reset of the velocities (< 0),
 *   then the update of dt, alpha and n_steps_positive.
 *   Only the vanilla branch exists.  uphill_flag is a device array, so the library cannot look
 *   at it without a synchronisation and does not: the caller must pass zeros (the Python
 *   wrapper checks and raises for anything else).  `active` as above.
 *   workspace: nvamd_fire_workspace_bytes(n_systems), all ZERO when it is first used (hipMemsetAsync once): the
 *   sums live in two slots taken in turn from call to call, each call clears the slot of the next one, so the
 *   step is two launches (sums, update); calls through one workspace must not overlap and must all have the same
 *   n_systems (zero it again before a call with another n_systems).
 * ---------------------------------------------------------------------------------------- */
int32_t nvamd_fire_workspace_bytes(int32_t n_systems, size_t* bytes);

int32_t nvamd_fire_step(float* positions, float* velocities, const float* forces,
                        const float* masses, float* alpha, float* dt, const float* alpha_start,
                        const float* f_alpha, const float* dt_min, const float* dt_max,
                        const float* maxstep, int32_t* n_steps_positive, const int32_t* n_min,
                        const float* f_dec, const float* f_inc, const int32_t* uphill_flag,
                        float* vf, float* vv, float* ff, const int32_t* batch_idx,
                        int32_t compute_reductions, const uint8_t* active, int32_t n_atoms,
                        int32_t n_systems, void* workspace, size_t workspace_bytes,
                        void* stream);

/* One FIRE 2.0 step on the forces of the current positions: replaces the call into the kernel library
 * behind fire2_step_coord (nvalchemi/dynamics/_ops/fire.py:467-557; called from
 * nvalchemi/dynamics/optimizers/fire2.py:218-251).  positions, velocities (N,3), alpha, dt (M) f32 and
 * nsteps_inc (M) i32 are updated in place; vf, v_sumsq, f_sumsq (sum F.v, v.v, F.F per system) and
 * max_norm (the largest atomic displacement the step would make before the maxstep limit) are outputs
 * and may be NULL; the hyper-parameters are scalars as in the reference.  Unit masses (the reference's
 * op takes none).  active (M) bytes or NULL as for velocity Verlet.  The algorithm is FIRE 2.0 as
 * published with its LAMMPS implementation (Guenole et al. 2020): semi-implicit Euler, half step back
 * on a reset.  Workspace: nvamd_fire2_workspace_bytes(n_systems). */
int32_t nvamd_fire2_workspace_bytes(int32_t n_systems, size_t* bytes);
int32_t nvamd_fire2_step(float* positions, float* velocities, const float* forces,
                         const int32_t* batch_idx, float* alpha, float* dt, int32_t* nsteps_inc,
                         float* vf, float* v_sumsq, float* f_sumsq, float* max_norm,
                         int32_t delaystep, double dtgrow, double dtshrink, double alphashrink,
                         double alpha0, double tmax, double tmin, double maxstep,
                         const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* workspace,
                         size_t workspace_bytes, void* stream);

/* BAOAB Langevin pre-force half step B-A-O-A: replaces the Warp launch behind
 * nvalchemi::langevin_half_step (nvalchemi/dynamics/_ops/langevin.py:52-117; called from
 * nvalchemi/dynamics/integrators/nvt_langevin.py:160-181).  kT (M) f32 in energy units,
 * friction (M) f32 in 1/time, dt (M) f32; positions and velocities updated in place; active (M)
 * bytes or NULL as for velocity Verlet.  The normal deviates of atom i are a function of
 * (random_seed, i) only (Philox4x32-10, Box-Muller): callers advance the seed every step, as the
 * reference does (random_seed + step_count).  The final B step, nvalchemi::langevin_finalize
 * (:134-170), is nvamd_vv_velocity_finalize. */
int32_t nvamd_langevin_half_step(float* positions, float* velocities, const float* forces,
                                 const float* masses, const float* dt, const float* kT,
                                 const float* friction, uint64_t random_seed, const int32_t* batch_idx,
                                 const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* stream);

/* Nose-Hoover chain thermostat, half-step propagator: replaces the Warp launch behind
 * nvalchemi::nhc_chain_update (nvalchemi/dynamics/_ops/nose_hoover.py:143-246; called before and
 * after the velocity-Verlet core of a step, nvalchemi/dynamics/integrators/nvt_nose_hoover.py:215-281).
 * Per system: eta, eta_dot, chain_masses (M, chain_length) f32 row-major; kT (energy units), dt,
 * ndof (M) f32; ke2 (M) f32 receives sum m v^2 (compute_ke != 0) or supplies it (compute_ke == 0, for a
 * caller that holds the sum over more atoms than it passes); total_scale (M) f32 receives the factor
 * the velocities were multiplied by.  velocities, eta, eta_dot are updated in place; active (M) bytes
 * or NULL as for velocity Verlet.  chain_length 1..16; yoshida_order 1, 3 or 5 (the reference's
 * integrator takes 3 or 5 and defaults to 3).  The propagator is the one of Martyna, Tuckerman, Tobias
 * and Klein (1996) with one pass of the Suzuki-Yoshida weights; chain arithmetic in double.
 * Workspace: nvamd_nhc_workspace_bytes(n_systems). */
int32_t nvamd_nhc_workspace_bytes(int32_t n_systems, size_t* bytes);
int32_t nvamd_nhc_chain_update(float* velocities, const float* masses, float* eta, float* eta_dot,
                               const float* chain_masses, const float* kT, const float* dt,
                               const float* ndof, float* ke2, float* total_scale,
                               const int32_t* batch_idx, const uint8_t* active, int32_t compute_ke,
                               int32_t chain_length, int32_t yoshida_order, int32_t n_atoms,
                               int32_t n_systems, void* workspace, size_t workspace_bytes, void* stream);

/* r += v dt with the system's dt: replaces the Warp launch behind nvalchemi::nhc_position_update
 * (nvalchemi/dynamics/_ops/nose_hoover.py:291-325).  The third op of that integrator,
 * nvalchemi::nhc_velocity_half_step (:248-289), v += (F/m) dt/2, is nvamd_vv_velocity_finalize. */
int32_t nvamd_nhc_position_update(float* positions, const float* velocities, const float* dt,
                                  const int32_t* batch_idx, const uint8_t* active, int32_t n_atoms,
                                  int32_t n_systems, void* stream);

/* What ConvergenceHook does with the result of its criterion (nvalchemi/dynamics/base.py:2459-2502: systems
 * that are converged and whose status equals source_status get target_status), for a criterion of the form
 * value <= threshold: status[s] = target_status where values[s] <= threshold and status[s] == source_status, in
 * one launch instead of the reference's six Torch kernels and its host read of migrate.any().  values (M) f32 (for
 * the default criterion: the output of nvamd_segment_fmax), status (M) i64 contiguous, updated in place.  The
 * threshold is compared in the values' type, as Torch compares a tensor with a Python float; a NaN is not
 * converged.  nvamd_status_migrate_f64 takes double values. */
int32_t nvamd_status_migrate(const float* values, double threshold, int64_t* status, int64_t source_status,
                             int64_t target_status, int32_t n_systems, void* stream);
int32_t nvamd_status_migrate_f64(const double* values, double threshold, int64_t* status, int64_t source_status,
                                 int64_t target_status, int32_t n_systems, void* stream);

/* Per-system maximum atomic force norm (the default convergence criterion,
 * nvalchemi/dynamics/base.py:258-349: vector_norm over xyz, scatter amax over atoms).
 * fmax (M) f32; systems without atoms give -inf. */
int32_t nvamd_segment_fmax(const float* forces, const int32_t* batch_idx, int32_t n_atoms,
                           int32_t n_systems, float* fmax, void* stream);

/* The same, with two optional hints; results do not depend on either.  No counterpart in the reference.
 * row_order (N) i32 or null: a permutation of 0..N-1 in which the atoms of each system stay together and in
 *   system order (e.g. the cell order of the last neighbor build, nvamd_nl_atom_order); the kernel walks its
 *   rows in it.  For systems too large to stage in LDS, an order with spatial locality keeps the gathers of
 *   neighbor positions in the caches.
 * neighbor_list_cutoff: the cutoff (skin included) that the neighbor matrix was built with, or 0 if unknown.
 *   Every listed pair is then closer than that; in a system whose cell has all three perpendicular widths
 *   above twice it, no pair has two listed images, the listed image is the nearest one, and the kernel
 *   derives the shift from the positions instead of reading neighbor_matrix_shifts (12 of the 16 bytes per
 *   pair).  With a cutoff given, the matrix is taken to be what nvamd_nl_build wrote: in such a system the
 *   entries below a row's count are not checked one by one for being atoms of the row's own system (reads
 *   stay inside the arrays whatever the entries hold).  A matrix that holds pairs beyond this cutoff, or
 *   entries of other systems or padding below the counts, makes the results wrong: pass 0 when in doubt. */
int32_t nvamd_lj_energy_forces_hinted(const float* positions, const float* cells,
                                      const int32_t* neighbor_matrix,
                                      const int32_t* neighbor_matrix_shifts,
                                      const int32_t* num_neighbors, const int32_t* batch_idx,
                                      const int32_t* row_order, double neighbor_list_cutoff, int32_t n_atoms,
                                      int32_t max_neighbors, int32_t n_systems, int32_t fill_value,
                                      double epsilon, double sigma, double cutoff, double switch_width,
                                      int32_t half_list, float* atomic_energies, float* forces, float* virials,
                                      float* system_energies, void* workspace, size_t workspace_bytes,
                                      void* stream);

/* nvamd_lj_energy_forces_hinted (full list) for a caller that evaluates the same batch again and again (an MD
 * loop).  No counterpart in the reference.  The pair kernel's per-system tables in the workspace (first and
 * last atom of each system, how the images of its pairs are found) depend on batch_idx, cells,
 * neighbor_list_cutoff, n_atoms and n_systems only.  reuse_tables = 0: they are computed, as the other entry
 * points do on every call.  reuse_tables = 1: the caller promises that nothing else has written the workspace
 * since the previous call of this library's pair kernel through it, that this previous call had the same
 * batch_idx, cells (contents included), neighbor_list_cutoff, n_atoms, n_systems and the same choice of
 * virials / system_energies outputs, and was a full-list call: the tables are used as they stand, one launch
 * fewer.  (Every full-list call leaves the workspace's accumulators at zero for the next one.) */
int32_t nvamd_lj_energy_forces_repeat(const float* positions, const float* cells,
                                      const int32_t* neighbor_matrix,
                                      const int32_t* neighbor_matrix_shifts,
                                      const int32_t* num_neighbors, const int32_t* batch_idx,
                                      const int32_t* row_order, double neighbor_list_cutoff, int32_t n_atoms,
                                      int32_t max_neighbors, int32_t n_systems, int32_t fill_value,
                                      double epsilon, double sigma, double cutoff, double switch_width,
                                      int32_t reuse_tables, float* atomic_energies, float* forces, float* virials,
                                      float* system_energies, void* workspace, size_t workspace_bytes,
                                      void* stream);

/* nvamd_lj_energy_forces_repeat over the tiles of nvamd_nl_build_extras, for the positions that build read.  No
 * counterpart in the reference.  The rows are walked unit by unit of the build's search; a unit's tile (the atoms
 * of its stencil cells, a few hundred) is copied from ordered_positions into LDS with contiguous reads, laid out
 * by the unit's record, and each listed pair finds its neighbor there through its 16-bit tile_index: no gather from
 * memory per pair, and two bytes read per pair instead of four.  Meant for systems too large for the other entry
 * points to stage whole (more than 4096 atoms).  Images are derived from the positions, so neighbor_list_cutoff
 * must be the build's cutoff and every cell wider than twice that (systems where it is not, and units without a
 * tile, take their neighbors from memory as the other entry points do).  Full list, no switching.
 * neighbor_matrix / num_neighbors / row_order are those of the same build.  Results are those of the other entry
 * points, bit for bit. */
int32_t nvamd_lj_energy_forces_tiles(const float* positions, const float* cells,
                                     const int32_t* neighbor_matrix,
                                     const int32_t* neighbor_matrix_shifts,
                                     const int32_t* num_neighbors, const int32_t* batch_idx,
                                     const int32_t* row_order, const uint16_t* tile_index,
                                     const float* ordered_positions, const int32_t* tile_records,
                                     const int32_t* tile_count, double neighbor_list_cutoff, int32_t n_atoms,
                                     int32_t max_neighbors, int32_t n_systems, int32_t fill_value, double epsilon,
                                     double sigma, double cutoff, int32_t reuse_tables, float* atomic_energies,
                                     float* forces, float* virials, float* system_energies, void* workspace,
                                     size_t workspace_bytes, void* stream);

/* nvamd_lj_energy_forces_hinted for callers that cannot allocate device memory or carry a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in
 * the reference.  The scratch of the pair kernel (per-system float64 accumulators, first and last atom of
 * each system) lives in a device array built into the library, NVAMD_LJ_STATIC_SCRATCH_BYTES per GPU,
 * held until the process ends; the call allocates and frees nothing.  Limits: full list only (there is
 * no half_list argument), n_systems <= NVAMD_LJ_STATIC_MAX_SYSTEMS (more returns NVAMD_ERR_UNSUPPORTED);
 * n_atoms is not limited.  The first call on a device looks up the array's address
 * (hipGetSymbolAddress): make it outside a graph capture.  All calls on one GPU share the one array:
 * calls that overlap on a GPU (two streams, two threads) race; what has to start at zero is cleared
 * by every call.  Results are those of nvamd_lj_energy_forces_hinted. */
#define NVAMD_LJ_STATIC_MAX_SYSTEMS 16384
#define NVAMD_LJ_STATIC_SCRATCH_BYTES \
    ((((size_t)NVAMD_LJ_STATIC_MAX_SYSTEMS * 80 + 255) / 256 + 2 * (((size_t)NVAMD_LJ_STATIC_MAX_SYSTEMS * 4 + 255) / 256) + \
      ((size_t)NVAMD_LJ_STATIC_MAX_SYSTEMS * 96 + 255) / 256) * 256)
int32_t nvamd_lj_energy_forces_static(const float* positions, const float* cells,
                                      const int32_t* neighbor_matrix,
                                      const int32_t* neighbor_matrix_shifts,
                                      const int32_t* num_neighbors, const int32_t* batch_idx,
                                      const int32_t* row_order, double neighbor_list_cutoff, int32_t n_atoms,
                                      int32_t max_neighbors, int32_t n_systems, int32_t fill_value,
                                      double epsilon, double sigma, double cutoff, double switch_width,
                                      float* atomic_energies, float* forces, float* virials,
                                      float* system_energies, void* stream);

/* ------------------------------------------------------------------------------------------
 * float64 forms.  The reference's ops take float32 or float64 arrays (nvalchemi/dynamics/_ops/_bridge.py
 * _vec_type / _scalar_type; nvalchemi/dynamics/_ops/fire.py:281-287; nvalchemi/models/_ops/lj.py:116-216).
 * Same arguments, meaning and order of operations as the float32 entry points above, with every float
 * array a double array (cells included; per-system parameters too).  The neighbor decision is made in
 * double on the float64 positions.  The pair kernel's per-system energy is the sum of the float64 atomic
 * energies.  nvamd_f64_workspace_bytes(n_systems) serves nvamd_fire_step_f64, nvamd_segment_fmax_f64 and
 * nvamd_lj_energy_forces_f64 (which needs it only with virials or system_energies); the neighbor build uses
 * nvamd_nl_workspace_bytes.  nvamd_fire2_step_f64 also takes nvamd_f64_workspace_bytes(n_systems);
 * nvamd_nhc_chain_update_f64 takes nvamd_nhc_workspace_bytes(n_systems) like its float32 form.  The Langevin
 * step draws the same normal deviates for both types (a function of the seed and the atom index, made in double).
 * ---------------------------------------------------------------------------------------- */
int32_t nvamd_nl_build_f64(const double* positions, const double* cell, const uint8_t* pbc,
                           const int32_t* batch_ptr, const int32_t* batch_idx, const uint8_t* rebuild_flags,
                           int32_t n_atoms, int32_t n_systems, double cutoff, int32_t max_neighbors,
                           int32_t half_fill, int32_t tail_mode, int32_t sort_path, int32_t* neighbor_matrix,
                           int32_t* num_neighbors, int32_t* neighbor_matrix_shifts, void* workspace,
                           size_t workspace_bytes, void* stream);
int32_t nvamd_f64_workspace_bytes(int32_t n_systems, size_t* bytes);
int32_t nvamd_lj_energy_forces_f64(const double* positions, const double* cells, const int32_t* neighbor_matrix,
                                   const int32_t* neighbor_matrix_shifts, const int32_t* num_neighbors,
                                   const int32_t* batch_idx, int32_t n_atoms, int32_t max_neighbors,
                                   int32_t n_systems, int32_t fill_value, double epsilon, double sigma,
                                   double cutoff, double switch_width, int32_t half_list, double* atomic_energies,
                                   double* forces, double* virials, double* system_energies, void* workspace,
                                   size_t workspace_bytes, void* stream);
int32_t nvamd_vv_position_update_f64(double* positions, double* velocities, const double* forces,
                                     const double* masses, const double* dt, const int32_t* batch_idx,
                                     const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* stream);
int32_t nvamd_vv_velocity_finalize_f64(double* velocities, const double* forces_new, const double* masses,
                                       const double* dt, const int32_t* batch_idx, const uint8_t* active,
                                       int32_t n_atoms, int32_t n_systems, void* stream);
int32_t nvamd_fire_step_f64(double* positions, double* velocities, const double* forces, const double* masses,
                            double* alpha, double* dt, const double* alpha_start, const double* f_alpha,
                            const double* dt_min, const double* dt_max, const double* maxstep,
                            int32_t* n_steps_positive, const int32_t* n_min, const double* f_dec,
                            const double* f_inc, const int32_t* uphill_flag, double* vf, double* vv, double* ff,
                            const int32_t* batch_idx, int32_t compute_reductions, const uint8_t* active,
                            int32_t n_atoms, int32_t n_systems, void* workspace, size_t workspace_bytes,
                            void* stream);
int32_t nvamd_segment_fmax_f64(const double* forces, const int32_t* batch_idx, int32_t n_atoms, int32_t n_systems,
                               double* fmax, void* workspace, size_t workspace_bytes, void* stream);
int32_t nvamd_nl_rebuild_check_f64(double* reference_positions, const double* current_positions,
                                   const int32_t* batch_idx, const double* cell, const uint8_t* pbc,
                                   int32_t n_atoms, int32_t n_systems, double threshold,
                                   int32_t update_reference, uint8_t* rebuild_flags, void* stream);
int32_t nvamd_wrap_positions_f64(double* positions, const double* cell, const uint8_t* pbc,
                                 const int32_t* batch_idx, int32_t n_atoms, int32_t n_systems, void* stream);
int32_t nvamd_fire2_step_f64(double* positions, double* velocities, const double* forces, const int32_t* batch_idx,
                             double* alpha, double* dt, int32_t* nsteps_inc, double* vf, double* v_sumsq,
                             double* f_sumsq, double* max_norm, int32_t delaystep, double dtgrow, double dtshrink,
                             double alphashrink, double alpha0, double tmax, double tmin, double maxstep,
                             const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* workspace,
                             size_t workspace_bytes, void* stream);
int32_t nvamd_langevin_half_step_f64(double* positions, double* velocities, const double* forces,
                                     const double* masses, const double* dt, const double* kT,
                                     const double* friction, uint64_t random_seed, const int32_t* batch_idx,
                                     const uint8_t* active, int32_t n_atoms, int32_t n_systems, void* stream);
int32_t nvamd_nhc_chain_update_f64(double* velocities, const double* masses, double* eta, double* eta_dot,
                                   const double* chain_masses, const double* kT, const double* dt,
                                   const double* ndof, double* ke2, double* total_scale, const int32_t* batch_idx,
                                   const uint8_t* active, int32_t compute_ke, int32_t chain_length,
                                   int32_t yoshida_order, int32_t n_atoms, int32_t n_systems, void* workspace,
                                   size_t workspace_bytes, void* stream);
int32_t nvamd_nhc_position_update_f64(double* positions, const double* velocities, const double* dt,
                                      const int32_t* batch_idx, const uint8_t* active, int32_t n_atoms,
                                      int32_t n_systems, void* stream);

/* What the neighbor builds through this workspace had to report.  No counterpart in the reference, whose
 * kernels report nothing (a caller there compares num_neighbors with max_neighbors on the host:
 * nvalchemi/neighbors.py:269-273, nvalchemi/hooks/neighbor_list.py:446-469).
 * status (2) i32 on the device: status[0] = bits of the last build, status[1] = bits of every build since the
 *   bits were last cleared.  clear != 0 clears both words after they are read.  No host synchronisation.
 * NVAMD_NL_STATUS_CELL_TOO_THIN: some periodic cell is singular or thinner than cutoff / 32 along an axis; the
 *   search looks at 32 images per axis and direction at most, so that system's list is truncated.
 * NVAMD_NL_STATUS_ROW_OVERFLOW: some atom has more than max_neighbors neighbors (its count says how many; the
 *   row holds the first max_neighbors found). */
#define NVAMD_NL_STATUS_CELL_TOO_THIN 1
#define NVAMD_NL_STATUS_ROW_OVERFLOW 2
int32_t nvamd_nl_status(void* workspace, size_t workspace_bytes, int32_t n_atoms, int32_t n_systems,
                        int32_t* status, int32_t clear, void* stream);

/* Atom indices in the cell order of the neighbor build that last used this workspace with the same
 * n_atoms / n_systems: atom_order[k] for k in a system's range [batch_ptr[s], batch_ptr[s+1]) are that
 * system's atoms, cell by cell.  With rebuild_flags, only the ranges of flagged systems are written
 * (the others were not sorted by that build).  No counterpart in the reference. */
int32_t nvamd_nl_atom_order(const void* workspace, size_t workspace_bytes, const int32_t* batch_idx,
                            const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                            int32_t* atom_order, void* stream);

/* nvamd_nl_build_path (float32 positions) with two extras, each optional.  No counterpart in the reference.
 *
 * (1) The four tile outputs (all given or all NULL): what a pair kernel needs to walk the search's own tiles again
 * (nvamd_lj_energy_forces_tiles).  The search handles the atoms of a run of cells (a "unit") against one tile: the
 * atoms of the run's stencil cells, staged in LDS in a fixed order.
 *   tile_index (N, max_neighbors) u16    per listed pair, where the neighbor stood in the tile of the row's unit
 *   ordered_positions (N, 4) f32         the atoms in cell order: float32 coordinates as read, and the bits of the
 *                                        atom's index in the fourth word
 *   tile_records (R, NVAMD_NL_TILE_RECORD_INTS) i32, R from nvamd_nl_tile_records: per unit
 *                                        [first row, rows] (slots of the cell order), [system, atoms in the tile,
 *                                        or -1: the unit's stencil is not one tile], then per stencil cell
 *                                        [its first slot of the cell order, its offset in the tile]
 *   tile_count (1) i32                   units of this build
 * Full list, every system built (no rebuild_flags), max_neighbors a multiple of 8.  A tile holds at most
 * NVAMD_NL_TILE_ATOMS atoms.  Valid for the positions of this build only.
 *
 * (2) shift_groups (N) u32 or NULL: lets the build skip the stores of shifts that are zero over zeros.  Most listed
 * pairs of a system larger than a few cutoffs have a zero shift, and three quarters of what a build writes are
 * shifts.  Bit g of an atom's word says that slots [g << s, (g + 1) << s) of its row of neighbor_matrix_shifts may
 * hold a shift that is not zero, s the smallest number with (max_neighbors - 1) >> s < 32; the build writes a
 * pair's shift if it is not zero or if its slot's bit was set, and leaves the word for the next build.  The
 * contents of neighbor_matrix_shifts come out exactly as without it.  The contract is tail_mode 0's, extended to
 * the shifts: neighbor_matrix_shifts was zeroed once together with shift_groups and is written by this function
 * only, always with the same shift_groups and max_neighbors (after anything else has written it, or after
 * max_neighbors has changed, set every word to 0xffffffff once).  tail_mode must be 0. */
#define NVAMD_NL_TILE_RECORD_INTS 132
#define NVAMD_NL_TILE_ATOMS 1088
int32_t nvamd_nl_tile_records(int32_t n_atoms, int32_t n_systems, size_t* records);
int32_t nvamd_nl_build_extras(const float* positions, const float* cell, const uint8_t* pbc,
                              const int32_t* batch_ptr, const int32_t* batch_idx,
                              const uint8_t* rebuild_flags, int32_t n_atoms, int32_t n_systems,
                              double cutoff, int32_t max_neighbors, int32_t half_fill, int32_t tail_mode,
                              int32_t sort_path, int32_t* neighbor_matrix, int32_t* num_neighbors,
                              int32_t* neighbor_matrix_shifts, uint16_t* tile_index, float* ordered_positions,
                              int32_t* tile_records, int32_t* tile_count, uint32_t* shift_groups, void* workspace,
                              size_t workspace_bytes, void* stream);

/* Per-system reductions of a per-atom float32 vector: replace the Warp launches behind
 * nvalchemi_hooks::segmented_sum / _max / _min / _mean (nvalchemi/dynamics/hooks/_utils.py:58-136;
 * scatter_reduce_per_graph :172-212).  batch_idx (n) i32 must be sorted.  op: 0 sum, 1 max, 2 min, 3 mean.
 * out (m) f32; segments without elements give 0 (sum, mean), -inf (max), +inf (min).  Sums are
 * accumulated in float64 and rounded once. */
int32_t nvamd_segment_workspace_bytes(int32_t n_segments, size_t* bytes);
int32_t nvamd_segment_reduce(const float* values, const int32_t* batch_idx, int32_t n_values,
                             int32_t n_segments, int32_t op, float* out, void* workspace,
                             size_t workspace_bytes, void* stream);

/* Kinetic energy per system, 1/2 sum m |v|^2: replaces nvalchemi_hooks::compute_kinetic_energy
 * (nvalchemi/dynamics/hooks/_utils.py:138-155; kinetic_energy_per_graph :215-243).  Workspace as for
 * nvamd_segment_reduce. */
int32_t nvamd_kinetic_energy(const float* velocities, const float* masses, const int32_t* batch_idx,
                             int32_t n_atoms, int32_t n_systems, float* kinetic_energy, void* workspace,
                             size_t workspace_bytes, void* stream);

/* Verlet-skin displacement test: replaces the Warp launch behind
 * nvalchemi::_batch_neighbor_list_rebuild_inplace (nvalchemi/dynamics/_ops/neighbor_list_rebuild.py:37-139,
 * called at nvalchemi/hooks/neighbor_list.py:295-311).  rebuild_flags (M) bool is cleared, then set for
 * every system with an atom whose displacement from reference_positions exceeds threshold (strictly);
 * with cell and pbc the displacement is taken by the minimum-image convention on the periodic axes
 * (cell and pbc both given or both null).  With update_reference != 0 the reference positions of all
 * atoms of the flagged systems are overwritten with the current ones. */
int32_t nvamd_nl_rebuild_check(float* reference_positions, const float* current_positions,
                               const int32_t* batch_idx, const float* cell, const uint8_t* pbc,
                               int32_t n_atoms, int32_t n_systems, double threshold,
                               int32_t update_reference, uint8_t* rebuild_flags, void* stream);

/* Wrap positions into the cell, in place: replaces nvalchemi_hooks::wrap_positions and the masking
 * after it (nvalchemi/hooks/periodic.py:42-114).  All three fractional coordinates are reduced to
 * [0, 1) (frac = r . inv(cell), rows of cell = lattice vectors) and mapped back; of the result, the
 * Cartesian components whose pbc flag is set replace the old ones, the others are kept (:111-113). */
int32_t nvamd_wrap_positions(float* positions, const float* cell, const uint8_t* pbc,
                             const int32_t* batch_idx, int32_t n_atoms, int32_t n_systems,
                             void* stream);

/* ------------------------------------------------------------------------------------------
 * Masked copy and in-place compaction of per-system rows and of per-system segments: replace the
 * Warp launches of nvalchemi/data/buffer_kernels.py (the data movement of Batch.put / Batch.defrag,
 * nvalchemi/data/batch.py:876-985).  Rows are opaque runs of row_bytes bytes (any dtype; source and
 * destination share it); masks are one byte per system, 0 or 1.
 * Workspace for all of them: nvamd_buffer_workspace_bytes(number of source systems, data bytes),
 * where data bytes is the size of `source` for the two defrag calls and 0 for the others.
 * ---------------------------------------------------------------------------------------- */
int32_t nvamd_buffer_workspace_bytes(int64_t n_systems, int64_t data_bytes, size_t* bytes);

/* put_masked_per_system (buffer_kernels.py:970-1079,1171-1220): of the rows with source_mask set,
 * the first min(#masked, #empty destination slots) go to consecutive destination slots starting at
 * the first empty one (dest_mask 0 = empty); dest_mask is set for the written slots and
 * source_data_copied for the moved rows (neither is cleared elsewhere). */
int32_t nvamd_put_masked_per_system(const void* source, const uint8_t* source_mask, void* dest,
                                    uint8_t* dest_mask, uint8_t* source_data_copied, int32_t num_src,
                                    int32_t num_dest, int64_t row_bytes, void* workspace,
                                    size_t workspace_bytes, void* stream);

/* compute_put_fit_mask_per_system (buffer_kernels.py:1081-1169): fit_mask[i] = the row would be
 * moved by the call above.  Nothing is copied. */
int32_t nvamd_put_fit_mask_per_system(const uint8_t* source_mask, const uint8_t* dest_mask,
                                      uint8_t* fit_mask, int32_t num_src, int32_t num_dest,
                                      void* workspace, size_t workspace_bytes, void* stream);

/* defrag_per_system (buffer_kernels.py:1222-1333): rows with source_data_copied 0 move to the
 * front in their order, the rows behind them are zeroed, and source_data_copied[i] becomes
 * (i >= number kept). */
int32_t nvamd_defrag_per_system(void* source, uint8_t* source_data_copied, int32_t num_src,
                                int64_t row_bytes, void* workspace, size_t workspace_bytes,
                                void* stream);

/* put_masked_segmented (buffer_kernels.py:1335-1527): segment i is rows
 * [source_batch_ptr[i], source_batch_ptr[i+1]).  Masked segments are laid out one after another
 * from dest_batch_ptr[num_dest_segments]; those that end at or before dest_capacity rows are
 * copied, their ends appended to dest_batch_ptr (which must hold num_dest_segments + num_systems
 * + 2 entries: one more copy of the last end follows the new ones), source_data_copied set for
 * them, and *new_num_dest = num_dest_segments + number copied.  total_rows = rows of `source`. */
int32_t nvamd_put_masked_segmented(const void* source, const int32_t* source_batch_ptr,
                                   const uint8_t* source_mask, void* dest, int32_t* dest_batch_ptr,
                                   int32_t num_dest_segments, int32_t dest_capacity,
                                   uint8_t* source_data_copied, int32_t* new_num_dest,
                                   int32_t num_systems, int32_t total_rows, int64_t row_bytes,
                                   void* workspace, size_t workspace_bytes, void* stream);

/* compute_put_fit_mask_segmented (buffer_kernels.py:500-610): fit_mask[i] = segment i would be
 * copied by the call above.  (The reference's host wrapper clears the mask instead when
 * dest_batch_ptr is too short; that check stays with the caller.) */
int32_t nvamd_put_fit_mask_segmented(const int32_t* source_batch_ptr, const uint8_t* source_mask,
                                     const int32_t* dest_batch_ptr, int32_t num_dest_segments,
                                     int32_t dest_capacity, uint8_t* fit_mask, int32_t num_systems,
                                     void* workspace, size_t workspace_bytes, void* stream);

/* defrag_segmented (buffer_kernels.py:1529-1741): segments with source_data_copied 0 move to the
 * front in their order, the rows behind them are zeroed; source_batch_ptr[0..kept] becomes the new
 * boundaries and every later entry the number of rows kept; *num_kept = segments kept.  With
 * num_systems == 0: source_batch_ptr[0] = 0 and *num_kept = 0. */
int32_t nvamd_defrag_segmented(void* source, int32_t* source_batch_ptr,
                               const uint8_t* source_data_copied, int32_t* num_kept,
                               int32_t num_systems, int32_t total_rows, int64_t row_bytes,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Filtering an existing list down to a tighter cutoff: the Torch code of
 * nvalchemi/models/_ops/neighbor_filter.py (filter_neighbor_matrix :43-144; the distance test of
 * filter_neighbor_list :147-224), used by prepare_neighbors_for_model (:286-430) when a model's
 * cutoff is below the one the list was built with.  cells: (3,3) for all atoms
 * (per_system_cells = 0) or (B,3,3) looked up through batch_idx (= 1); cells or shifts NULL: no
 * shift is applied (shifts are still carried along).  The distance is evaluated in double on the
 * float32 inputs (the reference: float32), strict <.
 * nvamd_nl_filter_matrix: every slot with an index below fill_value and inside the cutoff is kept;
 * kept entries move to the front of their row in order, the rest of the row becomes fill_value /
 * zero shifts, out_num_neighbors (N) = number kept.  Outputs must not alias the inputs.
 * nvamd_nl_filter_coo_flags: keep (E) bytes = 1 where edge e = (neighbor_list[e,0], [e,1]) is
 * inside the cutoff. */
int32_t nvamd_nl_filter_matrix(const float* positions, const float* cells, int32_t per_system_cells,
                               const int32_t* neighbor_matrix, const int32_t* neighbor_matrix_shifts,
                               const int32_t* batch_idx, int32_t n_atoms, int32_t max_neighbors,
                               int32_t fill_value, double cutoff, int32_t* out_neighbor_matrix,
                               int32_t* out_num_neighbors, int32_t* out_shifts, void* stream);
int32_t nvamd_nl_filter_coo_flags(const float* positions, const float* cells, int32_t per_system_cells,
                                  const int32_t* neighbor_list, const int32_t* neighbor_list_shifts,
                                  const int32_t* batch_idx, int64_t n_edges, double cutoff,
                                  uint8_t* keep, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NVALCHEMI_AMD_H */
