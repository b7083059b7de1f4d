"""Throughput of the batched MD inner loop on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--repeats R] [--config {2,3,4,5}] [--boxes B]
                    [--no-cpu-baseline] [--no-other-configs]

Other configurations of the baseline (``--config``): 2 = 64 FCC boxes of 500 atoms, NVE; 4 = 2048
triclinic cells of 8-2000 atoms, FIRE with per-system convergence masks; 5 = one box of 4 M atoms,
NVE.  They print the same line (without the CPU baseline, which is timed on the quoted workload only).

Workload (the configuration the metric is quoted on, ``--config 3``, the default): 256 periodic cubic Lennard-Jones
liquid boxes of 3900 atoms (998 400 atoms), reduced units, density 0.8 sigma^-3, uniform
random positions (seed 0) relaxed by 50 FIRE steps (dt 0.005, maxstep 0.07 sigma), then NVE velocity Verlet with dt = 0.005,
cutoff 2.5 sigma, the neighbor list rebuilt on every step.  One step is one pass of the hot
path through the package's own API: ``NVE.step`` = velocity-Verlet position update ->
``NeighborListHook`` (cell-list build) -> ``LennardJonesModelWrapper`` (pair kernel + per-system
energies) -> velocity finalize; the steps without stage events go through ``NVE.run``, which replays a
captured step as a HIP graph where the dynamics allows it (the same kernels on the same buffers, enqueued
by the device instead of the host).  All inputs are resident in HBM when the timed region starts.

Prints ONE JSON line.  The timed region of exactly ``--steps`` steps is run ``--repeats`` times (5) with a
device synchronisation on both sides of each; ``value`` = atoms x steps / wall time of the region of
median duration, and ``repeats`` lists them all.  ``roofline`` describes the neighbor build (the stage
that dominates the step): algorithmic bytes 20 N + 16 E per build divided by its average duration,
measured with HIP events recorded on the stream the kernels run on, inside the timed regions: at most
every 4th step is sampled and a sampled step times one entry point, the entry points taking turns (an
event between two kernels costs the device about 4 us; eight per step took 4.5 % off the throughput).
``stages`` gives the same for the pair kernel (36 N + 16 E + 4 B) and the two velocity-Verlet halves
(68 N and 44 N).  The default run appends ``other_configs``: configurations 2, 4 and 5 measured the
same way over fewer steps.
``cpu_baseline`` times the CPU oracle (a port of the same algorithms, not the product) on a
bounded sample of the same workload on this machine's host cores.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (ROOT, ROOT / "nvalchemi-toolkit_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
# largest displacement of an atom per FIRE step of the relaxation, in sigma (the optimizer's default of 0.2 is
# meant for Angstrom-sized atoms; from a random gas it lets overlapping atoms jump through each other)
RELAX_MAXSTEP = 0.07

# HBM bytes per launch on the default workload (256 boxes, seed 0), from rocprofv3 --pmc runs of
# this script (FETCH_SIZE, then WRITE_SIZE; averages over the timed steps).  FETCH_SIZE reads
# half of what a copy kernel of known size fetches and WRITE_SIZE reads its writes in KiB, so
# bytes = 1024 * (2 * FETCH_SIZE + WRITE_SIZE).  Summed over the kernels of each entry point.
MEASURED_TRAFFIC_BYTES = {
    "nl": 1024 * (2 * (32561 + 6106) + (850038 + 63352)),   # search + per-system sort
    "lj": 1024 * (2 * (165411 + 23) + 15748 + 21),          # pair kernel + conversion of the per-system sums
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def _batch_of(systems, device):
    """systems: list of (positions (n,3) float32 tensor, cell (3,3) tensor); argon-like atoms of unit mass."""
    import torch

    from nvalchemi_amd.data import AtomicData, Batch

    data = []
    for pos, cell in systems:
        n = pos.shape[0]
        data.append(AtomicData(pos, torch.full((n,), 18, dtype=torch.long), atomic_masses=torch.ones(n), cell=cell,
                               pbc=torch.tensor([True, True, True]), forces=torch.zeros(n, 3),
                               energy=torch.zeros(1, 1)))
    return Batch.from_data_list(data, device=device)


def make_liquid_batch(n_boxes: int, n_per_box: int, density: float, seed: int, device):
    import torch

    L = (n_per_box / density) ** (1.0 / 3.0)
    g = torch.Generator().manual_seed(seed)
    systems = [(torch.rand(n_per_box, 3, generator=g) * L, torch.eye(3) * L) for _ in range(n_boxes)]
    return _batch_of(systems, device), L


def make_fcc_batch(device, n_boxes=64, reps=5, a=3.6, jitter=0.05, seed=0):
    """BASELINE configuration 2: cubic FCC boxes of 4 reps^3 atoms with Gaussian jitter."""
    import numpy as np
    import torch

    rng = np.random.default_rng(seed)
    base = np.array([[0, 0, 0], [0.5, 0.5, 0], [0.5, 0, 0.5], [0, 0.5, 0.5]])
    g = np.stack(np.meshgrid(*[np.arange(reps)] * 3, indexing="ij"), -1).reshape(-1, 1, 3)
    lat = ((g + base[None]) * a).reshape(-1, 3)
    cell = torch.eye(3) * (reps * a)
    systems = [(torch.from_numpy((lat + rng.normal(0, jitter, lat.shape)).astype(np.float32)), cell)
               for _ in range(n_boxes)]
    return _batch_of(systems, device)


def _triclinic_cell(rng, length):
    """Lattice vectors of length 0.8-1.2 x ``length`` with angles uniform in 60-120 degrees."""
    import numpy as np

    while True:
        al, be, ga = np.deg2rad(rng.uniform(60.0, 120.0, 3))
        la, lb, lc = length * rng.uniform(0.8, 1.2, 3)
        cx = lc * np.cos(be)
        cy = lc * (np.cos(al) - np.cos(be) * np.cos(ga)) / np.sin(ga)
        cz2 = lc * lc - cx * cx - cy * cy
        if cz2 <= (0.3 * lc) ** 2:
            continue
        return np.array([[la, 0, 0], [lb * np.cos(ga), lb * np.sin(ga), 0], [cx, cy, np.sqrt(cz2)]])


def make_inflight_mix(device, n_systems=2048, n_lo=8, n_hi=2000, density=0.0764, seed=0):
    """BASELINE configuration 4: triclinic cells of 8-2000 atoms (log-uniform), about 40 neighbors per
    atom inside 5 Angstrom, uniform random positions."""
    import numpy as np
    import torch

    rng = np.random.default_rng(seed)
    counts = np.exp(rng.uniform(np.log(n_lo), np.log(n_hi), n_systems)).astype(np.int64)
    systems = []
    for n in counts:
        H = _triclinic_cell(rng, (n / density) ** (1.0 / 3.0))
        pos = rng.uniform(0, 1, (n, 3)) @ H
        systems.append((torch.from_numpy(pos.astype(np.float32)), torch.from_numpy(H.astype(np.float32))))
    return _batch_of(systems, device)


def make_single_box(device, n_atoms=4_000_000, density=0.1, seed=0):
    """BASELINE configuration 5: one periodic cubic box, uniform random positions."""
    import torch

    L = (n_atoms / density) ** (1.0 / 3.0)
    g = torch.Generator().manual_seed(seed)
    return _batch_of([(torch.rand(n_atoms, 3, generator=g) * L, torch.eye(3) * L)], device)


class StageTimer:
    """HIP events around one C-ABI entry point of a sampled step (neighbor build, pair kernel, the two
    velocity-Verlet halves, FIRE, fmax), recorded on the stream the kernels are enqueued on.  The entry points
    that a configuration calls take turns from one sampled step to the next, so a sampled step carries two
    events, not two per stage."""

    ENTRY = {"nl": "nl_build", "lj": "lj_energy_forces", "vv_pre": "vv_position_update",
             "vv_post": "vv_velocity_finalize", "fire": "fire_step", "fmax": "segment_fmax"}

    def __init__(self):
        import torch

        from nvalchemi_amd import _lib

        self.torch = torch
        self.reset()
        for key, name in self.ENTRY.items():
            setattr(_lib, name, self._timed(getattr(_lib, name), key))

    def reset(self):
        self.ev = {k: [] for k in self.ENTRY}
        self.seen = []      # entry points called so far, in the order of their first call
        self.want = None    # the entry point the current step times (None: none)
        self.turn = None

    def select(self, turn):
        """``turn``: running number of the sampled step, or None for a step that records nothing."""
        self.turn = turn
        self.want = None if (turn is None or not self.seen) else self.seen[turn % len(self.seen)]

    def _timed(self, fn, key):
        def call(*a, **k):
            if key not in self.seen:
                self.seen.append(key)
            if self.turn is None or self.want != key:
                return fn(*a, **k)
            e0 = self.torch.cuda.Event(enable_timing=True)
            e1 = self.torch.cuda.Event(enable_timing=True)
            e0.record()
            out = fn(*a, **k)
            e1.record()
            self.ev[key].append((e0, e1))
            return out

        return call

    def mean_ms(self):
        return {k: (sum(a.elapsed_time(b) for a, b in v) / len(v) if v else float("nan")) for k, v in self.ev.items()}


def cpu_baseline(pos, cell, pbc, n_per_box, n_boxes_sample, K, steps):
    """Oracle (CPU port) on the first ``n_boxes_sample`` boxes: the same step, single thread."""
    import numpy as np

    import oracle

    n = n_per_box * n_boxes_sample
    P = np.ascontiguousarray(pos[:n])
    C = np.ascontiguousarray(cell[:n_boxes_sample])
    pb = np.ascontiguousarray(pbc[:n_boxes_sample])
    ptr = (np.arange(n_boxes_sample + 1) * n_per_box).astype(np.int32)
    bi = oracle.batch_idx_from_ptr(ptr)
    M = np.ones(n, dtype=np.float32)
    dt = np.full(n_boxes_sample, 0.005, dtype=np.float32)
    out = {}
    # (the host share of a one-GPU box is 16 cores, whatever the machine reports)
    share = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16))
    for label, threads in (("1", 1), ("all", share)):
        oracle.set_threads(threads)
        Pc, V, F = P.copy(), np.zeros_like(P), np.zeros_like(P)
        t0 = time.perf_counter()
        for _ in range(steps):
            oracle.vv_pre(Pc, V, F, M, dt, bi)
            nm, nn, sh = oracle.nl_cell(Pc, C, pb, ptr, 2.5, K)
            F = oracle.lj_matrix(Pc, C, nm, sh, nn, bi, n, 1.0, 1.0, 2.5)["forces"]
            oracle.vv_post(V, F, M, dt, bi)
        dtw = time.perf_counter() - t0
        out[label] = (n * steps / dtw, threads, dtw)
    return out, n


# fp64 operations of one pair on the shifts-derived path of the pair kernel, multiply-adds counted twice:
# r_j - r_i (3), nearest image per component (mul, rint, fma: 12), r^2 (5), reciprocal (estimate + two
# Newton steps: 9), (s/r)^2, ^6, ^12 (4), u (2), u'/r (4), energy sum (2), force sums (6)
LJ_FP64_FLOPS_PER_PAIR = 47
FP64_PEAK_TFLOPS = 78.6  # MI355X vector fp64, published


def setup_config(cfg: int, args, device):
    """Batch, model and dynamics of a BASELINE configuration; returns (batch, dyn, description, warm)."""
    import torch

    from nvalchemi_amd.dynamics import FIRE, NVE, ConvergenceHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    fs = 10.180505710759414  # NVE takes femtoseconds; one internal time unit of the eV / Angstrom / amu system
    if cfg == 3:
        n_per_box, density, rc, dt = 3900, 0.8, 2.5, 0.005
        batch, L = make_liquid_batch(args.boxes, n_per_box, density, 0, device)
        model = LennardJonesModelWrapper(epsilon=1.0, sigma=1.0, cutoff=rc)
        t0 = time.perf_counter()
        relax = FIRE(model, dt=dt, maxstep=RELAX_MAXSTEP, hooks=model.make_neighbor_hooks())
        relax.run(batch, n_steps=args.relax_steps)
        torch.cuda.synchronize()
        log(f"[bench] L={L:.3f}; {args.relax_steps} FIRE steps in {time.perf_counter() - t0:.2f}s; "
            f"E/atom={float(batch.energy.sum()) / batch.num_nodes:.3f} fmax={float(batch.forces.norm(dim=1).max()):.3e}")
        batch.velocities.zero_()
        if args.skin > 0.0:
            model.model_config.neighbor_config.skin = args.skin
        dyn = NVE(model, dt=dt * fs, hooks=model.make_neighbor_hooks())
        what = (f"{batch.num_graphs} periodic LJ-liquid boxes x {n_per_box} atoms, rho=0.8, rc=2.5 sigma, "
                f"{args.relax_steps} FIRE steps (relaxation maxstep {RELAX_MAXSTEP} sigma, not the FIRE default of 0.2) "
                "then NVE dt=0.005, "
                + ("neighbor rebuild every step" if args.skin <= 0.0 else
                   f"Verlet skin {args.skin} sigma (rebuild when an atom has moved skin/2)"))
        return batch, dyn, what
    if cfg == 2:
        batch = make_fcc_batch(device)
        model = LennardJonesModelWrapper(epsilon=0.0104, sigma=2.268, cutoff=6.0)  # pair minimum at the FCC spacing
        dyn = NVE(model, dt=0.5, hooks=model.make_neighbor_hooks())
        return batch, dyn, ("64 periodic cubic boxes x 500 atoms (FCC a=3.6 A + N(0, 0.05 A) jitter), cutoff 6 A, LJ, "
                            "NVE velocity Verlet dt=0.5 fs, neighbor rebuild every step")
    if cfg == 4:
        batch = make_inflight_mix(device)
        batch.status = torch.zeros(batch.num_graphs, 1, dtype=torch.long, device=device)
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=2.5, cutoff=5.0)
        hook = ConvergenceHook.from_fmax(0.05, source_status=0, target_status=1)
        dyn = FIRE(model, dt=0.02, maxstep=0.1, hooks=model.make_neighbor_hooks() + [hook])
        return batch, dyn, ("2048 periodic triclinic cells of 8-2000 atoms (log-uniform, angles 60-120 deg, uniform random "
                            "positions, ~40 neighbors/atom), cutoff 5 A, LJ, FIRE with a per-system fmax criterion that "
                            "freezes converged systems, neighbor rebuild every step")
    if cfg == 5:
        batch = make_single_box(device)
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=1.5, cutoff=6.0)
        # (a random gas has pairs far up the repulsive wall: a few FIRE steps with a short leash take them
        # off it, so that the timed dynamics stays finite)
        t0 = time.perf_counter()
        FIRE(model, dt=0.02, maxstep=0.05, hooks=model.make_neighbor_hooks()).run(batch, n_steps=args.relax_steps)
        torch.cuda.synchronize()
        log(f"[bench] {args.relax_steps} FIRE steps in {time.perf_counter() - t0:.2f}s; "
            f"E/atom={float(batch.energy.sum()) / batch.num_nodes:.3e} fmax={float(batch.forces.norm(dim=1).max()):.3e}")
        batch.velocities.zero_()
        dyn = NVE(model, dt=0.05, hooks=model.make_neighbor_hooks())
        return batch, dyn, ("one periodic cubic box of 4,000,000 atoms, density 0.1 /A^3 (uniform random positions, "
                            f"{args.relax_steps} FIRE steps), cutoff 6 A (~90 neighbors/atom), LJ with fp64 per-system "
                            "energy, NVE velocity Verlet dt=0.05 fs, neighbor rebuild every step")
    raise ValueError(f"unknown configuration {cfg}")


def measure(cfg: int, args, dev, steps: int, warmup: int, repeats: int, timer, with_cpu_baseline: bool):
    """One configuration: set-up, ``warmup`` untimed steps, then ``repeats`` timed regions of exactly ``steps``
    steps each (a device synchronisation on both sides of every region).  The region of median duration is the one
    reported; the others are listed beside it."""
    import torch

    batch, dyn, what = setup_config(cfg, args, dev)
    N, B = batch.num_nodes, batch.num_graphs
    log(f"[bench] configuration {cfg}: N={N} B={B}")
    if timer:
        timer.reset()
    dyn.run(batch, n_steps=warmup)  # (run() captures a steady-state step as a HIP graph where the dynamics allows it)
    torch.cuda.synchronize()
    # Per-stage HIP events: a sampled step times ONE entry point (they take turns), and at most every 4th step is
    # sampled, because an event between two kernels costs the device about 4 us.
    stage_every = max(1, args.stage_every) if args.stage_every else (8 if steps >= 32 else 4 if steps >= 8 else 1)
    walls, hosts = [], []
    sampled = 0
    for _ in range(repeats):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        i = 0
        while i < steps:
            if timer and i % stage_every == 0:
                # a sampled step is taken eagerly, with two HIP events around one of its entry points
                timer.select(sampled)
                sampled += 1
                dyn.step(batch)
                timer.select(None)
                i += 1
            else:
                # the steps up to the next sampled one: the package's own loop (graph replay where it applies)
                k = (min(steps, (i // stage_every + 1) * stage_every) - i) if timer else steps - i
                dyn.run(batch, n_steps=k)
                i += k
        hosts.append(time.perf_counter() - t0)  # what the host needed to enqueue the steps (the device may lag behind it)
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
    if timer:
        timer.select(None)
    order = sorted(range(repeats), key=lambda r: walls[r])
    wall = walls[order[repeats // 2]]
    host = hosts[order[repeats // 2]]
    log(f"[bench] host enqueued {steps} steps in {host / steps * 1e3:.3f} ms/step; with the device: "
        f"{wall / steps * 1e3:.3f} ms/step (median of {repeats}: "
        + ", ".join(f"{w / steps * 1e3:.3f}" for w in walls) + ")")

    nn = batch.num_neighbors
    K = batch.neighbor_matrix.shape[1]
    E = int(nn.clamp(max=K).sum())
    ke = 0.5 * float((batch.atomic_masses.unsqueeze(1) * batch.velocities ** 2).sum())
    finite = bool(torch.isfinite(batch.positions).all())
    log(f"[bench] E={E} ({E / N:.1f}/atom, max {int(nn.max())}, K={K}); PE/atom={float(batch.energy.sum()) / N:.3f} "
        f"KE/atom={ke / N:.3f} finite={finite}")

    ms_per_step = wall / steps * 1e3
    value = N * steps / wall
    quoted = cfg == 3 and B == 256 and args.relax_steps == 50 and args.skin <= 0.0
    stages = {}
    if timer:
        ms = timer.mean_ms()
        # Algorithmic bytes are the compulsory traffic at the API's own I/O layout: a pair is its
        # 4-byte index and its 12-byte shift.  The pair kernel derives shifts from positions in
        # cells wider than twice the search radius and then does not read them; it is then bound
        # by its double-precision arithmetic, and both figures are given.
        stamp = getattr(batch, "_neighbor_search_cutoff", None)
        widths = 1.0 / torch.linalg.inv(batch.cell.double()).norm(dim=1)
        shifts_derived = bool(stamp) and bool((widths > 2.0002 * stamp[0]).all())
        alg = {"nl": 20 * N + 16 * E, "lj": 36 * N + 16 * E + 4 * B, "vv_pre": 68 * N, "vv_post": 44 * N,
               "fire": 96 * N, "fmax": 12 * N + 4 * B}
        for k, b in alg.items():
            if not (ms[k] == ms[k]):  # an entry point this configuration never calls
                continue
            gbps = b / (ms[k] * 1e-3) / 1e9
            stages[k] = {"ms": round(ms[k], 4), "alg_bytes": b, "GBps": round(gbps, 1),
                         "frac": round(gbps / HBM_PEAK_GBPS, 4), "samples": len(timer.ev[k])}
        lj = stages["lj"]
        tflops = LJ_FP64_FLOPS_PER_PAIR * E / (ms["lj"] * 1e-3) / 1e12
        lj["fp64_flops_per_pair"] = LJ_FP64_FLOPS_PER_PAIR
        lj["fp64_TFLOPs"] = round(tflops, 2)
        lj["fp64_frac"] = round(tflops / FP64_PEAK_TFLOPS, 4)
        if shifts_derived:
            # the API-level figure counts 12 bytes of shifts per pair that this path never reads: the
            # fraction of the HBM peak that stands for this stage is that of the bytes it must touch
            touched = 36 * N + 4 * E + 4 * B
            lj["shifts_derived_not_read"] = True
            lj["api_alg_bytes"], lj["api_GBps"], lj["api_frac"] = lj["alg_bytes"], lj["GBps"], lj["frac"]
            lj["alg_bytes"] = touched
            lj["GBps"] = round(touched / (ms["lj"] * 1e-3) / 1e9, 1)
            lj["frac"] = round(lj["GBps"] / HBM_PEAK_GBPS, 4)
            lj["bound"] = "fp64 vector arithmetic"
        log("[bench] stage ms: " + ", ".join(f"{k}={v['ms']}" for k, v in stages.items())
            + f"; sum={sum(v['ms'] for v in stages.values()):.3f} vs wall/step={ms_per_step:.3f}")
    out = {"value": value, "ms_per_step": ms_per_step, "what": what, "N": N, "B": B, "E": E, "K": K,
           "stages": stages, "quoted": quoted, "stage_every": stage_every, "sampled_steps": sampled,
           "repeat_ms_per_step": [round(w / steps * 1e3, 5) for w in walls], "finite": finite}
    if with_cpu_baseline and cfg == 3:
        # about ten seconds of host work: 32 boxes, 20 steps on one thread, then on the box's share of cores
        n_per_box = 3900
        sample_boxes, cpu_steps = min(B, 32), 20
        cb, n_s = cpu_baseline(batch.positions.cpu().numpy(), batch.cell.cpu().numpy(), batch.pbc.cpu().numpy(),
                               n_per_box, sample_boxes, K, steps=cpu_steps)
        v1, c1, t1 = cb["1"]
        va, ca, ta = cb["all"]
        log(f"[bench] cpu oracle: {v1:.3e} atom-steps/s on 1 thread ({t1:.1f}s), {va:.3e} on {ca} threads ({ta:.1f}s)")
        out["cpu_baseline"] = {"value": v1, "unit": "atom-steps/s", "cores": c1, "kind": "port",
                               "sample": f"first {sample_boxes} boxes ({n_s} atoms) of the same workload, {cpu_steps} steps "
                                         "(VV + cell-list build + LJ + VV), C oracle -O3",
                               "all_cores": {"value": va, "cores": ca,
                                             "note": "OpenMP over systems in the neighbor build only"}}
    del batch, dyn
    torch.cuda.empty_cache()
    return out


# steps and warm-up of the configurations that ride along with the default run (kept short: the whole default
# command stays well within a few minutes)
OTHER_CONFIG_STEPS = {2: (100, 20), 4: (40, 10), 5: (10, 3)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--config", type=int, default=3, choices=(2, 3, 4, 5),
                    help="BASELINE configuration (3 = the 1M-atom liquid the metric is quoted on)")
    ap.add_argument("--boxes", type=int, default=256, help="configuration 3: number of 3900-atom boxes (256 = the quoted workload)")
    ap.add_argument("--relax-steps", type=int, default=50)
    ap.add_argument("--skin", type=float, default=0.0,
                    help="configuration 3: Verlet skin of the neighbor hook (0 = rebuild every step, the quoted workload)")
    ap.add_argument("--repeats", type=int, default=5,
                    help="the timed region of exactly --steps steps is run this many times; the median one is reported")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="default run only: do not append the short runs of configurations 2, 4 and 5")
    ap.add_argument("--no-stage-events", action="store_true", help="do not record per-stage HIP events")
    ap.add_argument("--stage-every", type=int, default=None,
                    help="record per-stage HIP events on every n-th timed step (one entry point per sampled step, in "
                         "turn: an event between two kernels costs the device about 4 us); default: every 8th step "
                         "of 32 or more, every 4th of 8 or more")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2
    if args.steps is None:
        args.steps = 30 if args.config == 5 else 200
    if args.warmup is None:
        args.warmup = 5 if args.config == 5 else 20
    args.repeats = max(1, args.repeats)

    import torch

    from nvalchemi_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py needs a ROCm device", file=sys.stderr)
        return 2
    _lib.library()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    timer = None if args.no_stage_events else StageTimer()
    m = measure(args.config, args, dev, args.steps, args.warmup, args.repeats, timer, not args.no_cpu_baseline)
    stages = m["stages"]
    result = {
        "metric": "atom-steps/s",
        "value": m["value"],
        "unit": "atom-steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": m["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": m["what"], "baseline_config": args.config,
                   "n_atoms": m["N"], "n_systems": m["B"], "edges": m["E"], "max_neighbors": m["K"], "seed": 0},
        "repeats": {"n": args.repeats, "reported": "median", "ms_per_step": m["repeat_ms_per_step"]},
        "edges_per_s": (m["E"] / (stages["nl"]["ms"] * 1e-3)) if stages else None,
    }
    if stages:
        nl = stages["nl"]
        result["roofline"] = {"bound": "hbm", "achieved": nl["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                              "frac": nl["frac"],
                              "traffic": MEASURED_TRAFFIC_BYTES["nl"] if m["quoted"] else None,
                              "traffic_source": ("profiles/hbm_traffic_lj_liquid_1M.txt: rocprofv3 --pmc FETCH_SIZE and "
                                                 "WRITE_SIZE runs of this command, not measured in this run") if m["quoted"] else None,
                              "kernel": "neighbor build (nvamd_nl_build)",
                              "alg_bytes_per_launch": nl["alg_bytes"], "ms_per_launch": nl["ms"]}
        result["stages"] = stages
        result["stage_events"] = {"sampled_steps": m["sampled_steps"], "every": m["stage_every"],
                                  "entry_points_per_sampled_step": 1}
    if "cpu_baseline" in m:
        result["cpu_baseline"] = m["cpu_baseline"]
    if args.config == 3 and m["quoted"] and not args.no_other_configs:
        # the other configurations of the baseline, shorter, same measurement (no CPU baseline)
        others = {}
        for cfg, (st, wu) in OTHER_CONFIG_STEPS.items():
            o = measure(cfg, args, dev, st, wu, 3, timer, False)
            others[str(cfg)] = {"workload": o["what"], "n_atoms": o["N"], "n_systems": o["B"], "steps": st, "warmup": wu,
                                "ms_per_step": o["ms_per_step"], "atom_steps_per_s": o["value"],
                                "repeat_ms_per_step": o["repeat_ms_per_step"], "stages": o["stages"],
                                "edges": o["E"], "K": o["K"], "finite": o["finite"]}
        result["other_configs"] = others
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
