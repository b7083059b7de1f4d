"""Throughput of the batched MD inner loop on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--boxes B] [--no-cpu-baseline]

Workload (the configuration the metric is quoted on): 256 periodic cubic Lennard-Jones
liquid boxes of 3900 atoms (998 400 atoms), reduced units, density 0.8 sigma^-3, uniform
random positions (seed 0) relaxed by 50 FIRE steps (dt 0.005, maxstep 0.07 sigma), then NVE velocity Verlet with dt = 0.005,
cutoff 2.5 sigma, the neighbor list rebuilt on every step.  One step is one pass of the hot
path through the package's own API: ``NVE.step`` = velocity-Verlet position update ->
``NeighborListHook`` (cell-list build) -> ``LennardJonesModelWrapper`` (pair kernel + per-system
energies) -> velocity finalize.  All inputs are resident in HBM when the timed region starts.

Prints ONE JSON line.  ``value`` = atoms x steps / wall time of the timed region.  ``roofline``
describes the neighbor build (the stage that dominates the step): algorithmic bytes
20 N + 16 E per build divided by its average duration, measured with HIP events recorded on
the stream the kernels run on, inside the timed region.  ``stages`` gives the same for the
pair kernel (36 N + 16 E + 4 B) and the two velocity-Verlet halves (68 N and 44 N).
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
    "nl": 1024 * (2 * (31569 + 6576) + (845320 + 62277)),   # search + per-system sort
    "lj": 1024 * (2 * (178661 + 2448) + 78193 + 13),        # pair kernel + system ranges
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_liquid_batch(n_boxes: int, n_per_box: int, density: float, seed: int, device):
    import torch

    from nvalchemi_amd.data import AtomicData, Batch

    L = (n_per_box / density) ** (1.0 / 3.0)
    g = torch.Generator().manual_seed(seed)
    data = []
    for _ in range(n_boxes):
        pos = torch.rand(n_per_box, 3, generator=g) * L
        data.append(AtomicData(pos, torch.full((n_per_box,), 18, dtype=torch.long),
                               atomic_masses=torch.ones(n_per_box), cell=torch.eye(3) * L,
                               pbc=torch.tensor([True, True, True]), forces=torch.zeros(n_per_box, 3),
                               energy=torch.zeros(1, 1)))
    return Batch.from_data_list(data, device=device), L


class StageTimer:
    """HIP events around each C-ABI entry point of a step (neighbor build, pair kernel, the two
    velocity-Verlet halves), recorded on the stream the kernels are enqueued on."""

    ENTRY = {"nl": "nl_build", "lj": "lj_energy_forces", "vv_pre": "vv_position_update",
             "vv_post": "vv_velocity_finalize"}

    def __init__(self):
        import torch

        from nvalchemi_amd import _lib

        self.torch = torch
        self.ev = {k: [] for k in self.ENTRY}
        self.enabled = False
        for key, name in self.ENTRY.items():
            setattr(_lib, name, self._timed(getattr(_lib, name), key))

    def _timed(self, fn, key):
        def call(*a, **k):
            if not self.enabled:
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


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--boxes", type=int, default=256, help="number of 3900-atom boxes (256 = the quoted workload)")
    ap.add_argument("--relax-steps", type=int, default=50)
    ap.add_argument("--skin", type=float, default=0.0,
                    help="Verlet skin of the neighbor hook (0 = rebuild every step, the quoted workload)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-stage-events", action="store_true", help="do not record per-stage HIP events")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from nvalchemi_amd import _lib
    from nvalchemi_amd.dynamics import FIRE, NVE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    if not torch.cuda.is_available():
        print("bench.py needs a ROCm device", file=sys.stderr)
        return 2
    _lib.library()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    n_per_box, density, rc, dt = 3900, 0.8, 2.5, 0.005
    batch, L = make_liquid_batch(args.boxes, n_per_box, density, 0, dev)
    N, B = batch.num_nodes, batch.num_graphs
    model = LennardJonesModelWrapper(epsilon=1.0, sigma=1.0, cutoff=rc)

    t0 = time.perf_counter()
    relax = FIRE(model, dt=dt, maxstep=RELAX_MAXSTEP, hooks=model.make_neighbor_hooks())
    relax.run(batch, n_steps=args.relax_steps)
    torch.cuda.synchronize()
    log(f"[bench] N={N} B={B} L={L:.3f}; {args.relax_steps} FIRE steps in {time.perf_counter() - t0:.2f}s; "
        f"E/atom={float(batch.energy.sum()) / N:.3f} fmax={float(batch.forces.norm(dim=1).max()):.3e}")
    batch.velocities.zero_()

    if args.skin > 0.0:
        model.model_config.neighbor_config.skin = args.skin
    hooks = model.make_neighbor_hooks()
    dyn = NVE(model, dt=dt * 10.180505710759414, hooks=hooks)  # NVE takes fs; 0.005 internal units
    timer = None if args.no_stage_events else StageTimer()
    for _ in range(args.warmup):
        dyn.step(batch)
    torch.cuda.synchronize()
    if timer:
        timer.enabled = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        dyn.step(batch)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    if timer:
        timer.enabled = False

    nn = batch.num_neighbors
    K = batch.neighbor_matrix.shape[1]
    E = int(nn.clamp(max=K).sum())
    ke = 0.5 * float((batch.atomic_masses.unsqueeze(1) * batch.velocities ** 2).sum())
    finite = bool(torch.isfinite(batch.positions).all())
    log(f"[bench] E={E} ({E / N:.1f}/atom, max {int(nn.max())}, K={K}); PE/atom={float(batch.energy.sum()) / N:.3f} "
        f"KE/atom={ke / N:.3f} finite={finite}")

    ms_per_step = wall / args.steps * 1e3
    value = N * args.steps / wall
    stages = {}
    if timer:
        ms = timer.mean_ms()
        # Algorithmic bytes are the compulsory traffic at the API's own I/O layout: a pair is its
        # 4-byte index and its 12-byte shift.  The pair kernel derives shifts from positions in
        # cells wider than twice the search radius (this workload's are) and then does not read
        # them: the bytes it still has to touch are reported beside the API-level figure.
        stamp = getattr(batch, "_neighbor_search_cutoff", None)
        widths = 1.0 / torch.linalg.inv(batch.cell.double()).norm(dim=1)
        shifts_derived = bool(stamp) and bool((widths > 2.0002 * stamp[0]).all())
        alg = {"nl": 20 * N + 16 * E, "lj": 36 * N + 16 * E + 4 * B, "vv_pre": 68 * N, "vv_post": 44 * N}
        for k, b in alg.items():
            gbps = b / (ms[k] * 1e-3) / 1e9
            stages[k] = {"ms": round(ms[k], 4), "alg_bytes": b, "GBps": round(gbps, 1),
                         "frac": round(gbps / HBM_PEAK_GBPS, 4)}
        if shifts_derived:
            touched = 36 * N + 4 * E + 4 * B
            stages["lj"]["shifts_derived_not_read"] = True
            stages["lj"]["bytes_it_must_touch"] = touched
            stages["lj"]["GBps_touched"] = round(touched / (ms["lj"] * 1e-3) / 1e9, 1)
        log("[bench] stage ms: " + ", ".join(f"{k}={v['ms']}" for k, v in stages.items())
            + f"; sum={sum(v['ms'] for v in stages.values()):.3f} vs wall/step={ms_per_step:.3f}")
    result = {
        "metric": "atom-steps/s",
        "value": value,
        "unit": "atom-steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{B} periodic LJ-liquid boxes x {n_per_box} atoms, rho=0.8, rc=2.5 sigma, "
                               f"{args.relax_steps} FIRE steps then NVE dt=0.005, "
                               + ("neighbor rebuild every step" if args.skin <= 0.0 else
                                  f"Verlet skin {args.skin} sigma (rebuild when an atom has moved skin/2)"),
                   "n_atoms": N, "n_systems": B, "edges": E, "max_neighbors": K, "seed": 0},
        "edges_per_s": (E / (stages["nl"]["ms"] * 1e-3)) if stages else None,
    }
    if stages:
        nl = stages["nl"]
        result["roofline"] = {"bound": "hbm", "achieved": nl["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                              "frac": nl["frac"],
                              "traffic": MEASURED_TRAFFIC_BYTES["nl"] if (B == 256 and args.relax_steps == 50 and args.skin <= 0.0) else None,
                              "kernel": "neighbor build (nvamd_nl_build)",
                              "alg_bytes_per_launch": nl["alg_bytes"], "ms_per_launch": nl["ms"]}
        result["stages"] = stages
    if not args.no_cpu_baseline:
        # about ten seconds of host work: 32 boxes, 20 steps on one thread, then on the box's share of cores
        sample_boxes, cpu_steps = min(B, 32), 20
        cb, n_s = cpu_baseline(batch.positions.cpu().numpy(), batch.cell.cpu().numpy(), batch.pbc.cpu().numpy(),
                               n_per_box, sample_boxes, K, steps=cpu_steps)
        v1, c1, t1 = cb["1"]
        va, ca, ta = cb["all"]
        log(f"[bench] cpu oracle: {v1:.3e} atom-steps/s on 1 thread ({t1:.1f}s), {va:.3e} on {ca} threads ({ta:.1f}s)")
        result["cpu_baseline"] = {"value": v1, "unit": "atom-steps/s", "cores": c1, "kind": "port",
                                  "sample": f"first {sample_boxes} boxes ({n_s} atoms) of the same workload, {cpu_steps} steps "
                                            "(VV + cell-list build + LJ + VV), C oracle -O3",
                                  "all_cores": {"value": va, "cores": ca,
                                                "note": "OpenMP over systems in the neighbor build only"}}
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
