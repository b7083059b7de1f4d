"""bench.py without a GPU: the contract of its command line and the shapes of its synthetic workloads."""

import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))

import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0
    assert "one GPU" in (out.stdout + out.stderr)


def test_fcc_batch_is_configuration_two():
    batch = bench.make_fcc_batch("cpu", n_boxes=3, reps=2)
    assert batch.num_graphs == 3 and batch.num_nodes == 3 * 32
    cell = batch.cell[0]
    assert torch.allclose(cell, torch.eye(3) * 7.2)
    assert bool(batch.pbc.all())


def test_inflight_mix_sizes_are_log_uniform_between_the_bounds():
    batch = bench.make_inflight_mix("cpu", n_systems=64, n_lo=8, n_hi=200, seed=1)
    n = np.asarray(batch.num_nodes_list)
    assert n.min() >= 8 and n.max() < 200 and len(n) == 64
    # triclinic: lattice vectors of 0.8-1.2 x the cube root of the volume per system, angles 60-120 degrees
    H = batch.cell.double()
    lengths = H.norm(dim=2)
    cosines = torch.stack([(H[:, i] * H[:, j]).sum(1) / (lengths[:, i] * lengths[:, j]) for i, j in ((0, 1), (0, 2), (1, 2))], 1)
    assert float(cosines.abs().max()) <= 0.5 + 1e-9
    # about the stated density
    vol = torch.linalg.det(H).abs()
    rho = torch.as_tensor(n, dtype=torch.double) / vol
    assert 0.02 < float(rho.median()) < 0.2


def test_liquid_batch_is_the_quoted_density():
    batch, L = bench.make_liquid_batch(2, 100, 0.8, 0, "cpu")
    assert batch.num_nodes == 200
    assert L == pytest.approx((100 / 0.8) ** (1 / 3))
    assert float(batch.positions.min()) >= 0.0 and float(batch.positions.max()) <= L


def test_measured_traffic_names_both_stages():
    assert set(bench.MEASURED_TRAFFIC_BYTES) == {"nl", "lj"}
    assert all(v > 0 for v in bench.MEASURED_TRAFFIC_BYTES.values())
