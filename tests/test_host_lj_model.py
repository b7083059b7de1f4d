"""``LennardJonesModelWrapper`` on the host: construction, configuration, ``adapt_input`` /
``adapt_output`` / ``output_data`` -- the reference's own cases (test/models/test_lj_model.py:80-500),
which never reach the pair kernel, restated against this package's wrapper."""

from pathlib import Path

import pytest
import torch

from nvalchemi_amd.data import AtomicData, Batch
from nvalchemi_amd.models import LennardJonesModelWrapper, ModelConfig, NeighborListFormat


def lj_batch(n_atoms=4, max_neighbors=8):
    data = AtomicData(torch.randn(n_atoms, 3), torch.ones(n_atoms, dtype=torch.int64),
                      atomic_masses=torch.ones(n_atoms))
    data.add_node_property("neighbor_matrix", torch.full((n_atoms, max_neighbors), n_atoms, dtype=torch.int32))
    data.add_node_property("num_neighbors", torch.zeros(n_atoms, dtype=torch.int32))
    return Batch.from_data_list([data])


def make_model(epsilon=0.0104, sigma=3.40, cutoff=8.5, **kw):
    return LennardJonesModelWrapper(epsilon=epsilon, sigma=sigma, cutoff=cutoff, **kw)


def test_construction_and_configuration():
    m = LennardJonesModelWrapper(epsilon=0.5, sigma=2.0, cutoff=6.0)
    assert (m.epsilon, m.sigma, m.cutoff, m.switch_width, m.half_list) == (0.5, 2.0, 6.0, 0.0, False)
    m = LennardJonesModelWrapper(epsilon=0.5, sigma=2.0, cutoff=6.0, switch_width=1.0, half_list=True)
    assert m.switch_width == 1.0 and m.half_list is True
    m = make_model()
    assert m._energies_buf is None
    for gone in ("_atomic_energies_buf", "_forces_buf", "_virials_buf"):
        assert not hasattr(m, gone)
    cfg = m.model_config
    assert isinstance(cfg, ModelConfig) and "forces" in cfg.active_outputs and "stress" not in cfg.active_outputs
    assert "forces" not in cfg.autograd_outputs and "stress" in cfg.outputs and cfg.supports_pbc is True
    assert cfg.neighbor_config is not None and cfg.neighbor_config.format == NeighborListFormat.MATRIX
    assert LennardJonesModelWrapper(epsilon=0.1, sigma=3.0, cutoff=9.0).model_config.neighbor_config.cutoff == 9.0
    assert m.embedding_shapes == {}
    with pytest.raises(NotImplementedError):
        m.compute_embeddings(lj_batch())
    with pytest.raises(NotImplementedError):
        m.export_model(Path("/tmp/fake.model"))


def test_the_per_system_energy_accumulator_is_kept_between_calls():
    m = make_model()
    cpu = torch.device("cpu")
    m._ensure_compute_buffers(B=1, dtype=torch.float32, device=cpu)
    first = m._energies_buf
    assert isinstance(first, torch.Tensor)
    m._ensure_compute_buffers(B=1, dtype=torch.float32, device=cpu)
    assert m._energies_buf is first
    m._ensure_compute_buffers(B=2, dtype=torch.float32, device=cpu)
    assert m._energies_buf is not first and m._energies_buf.shape == (2,)


def test_adapt_input_collects_what_the_kernel_needs():
    m = make_model()
    data = AtomicData(torch.randn(4, 3), torch.ones(4, dtype=torch.int64))
    data.add_node_property("neighbor_matrix", torch.full((4, 8), 4, dtype=torch.int32))
    data.add_node_property("num_neighbors", torch.zeros(4, dtype=torch.int32))
    with pytest.raises(TypeError, match="requires a Batch input"):
        m.adapt_input(data)
    b = lj_batch()
    r = m.adapt_input(b)
    assert isinstance(r, dict)
    for key in ("positions", "atomic_numbers", "neighbor_matrix", "num_neighbors", "batch_idx", "ptr", "num_graphs",
                "fill_value", "cells", "neighbor_matrix_shifts"):
        assert key in r, key
    assert isinstance(r["positions"], torch.Tensor) and r["batch_idx"].dtype == torch.int32
    assert r["num_graphs"] == 1 and r["fill_value"] == 4 and r["cells"] is None and r["neighbor_matrix_shifts"] is None
    b.cell = torch.eye(3).unsqueeze(0)
    assert m.adapt_input(b)["cells"] is not None
    b = lj_batch()
    b["neighbor_matrix_shifts"] = torch.zeros(4, 8, 3, dtype=torch.int32)
    assert m.adapt_input(b)["neighbor_matrix_shifts"] is not None
    b = lj_batch()
    del b["neighbor_matrix"]
    with pytest.raises(KeyError):
        m.adapt_input(b)


def test_adapt_output_and_output_data_follow_the_active_outputs():
    out = lambda **extra: dict(energy=torch.tensor([[1.0]]), forces=torch.randn(4, 3), **extra)  # noqa: E731
    m = make_model()
    assert "energy" in m.adapt_output(out(stress=torch.randn(1, 3, 3)), lj_batch())
    m.model_config.active_outputs = {"energy", "forces"}
    assert "forces" in m.adapt_output(out(), lj_batch()) and "forces" in m.output_data()
    assert "stress" not in m.adapt_output(out(virial=torch.randn(1, 3, 3)), lj_batch()) and "stress" not in m.output_data()
    m.model_config.active_outputs = {"energy"}
    assert "forces" not in m.adapt_output(out(), lj_batch()) and "energy" in m.output_data()

    m.model_config.active_outputs = {"energy", "forces", "stress"}
    assert "stress" in m.output_data()
    b = lj_batch()
    b.cell = 2.0 * torch.eye(3).unsqueeze(0)
    b.pbc = torch.ones(1, 3, dtype=torch.bool)
    w = torch.randn(1, 3, 3)
    got = m.adapt_output(out(virial=w), b)
    assert torch.allclose(got["stress"], -w / 8.0)
    s = torch.randn(1, 3, 3)
    assert torch.allclose(m.adapt_output(out(stress=s), lj_batch())["stress"], s)
    with pytest.raises(ValueError, match="stress output requires cell"):
        m.adapt_output(out(virial=w), lj_batch())
    with pytest.raises(RuntimeError, match="missing from model output"):
        m.adapt_output(out(), b)
