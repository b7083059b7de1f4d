"""CPU checks of the C-ABI boundary: the library loads, exports every symbol the header
declares, sizes workspaces without a device, and refuses CPU tensors (no fallback path)."""

import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "nvalchemi_amd.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nvamd_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from nvalchemi_amd import _lib

    lib = _lib.library()
    names = declared_symbols()
    assert len(names) >= 14
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(_lib.EXPORTED_SYMBOLS) == names
    assert lib.nvamd_abi_version() == 1


def test_workspace_sizes_are_host_computations():
    from nvalchemi_amd import _lib

    small = _lib.nl_workspace_bytes(1000, 4)
    big = _lib.nl_workspace_bytes(1_000_000, 256)
    assert 0 < small < big < 200 * 2**20
    assert _lib.nl_workspace_bytes(0, 0) > 0


def test_static_scratch_macro_is_the_workspace_of_its_largest_case(tmp_path):
    """NVAMD_LJ_STATIC_SCRATCH_BYTES in the header must equal what the pair kernel carves for
    NVAMD_LJ_STATIC_MAX_SYSTEMS systems (full list: the size does not depend on the number of atoms), so the
    macro cannot drift from the carving.  The header is read by a C compiler, as a C caller would."""
    import ctypes
    import subprocess

    from nvalchemi_amd import _lib

    src = tmp_path / "m.c"
    src.write_text('#include <stdio.h>\n#include "nvalchemi_amd.h"\nint main(void) { printf("%d %zu\\n", '
                   "(int)NVAMD_LJ_STATIC_MAX_SYSTEMS, (size_t)NVAMD_LJ_STATIC_SCRATCH_BYTES); return 0; }\n")
    exe = tmp_path / "m"
    subprocess.run(["gcc", "-std=c99", "-I", str(ROOT / "include"), str(src), "-o", str(exe)], check=True)
    max_systems, scratch = map(int, subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split())
    assert max_systems == _lib.LJ_STATIC_MAX_SYSTEMS
    for n_atoms in (0, 1, 10_000_000):
        out = ctypes.c_size_t(0)
        assert _lib.library().nvamd_lj_workspace_bytes(n_atoms, max_systems, 0, ctypes.byref(out)) == 0
        assert out.value == scratch


def test_error_codes_and_messages_cross_the_boundary():
    import ctypes

    from nvalchemi_amd import _lib

    lib = _lib.library()
    out = ctypes.c_size_t(0)
    assert lib.nvamd_nl_workspace_bytes(-1, 1, ctypes.byref(out)) == 1
    assert b"bad argument" in lib.nvamd_last_error()
    # invalid arguments are rejected before anything touches a device
    rc = lib.nvamd_nl_build(None, None, None, None, None, None, 10, 1, -1.0, 8, 0, 0, None, None, None, None, 0, None)
    assert rc == 1 and b"cutoff" in lib.nvamd_last_error()
    rc = lib.nvamd_lj_energy_forces(None, None, None, None, None, None, 0, 0, 0, 0, 1.0, 1.0, 1.0, 1.5, 0,
                                    None, None, None, None, None, 0, None)
    assert rc == 1 and b"switch_width" in lib.nvamd_last_error()


def test_cpu_tensors_are_refused_not_emulated():
    from nvalchemi_amd import _lib
    from nvalchemi_amd.dynamics._ops.velocity_verlet import vv_position_update

    n = 4
    z = torch.zeros(n, 3)
    with pytest.raises(_lib.KernelLibraryError):
        vv_position_update(z, z.clone(), z.clone(), torch.ones(n), torch.ones(1), torch.zeros(n, dtype=torch.int32))
    with pytest.raises(_lib.KernelLibraryError):
        _lib.segment_fmax(z, torch.zeros(n, dtype=torch.int32), torch.zeros(1))


def test_product_never_imports_the_oracle():
    pkg = ROOT / "nvalchemi-toolkit_amd"
    for path in list(pkg.rglob("*.py")) + list(pkg.rglob("*.hip")) + list(pkg.rglob("*.h")):
        text = path.read_text()
        assert "import oracle" not in text and "md_oracle" not in text, path
