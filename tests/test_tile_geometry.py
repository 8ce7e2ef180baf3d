"""The tile geometry of the HIP kernels (odc_amd/csrc/odc_tiles.h), brute-forced on the CPU.

The header compiles for the device and for the host; here g++ builds it alone, with
AddressSanitizer and UndefinedBehaviorSanitizer, into tests/cpu/tile_geometry_check.cpp, which
walks every tile of random and edge-case launches and asserts exact-once coverage of every unit,
in-bounds roles and aligned bodies for all three tile orders, rotated first ranks, one workgroup
per tile and persistent grids, world sizes 1..200 and item lists longer than one launch takes.
"""

import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
SOURCE = ROOT / "tests" / "cpu" / "tile_geometry_check.cpp"


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = tmp_path_factory.mktemp("tiles") / "tile_geometry_check"
    cmd = [
        "g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
        "-Wall", "-Wextra", "-Werror", "-Wno-unknown-pragmas", f"-I{ROOT / 'odc_amd' / 'csrc'}",
        str(SOURCE), "-o", str(exe),
    ]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    return exe


@pytest.mark.parametrize("seed", [1, 2])
def test_every_unit_is_owned_by_exactly_one_tile_role(checker, seed):
    proc = subprocess.run([str(checker), str(seed), "80"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-4000:] + proc.stderr[-4000:]
    assert "tile geometry ok" in proc.stdout


def test_the_library_is_built_from_the_checked_header():
    """The kernels and the launch planning must take their geometry from odc_tiles.h, not from a
    private copy."""
    csrc = ROOT / "odc_amd" / "csrc"
    device, host = (csrc / "odc_kernels.hip").read_text(), (csrc / "odc_host.cpp").read_text()
    for text in (device, host):
        assert '#include "odc_tiles.h"' in text
    for name in ("cursor_seek(", "cursor_enter(", "cursor_coord(", "seg_shape(", "tile_work("):
        assert name in device, name
    assert "fill_tile_table(" in host
    for private in ("struct TileTable", "struct SegShape", "TileCoord locate_tile"):
        assert private not in device + host, f"{private} is defined outside odc_tiles.h again"
