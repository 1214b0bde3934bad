"""Host logic of the prefill GEMMs' workgroup -> tile map, checked on the CPU: the header
(torchlette_amd/csrc/tile_map.h) has no HIP types, so tests/cpp/tile_map_check.cpp is built
with g++ and run here.  It covers 35 000 tile counts x 5 tile cost pairs: every tile taken
exactly once, the host's XCD account equal to the real one, no XCD crowded into more
rounds than the chip needs."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def test_tile_map_covers_every_tile_once_and_keeps_the_xcds_level(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++ on this machine")
    exe = str(tmp_path / "tile_map_check")
    subprocess.run([gxx, "-O2", "-std=c++17", "-I", os.path.join(HERE, "..", "torchlette_amd", "csrc"),
                    os.path.join(HERE, "cpp", "tile_map_check.cpp"), "-o", exe], check=True)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.startswith("ok "), out.stdout + out.stderr
