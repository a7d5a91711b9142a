"""The library's boundary is a C ABI: `include/flashlight_amd.h` must be usable from plain C, and a host program that is
not Python and links neither torch nor anything of this package but the shared library must get the right numbers.
tests/c_host/attn_host.c is such a program (hipMalloc'ed operands, its own stream, forward + backward, checked against
loops in double precision inside the program); `python -m flashlight_amd.build` compiles it next to its source."""
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
SRC = ROOT / "tests" / "c_host" / "attn_host.c"
BIN = SRC.with_suffix("")


def test_the_header_is_plain_c99():
    gcc = shutil.which("gcc")
    assert gcc, "gcc is part of this image"
    probe = '#include "flashlight_amd.h"\n#include "flashlight_amd_probe.h"\nint main(void) { return (int)sizeof(fl_attn_bwd_params) == 0; }\n'
    r = subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", f"-I{ROOT / 'include'}",
                        "-x", "c", "-"], input=probe, text=True, capture_output=True)
    assert r.returncode == 0, r.stderr


def test_the_host_program_is_built_and_links_only_the_library_and_the_hip_runtime():
    assert BIN.exists(), "run `python -m flashlight_amd.build` (it compiles tests/c_host/attn_host.c)"
    needed = subprocess.run(["readelf", "-d", str(BIN)], text=True, capture_output=True).stdout
    libs = [line.split("[")[1].split("]")[0] for line in needed.splitlines() if "(NEEDED)" in line]
    assert any(n.startswith("libflashlight_amd") for n in libs) and any(n.startswith("libamdhip64") for n in libs), libs
    assert not any("torch" in n or "python" in n for n in libs), libs


@pytest.mark.gpu
def test_the_host_program_gets_the_right_numbers():
    assert BIN.exists(), "run `python -m flashlight_amd.build` (it compiles tests/c_host/attn_host.c)"
    r = subprocess.run([str(BIN)], text=True, capture_output=True, timeout=100)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert r.stdout.count(" ok") == 4, r.stdout
