"""Compiles step_harness.c and epoch_harness.c as strict C99 against include/scanet_hip.h and links them with the
in-tree library.

    python tests/c_harness/build.py

The binaries stay next to this file (git-ignored) and find the library through a relative rpath.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
PROGRAMS = ("step_harness", "epoch_harness")
BINARY = os.path.join(HERE, "step_harness")
C_FLAGS = ["-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-O1"]


def syntax_check_header() -> None:
    """include/scanet_hip.h alone must be valid C99 (no C++ leaking into the boundary)."""
    cmd = ["gcc", *C_FLAGS, "-fsyntax-only", "-x", "c", "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "include", "scanet_hip.h")]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"scanet_hip.h is not clean C99:\n{res.stdout}\n{res.stderr}")


def build_harness() -> list:
    lib_dir = os.path.join(ROOT, "scanet3_amd")
    built = []
    for name in PROGRAMS:
        binary = os.path.join(HERE, name)
        cmd = ["gcc", *C_FLAGS, "-I", os.path.join(ROOT, "include"), os.path.join(HERE, name + ".c"), "-o", binary,
               "-L", lib_dir, "-lscanet_hip", "-Wl,-rpath,$ORIGIN/../../scanet3_amd", "-Wl,-rpath-link,/opt/rocm/lib",
               "-Wl,-rpath,/opt/rocm/lib"]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"building {name} failed:\n{res.stdout}\n{res.stderr}")
        built.append(binary)
    return built


if __name__ == "__main__":
    syntax_check_header()
    print("built", build_harness())
    sys.exit(0)
