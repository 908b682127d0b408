"""Builds tests/cpp/ops_mirror_check.cpp with g++ against include/rmlx_ops.hpp and the C-ABI library."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
SRC = os.path.join(ROOT, "tests", "cpp", "ops_mirror_check.cpp")
EXE = os.path.join(ROOT, "tests", "cpp", "build", "ops_mirror_check")


def build_check_program(force=False):
    """g++ build of the check program; also called by the repository's build entry point."""
    deps = [SRC, os.path.join(ROOT, "include", "rmlx_ops.hpp"), os.path.join(ROOT, "include", "rmlx_hip.h")]
    if not force and os.path.exists(EXE) and all(os.path.getmtime(EXE) >= os.path.getmtime(d) for d in deps):
        return EXE
    os.makedirs(os.path.dirname(EXE), exist_ok=True)
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
                           SRC, "-o", EXE, "-L", os.path.join(ROOT, "rmlx_amd", "lib"), "-lrmlx_hip",
                           "-Wl,-rpath,$ORIGIN/../../../rmlx_amd/lib"])
    return EXE
