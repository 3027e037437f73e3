"""The C++ mirror of the reference's operator API (host/fnx.hpp) compiles against the C ABI and its host-only functions
return what the oracle says (no GPU: lookup, acceptance, the sampler's distribution, the GGUF reader)."""
import os
import subprocess

import numpy as np

import fnx_gpu
import gguf_files as gf

HERE = os.path.dirname(os.path.abspath(__file__))


def test_host_mirror_compiles_and_runs(oracle, tmp_path):
    lib = os.path.join(fnx_gpu.PKG_DIR, "libfnx_mi355x.so")
    assert os.path.exists(lib), "build the library first (__graft_entry__.build())"
    exe = str(tmp_path / "host_mirror_check")
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-o", exe, os.path.join(HERE, "host_mirror_check.cpp"), lib,
                    "-Wl,-rpath," + fnx_gpu.PKG_DIR, "-Wl,-rpath,/opt/rocm/lib"], check=True, capture_output=True, text=True)
    path = gf.write(tmp_path / "h.gguf", [("w", gf.F32, [8, 3], b"\0" * 96)], keys=[gf.kv("general.architecture", gf.STR, "demo")])
    r = subprocess.run([exe, path], check=True, capture_output=True, text=True, timeout=120)
    lines = r.stdout.strip().splitlines()
    ctx = np.array([5, 6, 7, 8, 9, 1, 2, 5, 6, 7], np.int32)
    want, match = oracle.lookup_drafts(ctx, 4, 8)
    assert lines[0] == f"drafts {len(want)} match {match} first {int(want[0])}"
    assert lines[1] == f"accept {oracle.accept_greedy(np.array([9, 4, 5, 6], np.int32), np.array([4, 5, 7, 1], np.int32))}"
    p0 = 1.0 / (1.0 + np.exp(-1.0))
    assert lines[2] == f"dist 2 p0 {p0:.6f} draw 11 12"
    assert lines[3] == "gguf tensors 1 ne0 8 arch demo"
    assert lines[4] == "refused: gguf: no tensor missing"


def test_attention_window_bounds(tmp_path):
    """the attention kernels' index arithmetic for a position word the host cannot see, compiled for the host: caches of
    192, 520 and 32,768 cells with windows from below 0 to past the end never index outside the cache"""
    exe = str(tmp_path / "attn_window_check")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(fnx_gpu.PKG_DIR, "csrc"), "-o", exe,
                    os.path.join(HERE, "attn_window_check.cpp")], check=True, capture_output=True, text=True)
    r = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=120)
    assert r.stdout.startswith("ok "), r.stdout


def test_window_plan(tmp_path):
    """the one-launch verify window's split of a window over the grid, compiled for the host: every router row, gate|up item
    and unit of the down matrices is taken exactly once and every hand-over waits for exactly the blocks that arrive"""
    exe = str(tmp_path / "moe_window_plan_check")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(fnx_gpu.PKG_DIR, "csrc"), "-o", exe,
                    os.path.join(HERE, "moe_window_plan_check.cpp")], check=True, capture_output=True, text=True)
    r = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=120)
    assert r.stdout.startswith("ok "), r.stdout
