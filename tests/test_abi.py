"""CPU-side checks of the drop-in boundary: the library loads, exports every symbol the header declares, and rejects
bad arguments before touching a device (no compute calls here)."""
import ctypes as C
import os
import re

import numpy as np

import fnx_gpu

ROOT = fnx_gpu.ROOT


def header_functions():
    text = open(os.path.join(ROOT, "include", "fnx_mi355x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fnx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    pkg = fnx_gpu.package()
    lib = pkg.lib()
    names = header_functions()
    assert len(names) >= 18
    for name in names:
        assert hasattr(lib, name), name
    assert set(names) == set(pkg.EXPORTS), "the Python binding and the header list the same entry points"
    assert b"gfx950" in lib.fnx_version()


def test_struct_layouts_match_the_reference_pods():
    pkg = fnx_gpu.package()
    assert C.sizeof(pkg.Job) == 4 * (2 + 2 * 16)          # kernels.hpp:18-23
    assert C.sizeof(pkg.BigJob) == 4 * (2 + 2 * 64)       # kernels.hpp:32-37 with PF_JOB 64
    assert pkg.Job.y.offset == 8 and pkg.Job.out.offset == 8 + 64


def test_bad_arguments_are_refused_with_a_message():
    pkg = fnx_gpu.package()
    lib = pkg.lib()
    buf = np.zeros(64, dtype=np.float32).ctypes.data
    assert lib.fnx_quantize_q8_1(buf, buf, 33, 1, None) != 0
    assert b"32" in lib.fnx_last_error()
    assert lib.fnx_quantize_q8_1(None, buf, 32, 1, None) != 0
    assert lib.fnx_gemv_f32(buf, buf, buf, 4, 100, 1, None) != 0
    assert lib.fnx_gemv_f32(buf, buf, buf, 4, 256, 0, None) != 0 and b"T out of range" in lib.fnx_last_error()
    bad = pkg.DW(buf, 14, 2048, 16, 880, None)              # Q6_K experts are not handled
    assert lib.fnx_moe_gate_up(C.byref(bad), 0, buf, None, 10, buf, buf, 10, None) != 0
    assert b"IQ3_S" in lib.fnx_last_error()
    bad = pkg.DW(buf, 8, 2048, 16, 880, None)               # Q8_0 rows of 2048 values take 2,176 bytes
    assert lib.fnx_moe_gate_up(C.byref(bad), 0, buf, None, 10, buf, buf, 10, None) != 0 and b"row_bytes" in lib.fnx_last_error()
    bad = pkg.DW(buf, pkg.T_IQ3_S, 2048, 16, 881, None)     # row_bytes must be n_in / 256 * 110
    assert lib.fnx_mmvq(C.byref(bad), 0, buf, None, 1, buf, buf, 16, None) != 0
    assert lib.fnx_route(buf, 8, 1, 2000, 10, buf, buf, buf, buf, buf, None) != 0
    assert lib.fnx_argmax(buf, 0, 1, 0, buf, buf, buf, buf, None) != 0
    assert lib.fnx_q8s_tile(buf, buf, 16, 256, None) != 0 and b"two buffers" in lib.fnx_last_error()
    assert lib.fnx_q8s_tile_bytes(17, 256) == 32 * 256 and lib.fnx_q8s_tile_bytes(16, 100) == 0
    # a cache whose capacity ends inside a block of eight positions would be read past its end by the attention's V fetches
    assert lib.fnx_attn(buf, buf, buf, buf, 16, 2, buf, 1, 100, buf, None) != 0 and b"multiple of 8" in lib.fnx_last_error()
    assert lib.fnx_attn(buf, buf, buf, buf, 16, 2, buf, 1, 4, buf, None) != 0 and b"multiple of 8" in lib.fnx_last_error()


def test_the_grouped_gemm_takes_tile16_in_its_two_forms_only():
    """tile16 matrices are the prompt path's stacked gate|up (which leaves h) and rows of 512 columns; h alone comes from
    tile16 only: everything else is refused before a launch"""
    pkg = fnx_gpu.package()
    lib = pkg.lib()
    buf = np.zeros(64, dtype=np.float32).ctypes.data
    gu16, dn16_1024 = pkg.dw(buf, 2048, 1024, tile16=True), pkg.dw(buf, 1024, 2048, tile16=True)
    assert lib.fnx_moe_gate_up_mma(C.byref(gu16), 0, buf, buf, 4, buf, buf, None) != 0 and b"tile16" in lib.fnx_last_error()
    assert lib.fnx_moe_down_mma(C.byref(dn16_1024), 0, buf, buf, 4, buf, buf, None) != 0 and b"tile16" in lib.fnx_last_error()
    for packed in (False, True):
        w = pkg.dw(buf, 2048, 1024, packed=packed)
        assert lib.fnx_moe_gate_up_h16_mma(C.byref(w), 0, buf, buf, 4, buf, buf, None) != 0 and b"h alone" in lib.fnx_last_error()
        # the q8_1 family's jobs of up to 64 rows: tile16 only
        assert lib.fnx_moe_gate_up_big(C.byref(w), 0, buf, buf, 4, buf, buf, None) != 0 and b"tile16" in lib.fnx_last_error()
        assert lib.fnx_moe_down_big(C.byref(w), 0, buf, buf, 4, buf, buf, None) != 0 and b"tile16" in lib.fnx_last_error()
    assert lib.fnx_moe_gate_up_big(C.byref(gu16), 0, buf, buf, 5000, buf, buf, None) != 0 and b"4096" in lib.fnx_last_error()


def test_a_layer_wider_than_the_pair_buffer_is_refused():
    """operator by operator (raw ggml blocks) the pairs' q8_1 rows of h go through the library's pair buffer of rows of at most
    1024 values: a wider expert is refused before anything is launched"""
    pkg = fnx_gpu.package()
    lib = pkg.lib()
    buf = np.zeros(64, dtype=np.float32).ctypes.data
    n, ff, nexp, topk = 2048, 2048, 32, 10
    gu, down = pkg.dw(buf, n, 2 * ff), pkg.dw(buf, ff, n)
    L = pkg.MoeLayer(n, ff, nexp, topk, buf, 0, gu, 0, down, 0, gu, down)
    ws = pkg.MoeWs(*([buf] * len(pkg.MoeWs._fields_)))
    assert lib.fnx_moe_verify_layer(C.byref(L), buf, 16, buf, C.byref(ws), None) != 0
    assert b"pair buffer" in lib.fnx_last_error()


def test_host_lookup_and_accept_match_the_oracle(oracle):
    lib = fnx_gpu.package().lib()
    rng = np.random.default_rng(31)
    for key_n in (2, 3, 4):
        for _ in range(200):
            n = int(rng.integers(0, 50))
            ctx = rng.integers(0, 4, size=n).astype(np.int32)
            lk, d1 = int(rng.integers(0, 16)), int(rng.integers(-1, 4))
            out = np.zeros(32, dtype=np.int32)
            match = C.c_int(-7)
            got = lib.fnx_lookup_drafts(ctx.ctypes.data if n else out.ctypes.data, n, key_n, lk, d1, out.ctypes.data, C.byref(match))
            want, wmatch = oracle.lookup_drafts(ctx, lk, d1, key_n)
            assert got == len(want) and list(out[:got]) == list(want) and match.value == wmatch
    for _ in range(200):
        R = int(rng.integers(1, 17))
        rows = rng.integers(0, 3, size=R).astype(np.int32)
        o = rng.integers(0, 3, size=R).astype(np.int32)
        assert lib.fnx_accept_greedy(rows.ctypes.data, o.ctypes.data, R) == oracle.accept_greedy(rows, o)
    assert lib.fnx_lookup_drafts(None, 3, 3, 3, 0, None, None) == -1
