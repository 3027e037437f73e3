"""The library's GGUF reader and expert slicing (host code; no GPU): against the cases the reference's own reader test
holds (tools/gguf_test.cpp: one valid file, the metadata read back, nine malformed headers refused with a message that
names the tensor and the fault), against the reference's reader itself where oracle/_ref is built (the same files: the
same tensors, shapes, offsets, byte counts and bytes; the same files refused), and against numpy slicing for
expert_rows2 / expert_cols (model.cpp:722-741, 768-790)."""
import ctypes as C
import struct

import numpy as np
import pytest

import fnx_gpu
import gguf_files as gf


@pytest.fixture(scope="module")
def lib():
    return fnx_gpu.package().lib()


def describe(pkg, lib, g):
    out = {}
    for i in range(lib.fnx_gguf_count(g)):
        t = pkg.GgufTensor()
        assert lib.fnx_gguf_at(g, i, C.byref(t)) == 0
        out[t.name.decode()] = dict(type=t.type, n_dims=t.n_dims, ne=list(t.ne), nbytes=t.nbytes, shard=t.shard, offset=t.offset,
                                    row_bytes=lib.fnx_gguf_row_bytes(C.byref(t)), data=C.string_at(t.data, t.nbytes))
    return out


def one_f32(n_dims, ne, data_bytes, offset=0, keys=()):
    """tools/gguf_test.cpp make(): one F32 tensor "w" with the given dimensions, data_bytes of data section"""
    return gf.build([("w", gf.F32, ne, b"")], keys=keys, n_dims=n_dims, offsets=[offset], data_bytes=data_bytes)


def test_valid_file_and_metadata(lib, tmp_path):
    pkg = fnx_gpu.package()
    p = tmp_path / "valid.gguf"
    p.write_bytes(one_f32(2, [8, 3], 8 * 3 * 4))
    g = lib.fnx_gguf_open(str(p).encode())
    assert g, lib.fnx_last_error()
    t = describe(pkg, lib, g)["w"]
    assert (t["n_dims"], t["ne"], t["nbytes"], t["row_bytes"]) == (2, [8, 3, 1, 1], 96, 32)   # gguf_test.cpp "valid"
    lib.fnx_gguf_close(g)
    keys = [gf.kv("a.rope.scaling.type", gf.STR, "yarn"), gf.kv("a.rope.scaling.factor", gf.F32V, 4.0),
            gf.kv("a.rope.scaling.original_context_length", gf.U32, 32768), gf.kv("tokenizer.ggml.tokens", gf.ARR, ["a", "bc"], gf.STR),
            gf.kv("a.sections", gf.ARR, [3, 4, 5], gf.I32V), gf.kv("a.flag", gf.BOOL, 1), gf.kv("a.big", gf.I64, -(2**40)), gf.kv("a.d", gf.F64, 0.25),
            gf.kv("a.floats", gf.ARR, [1.0, 2.0], gf.F32V)]
    p.write_bytes(one_f32(2, [8, 3], 96, keys=keys))
    g = lib.fnx_gguf_open(str(p).encode())
    assert g, lib.fnx_last_error()
    v, d = C.c_int64(), C.c_double()
    assert lib.fnx_gguf_str(g, b"a.rope.scaling.type") == b"yarn"                                # gguf_test.cpp "keys"
    assert lib.fnx_gguf_num(g, b"a.rope.scaling.factor", C.byref(d)) == 0 and d.value == 4.0
    assert lib.fnx_gguf_num(g, b"a.rope.scaling.original_context_length", C.byref(d)) == 0 and d.value == 32768.0
    assert lib.fnx_gguf_int(g, b"a.rope.scaling.original_context_length", C.byref(v)) == 0 and v.value == 32768
    assert lib.fnx_gguf_key_type(g, b"a.rope.scaling.alpha") == -1 and lib.fnx_gguf_key_type(g, b"tokenizer.ggml.tokens") == gf.ARR
    assert lib.fnx_gguf_int(g, b"a.big", C.byref(v)) == 0 and v.value == -(2**40)
    assert lib.fnx_gguf_num(g, b"a.d", C.byref(d)) == 0 and d.value == 0.25
    assert lib.fnx_gguf_int(g, b"a.rope.scaling.factor", C.byref(v)) != 0 and lib.fnx_gguf_str(g, b"a.flag") is None
    assert describe(pkg, lib, g)["w"]["nbytes"] == 96
    lib.fnx_gguf_close(g)


MALFORMED = [   # tools/gguf_test.cpp expect_refused cases: tag, file, what the message must hold beside "tensor w"
    ("dims0", lambda: one_f32(0, [], 64), "0 dimensions"),
    ("dims5", lambda: one_f32(5, [1, 1, 1, 1, 1], 64), "5 dimensions"),
    ("dims_huge", lambda: one_f32(0xffffffff, [1], 64), "4294967295 dimensions"),
    ("ne_zero", lambda: one_f32(2, [8, 0], 64), "size 0 in dimension 1"),
    ("ne_negative", lambda: one_f32(1, [2**64 - 1], 64), "in dimension 0"),
    ("count_overflow", lambda: one_f32(2, [1 << 32, 1 << 32], 64), "element count overflows"),
    ("bytes_overflow", lambda: one_f32(1, [1 << 62], 64), "runs past the end"),
    ("past_end", lambda: one_f32(2, [8, 3], 95), "runs past the end"),
    ("offset_wraps", lambda: one_f32(1, [8], 64, offset=2**64 - 1 - 8), "runs past the end"),
]


@pytest.mark.parametrize("tag,make,want", MALFORMED, ids=[m[0] for m in MALFORMED])
def test_malformed_headers_are_refused_by_name(lib, tmp_path, tag, make, want):
    p = tmp_path / f"{tag}.gguf"
    p.write_bytes(make())
    assert not lib.fnx_gguf_open(str(p).encode())
    msg = lib.fnx_last_error().decode()
    assert "tensor w" in msg and want in msg, msg


def test_other_refusals(lib, tmp_path):
    p = tmp_path / "x.gguf"
    p.write_bytes(b"GGUX" + b"\0" * 60)
    assert not lib.fnx_gguf_open(str(p).encode()) and b"bad magic" in lib.fnx_last_error()
    p.write_bytes(gf.build([("w", gf.F32, [8], b"\0" * 32)])[:30])
    assert not lib.fnx_gguf_open(str(p).encode()) and b"truncated" in lib.fnx_last_error()
    p.write_bytes(gf.build([("w", 77, [8], b"\0" * 32)]))
    assert not lib.fnx_gguf_open(str(p).encode()) and b"unknown ggml type 77" in lib.fnx_last_error()
    p.write_bytes(gf.build([("w", gf.F32, [8], b"\0" * 32)], keys=[gf.kv("general.alignment", gf.U32, 0)]))
    assert not lib.fnx_gguf_open(str(p).encode()) and b"general.alignment" in lib.fnx_last_error()
    assert not lib.fnx_gguf_open(str(tmp_path / "missing.gguf").encode()) and b"cannot open" in lib.fnx_last_error()


def sample_files(tmp_path):
    """files with several tensors of several types, an alignment of their own, and a set of two shards"""
    rng = np.random.default_rng(5)
    raw = lambda n: rng.integers(0, 256, n, dtype=np.uint8).tobytes()
    a = gf.write(tmp_path / "several.gguf", [("tok.weight", gf.F16, [64, 10], raw(64 * 10 * 2)), ("blk.0.w", gf.Q8_0, [64, 6], raw(2 * 6 * 34)),
                                             ("blk.0.e", gf.IQ3_S, [512, 4, 3], raw(2 * 4 * 3 * 110)), ("v", gf.F32, [5], raw(20)),
                                             ("i", gf.I32, [3, 2], raw(24))],
                 keys=[gf.kv("general.architecture", gf.STR, "a"), gf.kv("a.expert_used_count", gf.U32, 10)])
    b = gf.write(tmp_path / "aligned.gguf", [("p", gf.F32, [3], raw(12)), ("q", gf.BF16, [7, 2], raw(28))],
                 keys=[gf.kv("general.alignment", gf.U32, 64)], alignment=64)
    s1 = gf.write(tmp_path / "m-00001-of-00002.gguf", [("one", gf.F32, [4], raw(16))], keys=[gf.kv("general.name", gf.STR, "first")])
    gf.write(tmp_path / "m-00002-of-00002.gguf", [("two", gf.F32, [2, 2], raw(16))], keys=[gf.kv("general.name", gf.STR, "second")])
    return [a, b, s1]


def test_several_tensors_alignment_and_shards(lib, tmp_path):
    pkg = fnx_gpu.package()
    a, b, s1 = sample_files(tmp_path)
    g = lib.fnx_gguf_open(a.encode())
    d = describe(pkg, lib, g)
    assert list(d) == sorted(d) and set(d) == {"tok.weight", "blk.0.w", "blk.0.e", "v", "i"}
    assert d["blk.0.e"]["ne"] == [512, 4, 3, 1] and d["blk.0.e"]["nbytes"] == 2 * 4 * 3 * 110 and d["blk.0.e"]["row_bytes"] == 220
    assert d["blk.0.w"]["row_bytes"] == 68 and all(v["offset"] % 32 == 0 for v in d.values())
    blob = open(a, "rb").read()
    assert all(blob[v["offset"]:v["offset"] + v["nbytes"]] == v["data"] for v in d.values())
    t = pkg.GgufTensor()
    assert lib.fnx_gguf_find(g, b"v", C.byref(t)) == 0 and t.nbytes == 20
    assert lib.fnx_gguf_find(g, b"nope", C.byref(t)) != 0 and b"no tensor nope" in lib.fnx_last_error()
    lib.fnx_gguf_close(g)
    g = lib.fnx_gguf_open(b.encode())
    d = describe(pkg, lib, g)
    assert all(v["offset"] % 64 == 0 for v in d.values()) and d["q"]["nbytes"] == 28
    lib.fnx_gguf_close(g)
    g = lib.fnx_gguf_open(s1.encode())
    d = describe(pkg, lib, g)
    assert lib.fnx_gguf_shards(g) == 2 and d["one"]["shard"] == 0 and d["two"]["shard"] == 1 and d["two"]["ne"] == [2, 2, 1, 1]
    assert lib.fnx_gguf_str(g, b"general.name") == b"first", "metadata is the first shard's"
    lib.fnx_gguf_close(g)


def test_reader_agrees_with_the_reference_reader(lib, ref, tmp_path):
    if not hasattr(ref, "fnx_ref_gguf_open"):
        pytest.skip("oracle/_ref was built without the reference's GGUF reader")
    pkg = fnx_gpu.package()
    err = C.create_string_buffer(512)
    for path in sample_files(tmp_path):
        g, r = lib.fnx_gguf_open(path.encode()), ref.fnx_ref_gguf_open(path.encode(), err, 512)
        assert g and r, (lib.fnx_last_error(), err.value)
        mine = describe(pkg, lib, g)
        assert ref.fnx_ref_gguf_count(r) == len(mine) and ref.fnx_ref_gguf_shards(r) == lib.fnx_gguf_shards(g)
        name, info = C.create_string_buffer(256), (C.c_int64 * 10)()
        for i, (k, v) in enumerate(mine.items()):   # both in name order
            assert ref.fnx_ref_gguf_tensor(r, i, name, 256, info) == 0 and name.value.decode() == k
            if info[7] < 0:
                continue   # re-quantised by the reference at load (no longer the file's bytes)
            assert list(info) == [v["type"], v["n_dims"]] + v["ne"] + [v["nbytes"], v["shard"], v["offset"], v["row_bytes"]], k
            assert C.string_at(ref.fnx_ref_gguf_data(r, k.encode()), v["nbytes"]) == v["data"]
        for key in (b"general.architecture", b"general.alignment", b"general.name", b"nope"):
            assert (lib.fnx_gguf_key_type(g, key) >= 0) == bool(ref.fnx_ref_gguf_has_key(r, key))
        a, b = C.c_double(), C.c_double()
        if lib.fnx_gguf_num(g, b"a.expert_used_count", C.byref(a)) == 0:
            assert ref.fnx_ref_gguf_num(r, b"a.expert_used_count", C.byref(b)) == 0 and a.value == b.value == 10
        lib.fnx_gguf_close(g)
        ref.fnx_ref_gguf_close(r)
    for tag, make, want in MALFORMED:
        p = tmp_path / f"{tag}.gguf"
        p.write_bytes(make())
        assert not lib.fnx_gguf_open(str(p).encode())
        assert not ref.fnx_ref_gguf_open(str(p).encode(), err, 512), tag
        assert want in err.value.decode() and want in lib.fnx_last_error().decode(), "both name the same fault"


def test_expert_slices_equal_numpy(lib, tmp_path):
    pkg = fnx_gpu.package()
    rng = np.random.default_rng(9)
    n, ff_total, nexp = 512, 768, 5
    ts, a = gf.moe_layer_tensors(rng, 3, n, ff_total, nexp, fnx_gpu.random_iq3s)
    path = gf.write(tmp_path / "layer.gguf", ts, keys=[gf.kv("general.architecture", gf.STR, "q"), gf.kv("q.expert_used_count", gf.U32, 2)])
    g = lib.fnx_gguf_open(path.encode())
    assert g, lib.fnx_last_error()
    T = lambda name: (lambda t: (lib.fnx_gguf_find(g, f"blk.3.{name}".encode(), C.byref(t)), t)[1])(pkg.GgufTensor())
    gate, up, down = T("ffn_gate_exps.weight"), T("ffn_up_exps.weight"), T("ffn_down_exps.weight")
    for r0, r1 in ((0, 768), (256, 512), (512, 768), (10, 11)):
        w, stride, nbytes = pkg.DW(), C.c_size_t(), C.c_size_t()
        assert lib.fnx_gguf_expert_rows2(C.byref(gate), C.byref(up), r0, r1, None, 0, C.byref(w), C.byref(stride), C.byref(nbytes)) == 0
        assert (w.n_in, w.n_out, w.row_bytes, w.type, stride.value) == (n, 2 * (r1 - r0), 220, 21, 2 * (r1 - r0) * 220)
        buf = np.zeros(nbytes.value, dtype=np.uint8)
        assert lib.fnx_gguf_expert_rows2(C.byref(gate), C.byref(up), r0, r1, buf.ctypes.data, buf.size, C.byref(w), C.byref(stride), None) == 0
        assert np.array_equal(buf, gf.slice_rows2(a["gate"], a["up"], n, ff_total, nexp, r0, r1))
    for c0, c1 in ((0, 768), (256, 512), (512, 768)):
        w, stride, nbytes = pkg.DW(), C.c_size_t(), C.c_size_t()
        assert lib.fnx_gguf_expert_cols(C.byref(down), c0, c1, None, 0, C.byref(w), C.byref(stride), C.byref(nbytes)) == 0
        assert (w.n_in, w.n_out, w.row_bytes, stride.value) == (c1 - c0, n, (c1 - c0) // 256 * 110, n * (c1 - c0) // 256 * 110)
        buf = np.zeros(nbytes.value, dtype=np.uint8)
        assert lib.fnx_gguf_expert_cols(C.byref(down), c0, c1, buf.ctypes.data, buf.size, C.byref(w), C.byref(stride), None) == 0
        assert np.array_equal(buf, gf.slice_cols(a["down"], n, ff_total, nexp, c0, c1))
    small = np.zeros(16, dtype=np.uint8)
    assert lib.fnx_gguf_expert_rows2(C.byref(gate), C.byref(up), 0, 769, None, 0, None, None, None) != 0 and b"rows [0, 769)" in lib.fnx_last_error()
    assert lib.fnx_gguf_expert_rows2(C.byref(gate), C.byref(down), 0, 8, None, 0, None, None, None) != 0 and b"do not stack" in lib.fnx_last_error()
    assert lib.fnx_gguf_expert_rows2(C.byref(gate), C.byref(up), 0, 8, small.ctypes.data, 16, None, None, None) != 0 and b"buffer" in lib.fnx_last_error()
    assert lib.fnx_gguf_expert_cols(C.byref(down), 32, 256, None, 0, None, None, None) != 0 and b"blocks of 256" in lib.fnx_last_error()
    z = pkg.MoeBufs()
    assert lib.fnx_gguf_moe_layer_bytes(g, 3, 0, ff_total, C.byref(z)) == 0
    per = lambda rows, cols: rows * cols // 256 * 110
    assert (z.router_bytes, z.gu_bytes, z.down_bytes, z.sh_gu_bytes, z.sh_down_bytes) == ((nexp + 1) * n * 4, nexp * per(2 * ff_total, n), nexp * per(n, ff_total),
                                                                                         per(2 * ff_total, n), per(n, ff_total))
    assert lib.fnx_gguf_moe_layer_bytes(g, 4, 0, ff_total, C.byref(z)) != 0 and b"no tensor blk.4." in lib.fnx_last_error()
    lib.fnx_gguf_close(g)


def test_cut_and_corrupted_headers_never_read_out_of_bounds(lib, tmp_path):
    # a valid layer file cut short at many lengths and with random bytes of its header changed: refused with a message, or,
    # where the damage left a header that still adds up, every tensor's bytes can be read where the reader says they are
    pkg = fnx_gpu.package()
    rng = np.random.default_rng(17)
    ts, _ = gf.moe_layer_tensors(rng, 0, 512, 256, 3, fnx_gpu.random_iq3s)
    full = gf.build(ts, keys=[gf.kv("general.architecture", gf.STR, "q"), gf.kv("q.arr", gf.ARR, [1, 2, 3], gf.I32V),
                              gf.kv("q.names", gf.ARR, ["a", "bc"], gf.STR)])
    variants = [full[:cut] for cut in range(1, 900, 9)]
    for _ in range(120):
        b = bytearray(full)
        for _ in range(3):
            b[int(rng.integers(4, 800))] = int(rng.integers(0, 256))
        variants.append(bytes(b))
    p = tmp_path / "v.gguf"
    refused = 0
    for v in variants:
        p.write_bytes(v)
        g = lib.fnx_gguf_open(str(p).encode())
        if not g:
            assert lib.fnx_last_error().startswith(b"gguf:")
            refused += 1
            continue
        for i in range(lib.fnx_gguf_count(g)):
            t = pkg.GgufTensor()
            assert lib.fnx_gguf_at(g, i, C.byref(t)) == 0
            assert len(C.string_at(t.data, t.nbytes)) == t.nbytes and t.offset + t.nbytes <= len(v)
        z = pkg.MoeBufs()
        lib.fnx_gguf_moe_layer_bytes(g, 0, 0, 256, C.byref(z))   # either answer; never a fault
        lib.fnx_gguf_close(g)
    assert refused >= 150
