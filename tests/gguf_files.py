"""Writes GGUF version 3 files for the tests, from the format's public description: the magic 'GGUF', the version, the
tensor and key counts, the keys (name, value type, value), the tensor infos (name, dimensions, ggml type, offset into
the data section) and the data section, which starts at the next multiple of general.alignment (32 when not given)."""
import struct

import numpy as np

F32, F16, Q8_0, IQ3_S, I32, BF16 = 0, 1, 8, 21, 26, 30
U8, I8, U16, I16, U32, I32V, F32V, BOOL, STR, ARR, U64, I64, F64 = range(13)   # metadata value types
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32V: "<i", F32V: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}


def _text(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def kv(key, vtype, value, elem=None):
    """one metadata entry; for ARR give the element type in elem"""
    out = _text(key) + struct.pack("<I", vtype)
    if vtype == STR:
        return out + _text(value)
    if vtype == ARR:
        out += struct.pack("<IQ", elem, len(value))
        return out + b"".join(_text(v) if elem == STR else struct.pack(_FMT[elem], v) for v in value)
    return out + struct.pack(_FMT[vtype], value)


def build(tensors, keys=(), alignment=32, version=3, n_dims=None, offsets=None, data_bytes=None):
    """tensors: (name, ggml type, ne list, bytes-like data). Overrides for malformed files: n_dims (of every tensor),
    offsets (per tensor), data_bytes (length of the data section instead of what the tensors need)."""
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(keys)) + b"".join(keys)
    infos, blob = b"", b""
    for i, (name, ttype, ne, data) in enumerate(tensors):
        data = bytes(data)
        off = len(blob) if offsets is None else offsets[i]
        infos += _text(name) + struct.pack("<I", len(ne) if n_dims is None else n_dims) + b"".join(struct.pack("<Q", int(v) & (2**64 - 1)) for v in ne)
        infos += struct.pack("<IQ", ttype, off)
        blob += data + b"\0" * (-len(data) % alignment)
    head += infos
    head += b"\0" * (-len(head) % alignment)
    if data_bytes is not None:
        blob = (blob + b"\0" * data_bytes)[:data_bytes]
    return head + blob


def write(path, *args, **kw):
    with open(path, "wb") as f:
        f.write(build(*args, **kw))
    return str(path)


def moe_layer_tensors(rng, layer, n, ff_total, nexp, random_iq3s, router_type=F32):
    """a layer's MoE tensors as the model files name and shape them (ne[0] = a row's values): returns the GGUF tensor
    list and the arrays by short name"""
    nb = lambda rows, cols: rows * cols // 256
    a = dict(gate=random_iq3s(rng, nexp * nb(ff_total, n)), up=random_iq3s(rng, nexp * nb(ff_total, n)), down=random_iq3s(rng, nexp * nb(n, ff_total)),
             sh_gate=random_iq3s(rng, nb(ff_total, n)), sh_up=random_iq3s(rng, nb(ff_total, n)), sh_down=random_iq3s(rng, nb(n, ff_total)),
             router=(rng.standard_normal((nexp, n)) * 0.05).astype(np.float32), sh_router=(rng.standard_normal((1, n)) * 0.05).astype(np.float32))
    if router_type == BF16:   # values that bf16 holds exactly
        for k in ("router", "sh_router"):
            a[k] = (a[k].view(np.uint32) & 0xFFFF0000).view(np.float32)
    rt = (lambda x: x.tobytes()) if router_type == F32 else (lambda x: (x.view(np.uint32) >> 16).astype(np.uint16).tobytes())
    b = f"blk.{layer}."
    ts = [(b + "ffn_gate_inp.weight", router_type, [n, nexp], rt(a["router"])), (b + "ffn_gate_inp_shexp.weight", router_type, [n, 1], rt(a["sh_router"])),
          (b + "ffn_gate_exps.weight", IQ3_S, [n, ff_total, nexp], a["gate"]), (b + "ffn_up_exps.weight", IQ3_S, [n, ff_total, nexp], a["up"]),
          (b + "ffn_down_exps.weight", IQ3_S, [ff_total, n, nexp], a["down"]), (b + "ffn_gate_shexp.weight", IQ3_S, [n, ff_total], a["sh_gate"]),
          (b + "ffn_up_shexp.weight", IQ3_S, [n, ff_total], a["sh_up"]), (b + "ffn_down_shexp.weight", IQ3_S, [ff_total, n], a["sh_down"])]
    return ts, a


def slice_rows2(gate, up, n, ff_total, nexp, r0, r1):
    """model.cpp:722-741: per expert, rows [r0, r1) of gate then of up"""
    rb = n // 256 * 110
    g, u = gate.reshape(nexp, ff_total, rb), up.reshape(nexp, ff_total, rb)
    return np.concatenate([g[:, r0:r1], u[:, r0:r1]], axis=1).reshape(-1)


def slice_cols(down, n, ff_total, nexp, c0, c1):
    """model.cpp:768-790: per expert, every row's columns [c0, c1) (whole 256-value blocks)"""
    d = down.reshape(nexp, n, ff_total // 256, 110)
    return np.ascontiguousarray(d[:, :, c0 // 256:c1 // 256]).reshape(-1)
