"""Test-side helpers: import the package (its directory name is not a Python identifier), the package's host-side
harness over the C ABI under this module's names, and a numpy restatement of the unit64 layout to check the library's against."""
import ctypes as C
import importlib.util
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "qwen3.8-flash-next-2x-p100_amd")


def package():
    name = "fnx_mi355x_pkg"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, os.path.join(PKG_DIR, "__init__.py"), submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


_h = importlib.import_module(package().__name__ + ".harness")
random_iq3s, JOB_DTYPE, V_BLOCK, v_blocked, v_rows, pad4 = _h.random_iq3s, _h.JOB_DTYPE, _h.V_BLOCK, _h.v_blocked, _h.v_rows, _h.pad4
Dev, pack_moe_weights, DecoderDev, PfLayerDev, MoeLayerDev, SyntheticDecoder = (_h.Dev, _h.pack_moe_weights, _h.DecoderDev, _h.PfLayerDev,
                                                                                _h.MoeLayerDev, _h.SyntheticDecoder)


def pack_unit64(raw):
    """numpy restatement of the unit64 layout (written from the layout's description, independent of the kernel):
    per 64 sub-blocks (880 bytes): each sub-block's eight 13-bit indexes (sign nibble << 9 | high bit << 8 | code) as
    a 104-bit little-endian string split over plane A (bytes 0..7 of every sub-block, 512 bytes), plane B (bytes 8..11,
    256 bytes) and plane C (byte 12, 64 bytes); then the 32 scale bytes in order, then the 8 d halves."""
    raw = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 8, 110)      # units of 8 super-blocks
    nu = raw.shape[0]
    qs = raw[:, :, 2:66].reshape(nu, 8, 8, 8).astype(np.uint64)               # [unit][sb][ib][group]
    qh = raw[:, :, 66:74].reshape(nu, 8, 8, 1).astype(np.uint64)
    sg = raw[:, :, 74:106].reshape(nu, 8, 8, 4).astype(np.uint64)             # 4 sign bytes per sub-block
    g = np.arange(8, dtype=np.uint64)
    hb = (qh >> g) & np.uint64(1)
    nib = (np.repeat(sg, 2, axis=3) >> ((g & np.uint64(1)) * np.uint64(4))) & np.uint64(0xF)
    idx = qs | (hb << np.uint64(8)) | (nib << np.uint64(9))                    # [unit][sb][ib][8] 13-bit
    idx = idx.reshape(nu, 64, 8)
    out = np.zeros((nu, 880), dtype=np.uint8)
    bits = np.zeros((nu, 64, 104), dtype=np.uint8)
    for j in range(8):
        for b in range(13):
            bits[:, :, 13 * j + b] = (idx[:, :, j] >> np.uint64(b)) & np.uint64(1)
    chunks = np.packbits(bits.reshape(nu, 64, 13, 8), axis=3, bitorder="little").reshape(nu, 64, 13)
    out[:, 0:512] = chunks[:, :, 0:8].reshape(nu, 512)
    out[:, 512:768] = chunks[:, :, 8:12].reshape(nu, 256)
    out[:, 768:832] = chunks[:, :, 12]
    out[:, 832:864] = raw[:, :, 106:110].reshape(nu, 32)
    out[:, 864:880] = raw[:, :, 0:2].reshape(nu, 16)
    return out.reshape(-1)
