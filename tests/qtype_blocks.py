"""Random blocks of the other expert types (any byte pattern is a valid block once the f16 scales are finite) and numpy
restatements of their decoders, written from the types' published layouts."""
import numpy as np

Q4_0, Q5_1, Q8_0, Q4_K, Q5_K, IQ4_NL, IQ4_XS = 2, 7, 8, 12, 13, 20, 23
SHAPE = {Q4_0: (32, 18), Q5_1: (32, 24), Q8_0: (32, 34), IQ4_NL: (32, 18), Q4_K: (256, 144), Q5_K: (256, 176), IQ4_XS: (256, 136)}
KV = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)


def random_blocks(rng, qtype, nblocks, dmax=0.02):
    values, nbytes = SHAPE[qtype]
    b = rng.integers(0, 256, size=(nblocks, nbytes), dtype=np.uint8)
    d = (rng.random(nblocks) * dmax + 1e-4).astype(np.float16)
    b[:, 0:2] = d.view(np.uint8).reshape(nblocks, 2)
    if qtype in (Q4_K, Q5_K, Q5_1):
        m = ((rng.random(nblocks) - (0.5 if qtype == Q5_1 else 0.0)) * dmax + 1e-4).astype(np.float16)
        b[:, 2:4] = m.view(np.uint8).reshape(nblocks, 2)
    return b.reshape(-1)


def scale_min(sc12):
    """the eight 6-bit (scale, min) pairs of a K-quant super-block's 12 bytes"""
    q = sc12.astype(np.int32)
    out = []
    for j in range(8):
        if j < 4:
            out.append((q[j] & 63, q[j + 4] & 63))
        else:
            out.append(((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4), (q[j + 4] >> 4) | ((q[j] >> 6) << 4)))
    return out


def np_dequant(qtype, blocks):
    values, nbytes = SHAPE[qtype]
    b = blocks.reshape(-1, nbytes)
    f32 = np.float32
    d = b[:, 0:2].copy().view(np.float16).astype(f32).reshape(-1)
    out = np.zeros((b.shape[0], values), f32)
    if qtype == Q8_0:
        out[:] = d[:, None] * b[:, 2:].view(np.int8).astype(f32)
    elif qtype == Q5_1:
        m = b[:, 2:4].copy().view(np.float16).astype(f32).reshape(-1)
        qh = b[:, 4:8].copy().view(np.uint32).reshape(-1).astype(np.int64)
        lo, hi = (b[:, 8:] & 0xF).astype(np.int64), (b[:, 8:] >> 4).astype(np.int64)
        j = np.arange(16)
        q = np.concatenate([lo | (((qh[:, None] >> j) & 1) << 4), hi | (((qh[:, None] >> (j + 16)) & 1) << 4)], axis=1)
        out[:] = d[:, None] * q.astype(f32) + m[:, None]
    elif qtype in (Q4_0, IQ4_NL):
        lo, hi = (b[:, 2:] & 0xF).astype(np.int32), (b[:, 2:] >> 4).astype(np.int32)
        q = np.concatenate([lo, hi], axis=1)
        out[:] = d[:, None] * ((q - 8).astype(f32) if qtype == Q4_0 else KV[q])
    elif qtype == IQ4_XS:
        sh = b[:, 2:4].copy().view(np.uint16).reshape(-1).astype(np.int32)
        for i in range(b.shape[0]):
            for ib in range(8):
                ls = ((int(b[i, 4 + ib // 2]) >> (4 * (ib % 2))) & 0xF) | (((sh[i] >> (2 * ib)) & 3) << 4)
                qs = b[i, 8 + 16 * ib:8 + 16 * ib + 16].astype(np.int32)
                dl = f32(d[i] * f32(ls - 32))
                out[i, 32 * ib:32 * ib + 16] = dl * KV[qs & 0xF]
                out[i, 32 * ib + 16:32 * ib + 32] = dl * KV[qs >> 4]
    else:
        mn = b[:, 2:4].copy().view(np.float16).astype(f32).reshape(-1)
        for i in range(b.shape[0]):
            sm = scale_min(b[i, 4:16])
            qh = b[i, 16:48].astype(np.int32)
            ql = b[i, (48 if qtype == Q5_K else 16):].astype(np.int32)
            for sb in range(8):
                src = ql[32 * (sb // 2):32 * (sb // 2) + 32]
                q = (src >> 4) if sb & 1 else (src & 0xF)
                if qtype == Q5_K:
                    q = q + (((qh >> sb) & 1) << 4)
                sc, m = sm[sb]
                out[i, 32 * sb:32 * sb + 32] = f32(d[i] * f32(sc)) * q.astype(f32) - f32(mn[i] * f32(m))
    return out.reshape(-1)
