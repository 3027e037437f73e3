#!/usr/bin/env python3
"""Writes tests/golden/verify_path.npz: small input/output vectors of the verify path, made with the CPU oracle after
it was pinned (tests/test_oracle_*.py). Inputs come from numpy's PCG64 with the seeds below; IQ3_S bytes come from the
oracle's own encoder (any valid encoder will do: parity is defined from the quantised bytes onward).

Run from the repo root: python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib  # noqa: E402


def main():
    o = oracle_lib.Oracle()
    out = {}
    rng = np.random.default_rng(20261125)
    # two IQ3_S super-blocks and their 512 decoded weights
    w2 = (rng.standard_normal(512) * 0.02).astype(np.float32)
    out["blocks2"] = o.iq3s_quantize(w2)
    out["blocks2_decoded"] = o.iq3s_dequant(out["blocks2"])
    # a 64 x 512 matrix, 3 activation rows: q8_1 bytes and mat-vec outputs
    W = (rng.standard_normal(64 * 512) * 0.02).astype(np.float32)
    out["w64x512"] = o.iq3s_quantize(W)
    out["x3"] = rng.standard_normal((3, 512)).astype(np.float32)
    out["x3_q8_1"] = o.quantize_q8_1(out["x3"])
    out["y3"] = o.gemv_iq3s(out["w64x512"], 64, 512, out["x3"])
    # routing: 4 rows of 512 logits (+ the shared gate's), with a run of ties
    logits = rng.standard_normal((4, 513)).astype(np.float32)
    logits[2, 100:104] = logits[2].max() + 1.0
    out["logits"] = logits
    topi, topw = o.topk_logits(logits, 512, 10)
    out["topi"], out["topw"] = topi, topw
    gu, dn = o.jobs(topi)
    out["jobs_gu"], out["jobs_dn"] = gu.view(np.uint8).reshape(len(gu), -1), dn.view(np.uint8).reshape(len(dn), -1)
    # router mat-vec in the fixed order
    Wr = (rng.standard_normal((13, 512)) * 0.02).astype(np.float32)
    out["router_w"], out["router_x"] = Wr, out["x3"]
    out["router_y"] = o.gemv_f32(Wr, out["x3"])
    # swiglu -> q8_1, combine
    g = rng.standard_normal((5, 64)).astype(np.float32) * 2
    out["swiglu_gu"] = g
    out["swiglu_hq"] = o.swiglu_stacked_q8_1(g, 32)
    part = rng.standard_normal((20, 32)).astype(np.float32)
    tw = rng.random((2, 10)).astype(np.float32)
    sh = rng.standard_normal((2, 32)).astype(np.float32)
    shl = rng.standard_normal(2).astype(np.float32)
    out["comb_part"], out["comb_topw"], out["comb_sh"], out["comb_shl"] = part, tw, sh, shl
    out["comb_out"] = o.moe_combine(part, tw, sh, shl)
    # argmax: 2 x 1000 with ties and one NaN
    am = rng.standard_normal((2, 1000)).astype(np.float32)
    am[0, [7, 300]] = 8.0
    am[1, 5] = np.nan
    out["argmax_logits"] = am
    bv, bi, err = o.argmax(am, v0=11)
    out["argmax_v"], out["argmax_i"], out["argmax_err"] = bv, bi, np.array([err], dtype=np.uint32)
    # lookup: 20 small contexts (flattened with offsets), lk, d1 -> drafts, match
    ctxs, offs, params, drafts, doffs = [], [0], [], [], [0]
    for case in range(20):
        n = int(rng.integers(3, 40))
        c = rng.integers(0, 4, size=n).astype(np.int32)
        lk, d1 = int(rng.integers(0, 16)), int(rng.integers(-1, 4))
        d, m = o.lookup_drafts(c, lk, d1)
        ctxs.append(c)
        offs.append(offs[-1] + n)
        params.append((lk, d1, m))
        drafts.append(d)
        doffs.append(doffs[-1] + len(d))
    out["lk_ctx"], out["lk_off"] = np.concatenate(ctxs), np.array(offs, dtype=np.int32)
    out["lk_params"] = np.array(params, dtype=np.int32)
    out["lk_drafts"] = np.concatenate(drafts).astype(np.int32) if doffs[-1] else np.zeros(0, dtype=np.int32)
    out["lk_doff"] = np.array(doffs, dtype=np.int32)
    # acceptance: 12 windows
    rows = rng.integers(0, 3, size=(12, 16)).astype(np.int32)
    pick = rng.integers(0, 3, size=(12, 16)).astype(np.int32)
    out["acc_rows"], out["acc_o"] = rows, pick
    out["acc_n"] = np.array([o.accept_greedy(rows[i], pick[i]) for i in range(12)], dtype=np.int32)
    np.savez_compressed(os.path.join(HERE, "verify_path.npz"), **out)
    print("wrote", os.path.join(HERE, "verify_path.npz"), sum(v.nbytes for v in out.values()), "bytes of arrays")


if __name__ == "__main__":
    main()
