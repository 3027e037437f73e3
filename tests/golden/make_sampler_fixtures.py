#!/usr/bin/env python3
"""Writes tests/golden/sampler_path.npz: small input/output vectors of the sampler (candidates, distribution, draw,
speculative sampling), made with the CPU oracle after it was pinned (tests/test_oracle_sampler.py). Inputs come from
numpy's PCG64 with the seed below.

Run from the repo root: python tests/golden/make_sampler_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib  # noqa: E402
from test_oracle_sampler import o_accept, o_dist, o_top_tokens  # noqa: E402


def main():
    o = oracle_lib.Oracle()
    out = {}
    rng = np.random.default_rng(20261126)
    # candidates: 3 rows of 3,000 logits from token 100 on, ties, a NaN, penalties on rows 0 and 2, a bias list on row 1
    x = rng.standard_normal((3, 3000)).astype(np.float32)
    x[0, rng.integers(0, 3000, 200)] = 2.0
    x[2, 77] = np.nan
    pen = [[(100 + int(t), int(c)) for t, c in zip(rng.choice(3000, 30, replace=False), rng.integers(1, 4, 30))], [],
           [(100 + int(t), 1) for t in np.argsort(-np.nan_to_num(x[2]))[:10]]]
    par = [(1.3, 0.1, 0.2), (1.0, 0.0, 0.0), (1.1, 0.0, 0.5)]
    bias = [[], [(100 + int(t), float(b)) for t, b in zip(rng.choice(3000, 6, replace=False), rng.standard_normal(6) * 6)], []]
    out["tk_logits"] = x
    out["tk_pen_tok"] = np.array([[t for t, _ in p] + [0] * (30 - len(p)) for p in pen], np.int32)
    out["tk_pen_cnt"] = np.array([[c for _, c in p] + [0] * (30 - len(p)) for p in pen], np.int32)
    out["tk_pen_n"] = np.array([len(p) for p in pen], np.int32)
    out["tk_par"] = np.array(par, np.float32)
    out["tk_bias_tok"] = np.array([t for b in bias for t, _ in b], np.int32)
    out["tk_bias_val"] = np.array([v for b in bias for _, v in b], np.float32)
    out["tk_bias_n"] = np.array([len(b) for b in bias], np.int32)
    ov, oi, L, err = o_top_tokens(o, x, v0=100, pen=pen, par=par, bias=bias)
    out["tk_out_v"], out["tk_out_i"], out["tk_logits_after"], out["tk_err"] = ov, oi, L, np.array([err], np.uint32)
    # distribution and speculative sampling over the first two rows' candidates
    kw = dict(temperature=0.8, top_p=0.9, min_p=0.02, top_k=40)
    out["sp_params"] = np.array([kw["temperature"], kw["top_p"], kw["min_p"], kw["top_k"]], np.float64)
    ids, p = o_dist(o, ov[0], oi[0], **kw)
    out["dist_ids"], out["dist_p"] = ids, p
    u = rng.random((8, 3))
    out["sp_u"] = u
    rows = np.array([5, int(oi[0, 1])], np.int32)   # the draft: row 0's second candidate, fixed (all of q on it)
    out["sp_rows"] = rows
    res = [o_accept(o, ov[:2], oi[:2], rows, u[i], **kw) for i in range(8)]
    out["sp_n"] = np.array([r[0] for r in res], np.int32)
    out["sp_o"] = np.array([r[1] + [-1] * (2 - len(r[1])) for r in res], np.int32)
    out["sp_used"] = np.array([r[2] for r in res], np.int32)
    np.savez_compressed(os.path.join(HERE, "sampler_path.npz"), **out)
    print("wrote", os.path.join(HERE, "sampler_path.npz"), {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
