"""Whole greedy decode rounds enqueued without the host in between (fnx_decode_round: verify -> accept -> commit -> draft
-> prompt lookup -> next window, the state in device words) against the host-driven round of tests/tiny_decoder.py
(session.cpp:530-679: the host waits for every step) on the device and on the CPU oracle, at hidden 2048 with unit64
experts (the one-launch window).

Bar: emitted tokens, drafts offered and tokens kept per round identical to the host-driven device loop (the same kernels
on the same rows: rows past the window's count are neither routed nor accepted); against the oracle: identical up to a
proven near-tie of two logits (test_gpu_decoder.same_until_near_tie), hidden rows and logits of a window as the chain
criteria of test_gpu_decoder say."""
import ctypes as C

import numpy as np
import pytest

import fnx_gpu
import tiny_decoder as td
from test_gpu_decoder import chain_close, same_until_near_tie

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


@pytest.fixture(scope="module")
def model(oracle):
    return td.TinyDecoder(oracle, seed=31, n=2048, nq=4, nkv=2, nlayers=2, vocab=1000, max_ctx=192, nexp=16, topk=4, ff=256)


@pytest.fixture(scope="module")
def cyclic_model(oracle):
    return td.TinyDecoder(oracle, seed=33, n=2048, nq=4, nkv=2, nlayers=1, vocab=256, max_ctx=512, nexp=16, topk=4, ff=256, cyclic=True)


def repeating_prompt(seed):
    rng = np.random.default_rng(seed)
    base = [int(t) for t in rng.integers(0, 1000, 12)]
    return base + base[:7] + [int(t) for t in rng.integers(0, 1000, 3)] + base[2:6]


class RoundDev:
    """a DecoderDev whose prompt has been read, plus the device words of fnx_decode_round"""

    def __init__(self, dev, model, prompt, speculate=True, lk=15, ctx_cap=512, chain=0):
        t, pkg = dev.torch, dev.pkg
        self.dev, self.d, self.prompt, self.pkg = dev, fnx_gpu.DecoderDev(dev, model), list(prompt), pkg
        d = self.d
        body, pos = self.prompt[:-1], 0
        for i in range(0, len(body), 16):   # the prompt pass of tiny_decoder.spec_generate
            w = body[i:i + 16]
            r = d.verify(w, pos)
            d.draft(r["hidden"], self.prompt[i + 1:i + 1 + len(w)], pos)
            pos += len(w)
        z = lambda n: dev.zeros(n, t.int32)
        self.ctx, self.state, self.rows, self.log, self.scratch = z(ctx_cap), z(pkg.RS_WORDS), z(16), z(2 * 64), z(16)
        self.ctx[:len(prompt)] = t.tensor(self.prompt, dtype=t.int32)
        self.state[pkg.RS_NCTX], self.state[pkg.RS_POS], self.state[pkg.RS_ROWS] = len(prompt), len(prompt) - 1, 1
        self.rows[0] = self.prompt[-1]
        self.chain_src = dev.zeros(model.cfg["n"], t.float32)
        self.R = pkg.Round(self.state.data_ptr(), self.rows.data_ptr(), self.ctx.data_ptr(), ctx_cap, self.log.data_ptr(), 64, int(speculate), 3, lk,
                           self.scratch.data_ptr(), chain, self.chain_src.data_ptr())

    def launch(self):
        d, dev = self.d, self.dev
        dev.ok(dev.lib.fnx_decode_round(C.byref(d.D), C.byref(d.M), C.byref(self.R), C.byref(d.ws), dev.st()))

    def result(self):
        self.dev.sync()
        st = self.state.cpu().numpy()
        pkg = self.pkg
        out = [int(v) for v in self.ctx.cpu().numpy()[len(self.prompt):st[pkg.RS_NCTX]]]
        log = self.log.cpu().numpy().reshape(-1, 2)[:st[pkg.RS_ROUNDS]]
        return out, [(int(a), int(b)) for a, b in log], st


def host_loop(dev, model, prompt, max_new, speculate=True, K=1, lk=15):
    def lookup_dev(ctx, lk, d1):
        return dev.lookup(np.asarray(ctx, dtype=np.int32), lk, d1)

    return td.spec_generate(fnx_gpu.DecoderDev(dev, model), lookup_dev, lambda r, o: dev.accept(r, o), prompt, max_new, K=K, lk=lk,
                            speculate=speculate)


def test_verify_window_at_hidden_2048_matches_oracle(dev, oracle, model):
    # the decoder over the one-launch window, which the rounds below use
    o, d = td.OracleSession(model), fnx_gpu.DecoderDev(dev, model)
    pos = 0
    for toks in ([3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7, 9, 3], [2, 7, 18], [281]):
        print(f"case decoder_verify n=2048 T={len(toks)} pos={pos}", flush=True)
        a, b = o.verify(toks, pos), d.verify(toks, pos)
        assert b["err"] == 0
        assert np.array_equal(a["best"], b["best"])
        chain_close(b["hidden"], a["hidden"], pos == 0)
        chain_close(b["logits"], a["logits"], pos == 0)
        nxt = toks[1:] + [int(a["best"][-1])]
        da, db = o.draft(a["hidden"], nxt, pos), d.draft(a["hidden"], nxt, pos)
        assert np.array_equal(da["best"], db["best"])
        chain_close(db["logits"], da["logits"], pos == 0)
        pos += len(toks)


@pytest.mark.parametrize("which,speculate", [("random", True), ("random", False), ("cyclic", True)])
def test_rounds_without_the_host_equal_the_host_driven_rounds(dev, oracle, model, cyclic_model, which, speculate):
    # random weights: the draft layer's pick is never right, so every round offers one draft and keeps one token;
    # the cyclic model: the lookup fires and whole windows of drafts are kept
    model = cyclic_model if which == "cyclic" else model
    prompt = [t % model.cfg["vocab"] for t in repeating_prompt(12)]
    r = RoundDev(dev, model, prompt, speculate=speculate)
    # rows that do not count must stay finite whatever the scratch holds (their attention output is zeros, not what the
    # q8_1 buffer happened to hold: bytes of ones read as NaN scales), or the head's finiteness check would fire
    r.d.b["xq"].fill_(0xFF)
    r.d.mb["xq"].fill_(0xFF)
    nrounds = 18 if which == "cyclic" else 14
    print(f"case decode_round eager model={which} speculate={speculate} rounds={nrounds}", flush=True)
    for _ in range(nrounds):
        r.launch()
    out, log, st = r.result()
    print("rounds", log, flush=True)
    assert st[dev.pkg.RS_STOP] == 0 and st[dev.pkg.RS_ROUNDS] == nrounds and len(out) == sum(k for _, k in log)
    assert int(r.d.b["err"].item()) == 0
    out_h, rounds_h = host_loop(dev, model, prompt, len(out), speculate=speculate)
    assert out == out_h, "the same tokens as the loop that waits for every step"
    assert log == rounds_h, "and the same drafts offered and tokens kept, round by round"
    if which == "cyclic":
        assert max(k for _, k in log) > 4 and max(dr for dr, _ in log) > 4, "the lookup fired and drafts were kept"
    if speculate:
        out_o, _ = td.spec_generate(td.OracleSession(model), lambda c, lk, d1: oracle.lookup_drafts(np.asarray(c, dtype=np.int32), lk, d1),
                                    lambda rw, o: oracle.accept_greedy(rw, o), prompt, len(out), K=1)
        same = same_until_near_tie(oracle, model, prompt, out, out_o)
        assert same >= 8
    else:
        assert all(entry == (0, 1) for entry in log)


@pytest.mark.parametrize("which,K,lk", [("random", 3, 15), ("cyclic", 3, 15), ("cyclic", 4, 0)])
def test_rounds_with_an_mtp_chain_equal_the_host_driven_rounds(dev, oracle, model, cyclic_model, which, K, lk):
    # session.cpp:666-678: when the lookup finds nothing, K - 1 more drafts from the draft layer's own rows. Random
    # weights: every round offers K drafts and keeps one token; the cyclic model with the lookup: most rounds take the
    # lookup's drafts and the chain's launches leave on the device word; without the lookup (lk = 0): every round runs the
    # chain, and its drafts are right
    model = cyclic_model if which == "cyclic" else model
    prompt = [t % model.cfg["vocab"] for t in repeating_prompt(12)]
    r = RoundDev(dev, model, prompt, lk=lk, chain=K)
    nrounds = 12
    print(f"case decode_round chain model={which} K={K} lk={lk} rounds={nrounds}", flush=True)
    for _ in range(nrounds):
        r.launch()
    out, log, st = r.result()
    print("rounds", log, flush=True)
    assert st[dev.pkg.RS_STOP] == 0 and st[dev.pkg.RS_ROUNDS] == nrounds and len(out) == sum(k for _, k in log)
    assert int(r.d.b["err"].item()) == 0
    out_h, rounds_h = host_loop(dev, model, prompt, len(out), K=K, lk=lk)
    assert out == out_h, "the same tokens as the loop that waits for every step"
    assert log == rounds_h, "and the same drafts offered and tokens kept, round by round"
    if which == "random":
        assert all(dr == K for dr, _ in log[1:]), "every round after the first offers the whole chain"
    elif lk == 0:
        assert all(dr == K for dr, _ in log[1:]) and max(k for _, k in log) > 2, "the chain's drafts were kept"
    else:
        assert max(dr for dr, _ in log) > K, "the lookup fired on some rounds"
    # fnx_run.cpp:1198-1238: whatever is drafted, the tokens are those of plain greedy decoding
    plain = RoundDev(dev, model, prompt, speculate=False)
    for _ in range(len(out)):
        plain.launch()
    out_p, _, _ = plain.result()
    assert out_p[:len(out)] == out
    out_o, _ = td.spec_generate(td.OracleSession(model), lambda c, lk_, d1: oracle.lookup_drafts(np.asarray(c, dtype=np.int32), lk_, d1),
                                lambda rw, o: oracle.accept_greedy(rw, o), prompt, len(out), K=K, lk=lk)
    assert same_until_near_tie(oracle, model, prompt, out, out_o) >= min(8, len(out))


@pytest.mark.parametrize("chain,lk", [(0, 15), (3, 15), (3, 0)])
def test_rounds_replayed_from_one_graph(dev, oracle, cyclic_model, chain, lk):
    torch = dev.torch
    model = cyclic_model
    prompt = [t % model.cfg["vocab"] for t in repeating_prompt(14)]
    e = RoundDev(dev, model, prompt, lk=lk, chain=chain)
    nrounds = 16
    for _ in range(nrounds):
        e.launch()
    out_e, log_e, _ = e.result()
    g = RoundDev(dev, model, prompt, lk=lk, chain=chain)
    print(f"case decode_round graph chain={chain} lk={lk}", flush=True)
    g.launch()   # the first round eagerly; it is not part of the graph
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g.launch()
    for i in range(nrounds - 1):
        graph.replay()
        if i % 3 == 0:
            torch.cuda.synchronize()   # replays with and without the host looking in between
    out_g, log_g, st = g.result()
    assert st[dev.pkg.RS_ROUNDS] == nrounds
    assert out_g == out_e and log_g == log_e, "a round has no argument that changes: one captured round replays as every round"


def test_rounds_stop_before_the_cache_is_full(dev, oracle, cyclic_model):
    model = cyclic_model
    prompt = [t % model.cfg["vocab"] for t in repeating_prompt(12)]
    r = RoundDev(dev, model, prompt)
    cap = model.cfg["max_ctx"]
    print("case decode_round until the cache is full", flush=True)
    for _ in range(cap):   # more rounds than the cache has room for
        r.launch()
    out, log, st = r.result()
    pkg = dev.pkg
    assert st[pkg.RS_STOP] == 1 and st[pkg.RS_POS] + 16 <= cap and st[pkg.RS_NCTX] == st[pkg.RS_POS] + 1
    assert st[pkg.RS_POS] + 16 + 16 > cap, "it stopped no earlier than it had to"
    for _ in range(3):
        r.launch()
    out2, log2, st2 = r.result()
    assert out2 == out and np.array_equal(st2, st), "a stopped session stays as it is"
    out_h, _ = host_loop(dev, model, prompt, len(out))
    assert out == out_h
