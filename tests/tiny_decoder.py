"""A reduced decoder with random weights (benchmark config 4's shape at test sizes), held as numpy arrays, and its two
renderings: the oracle's C structs (host pointers) and the device library's C structs (device pointers)."""
import ctypes as C

import numpy as np

import oracle_lib as ol
from fnx_gpu import SyntheticDecoder

HD = 256


class Q8sO(C.Structure):
    _fields_ = [("q", C.c_void_p), ("d", C.c_void_p), ("n_out", C.c_int), ("n_in", C.c_int)]


class RopeO(C.Structure):
    _fields_ = [("base", C.c_float), ("scaled", C.c_int), ("c_low", C.c_float), ("c_high", C.c_float), ("inv_scale", C.c_float),
                ("mscale", C.c_float)]


class DecLayerO(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p), ("ffn_norm", C.c_void_p), ("wq", Q8sO), ("wk", Q8sO),
                ("wv", Q8sO), ("wo", Q8sO), ("moe", ol.MoeLayer), ("kc", C.c_void_p), ("vc", C.c_void_p)]


class DecoderO(C.Structure):
    _fields_ = [("n", C.c_int), ("nq", C.c_int), ("nkv", C.c_int), ("nlayers", C.c_int), ("vocab", C.c_int), ("max_ctx", C.c_int),
                ("eps", C.c_float), ("rope", RopeO), ("layers", C.c_void_p), ("out_norm", C.c_void_p), ("head", Q8sO), ("emb", C.c_void_p)]


class MtpO(C.Structure):
    _fields_ = [("norm_emb", C.c_void_p), ("norm_hid", C.c_void_p), ("out_norm", C.c_void_p), ("fc_emb", Q8sO), ("fc_hid", Q8sO), ("head", Q8sO),
                ("layer", DecLayerO), ("dv0", C.c_int), ("dv1", C.c_int), ("pen", C.c_void_p), ("pen_par", C.c_void_p)]


def _oracle_q8s(oracle):
    def quantize(w):
        rows, cols = w.shape
        q = np.zeros((rows, cols), dtype=np.int8)
        d = np.zeros((rows, cols // 32), dtype=np.uint16)
        oracle.lib.fnx_o_quantize_q8_0_split(ol.ptr(w), rows, cols, ol.ptr(q), ol.ptr(d))
        return q, d
    return quantize


class TinyDecoder(SyntheticDecoder):
    """the package's synthetic model (Gaussian dense matrices quantised by the oracle unless cheap_draws), with the oracle's
    rendering of it beside the device's"""

    def __init__(self, oracle, **kw):
        super().__init__(quantize=_oracle_q8s(oracle) if oracle is not None else None, **kw)
        self.oracle = oracle

    @classmethod
    def of(cls, model, oracle):
        """a SyntheticDecoder built elsewhere, with the oracle's rendering added"""
        m = cls.__new__(cls)
        m.__dict__.update(model.__dict__)
        m.oracle = oracle
        return m


    # ---- the oracle's rendering: host arrays; the caches are numpy arrays kept here
    def oracle_structs(self):
        c = self.cfg
        keep = []

        def q8s(t, rows, cols):
            return Q8sO(ol.ptr(t[0]), ol.ptr(t[1]), rows, cols)

        def lay(L):
            kc = np.zeros((c["max_ctx"], c["nkv"], HD), dtype=np.uint16)
            vc = np.zeros_like(kc)
            keep.extend([kc, vc])
            moe = ol.MoeLayer(c["n"], c["ff"], c["nexp"], c["topk"], ol.ptr(L["router"]), ol.ptr(L["gu"]), ol.ptr(L["down"]), ol.ptr(L["sh_gu"]),
                              ol.ptr(L["sh_down"]))
            return DecLayerO(ol.ptr(L["attn_norm"]), ol.ptr(L["q_norm"]), ol.ptr(L["k_norm"]), ol.ptr(L["ffn_norm"]),
                             q8s(L["wq"], c["nq"] * 2 * HD, c["n"]), q8s(L["wk"], c["nkv"] * HD, c["n"]), q8s(L["wv"], c["nkv"] * HD, c["n"]),
                             q8s(L["wo"], c["n"], c["nq"] * HD), moe, ol.ptr(kc), ol.ptr(vc)), (kc, vc)

        arr = (DecLayerO * c["nlayers"])()
        caches = []
        for i, L in enumerate(self.layers):
            arr[i], kv = lay(L)
            caches.append(kv)
        D = DecoderO(c["n"], c["nq"], c["nkv"], c["nlayers"], c["vocab"], c["max_ctx"], c["eps"], RopeO(*self.rope), C.cast(arr, C.c_void_p),
                     ol.ptr(self.out_norm), q8s(self.head, c["vocab"], c["n"]), ol.ptr(self.emb))
        ml, mkv = lay(self.mtp["layer"])
        M = MtpO(ol.ptr(self.mtp["norm_emb"]), ol.ptr(self.mtp["norm_hid"]), ol.ptr(self.mtp["out_norm"]), q8s(self.mtp["fc_emb"], c["n"], c["n"]),
                 q8s(self.mtp["fc_hid"], c["n"], c["n"]), q8s(self.mtp["head"], c["vocab"], c["n"]), ml)
        keep.extend([arr, D, M])
        return D, M, caches, mkv, keep


class OracleSession:
    """verify / draft on the CPU oracle, with the caches kept between calls"""

    def __init__(self, model, threads=8):
        self.m, self.threads = model, threads
        self.D, self.M, self.caches, self.mtp_cache, self._keep = model.oracle_structs()
        lib = model.oracle.lib
        lib.fnx_o_decoder_verify.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        lib.fnx_o_decoder_verify.restype = None
        lib.fnx_o_mtp_draft.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        lib.fnx_o_mtp_draft.restype = None
        lib.fnx_o_layer_probe.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        lib.fnx_o_layer_probe.restype = None
        lib.fnx_o_layer_taps.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        lib.fnx_o_layer_taps.restype = None
        lib.fnx_o_decoder_layer.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int]
        lib.fnx_o_decoder_layer.restype = None

    def _probe(self, T, layers):
        c = self.m.cfg
        lg, ti = np.zeros((layers, T, c["nexp"] + 1), dtype=np.float32), np.zeros((layers, T, c["topk"]), dtype=np.int32)
        self.m.oracle.lib.fnx_o_layer_probe(ol.ptr(lg), ol.ptr(ti), layers)
        return lg, ti

    def _taps(self, T, layers):
        """arrays the next `layers` layers fill: the rows going in, the attention's rows before the output projection, the rows
        after the attention half, the MoE half's rows"""
        c = self.m.cfg
        t = dict(x_in=np.zeros((layers, T, c["n"]), dtype=np.float32), att=np.zeros((layers, T, c["nq"] * HD), dtype=np.float32),
                 x_mid=np.zeros((layers, T, c["n"]), dtype=np.float32), moe=np.zeros((layers, T, c["n"]), dtype=np.float32))
        self.m.oracle.lib.fnx_o_layer_taps(ol.ptr(t["x_in"]), ol.ptr(t["att"]), ol.ptr(t["x_mid"]), ol.ptr(t["moe"]), layers)
        return t

    def verify(self, tokens, pos0, routing=False, taps=False):
        """routing: also every layer's router logits [layer][T][nexp + 1] and picks [layer][T][topk]; taps: also every layer's
        rows on their way through it (see _taps)"""
        c = self.m.cfg
        tok = np.ascontiguousarray(tokens, dtype=np.int32)
        T = len(tok)
        hidden = np.zeros((T, c["n"]), dtype=np.float32)
        logits = np.zeros((T, c["vocab"]), dtype=np.float32)
        best = np.zeros(T, dtype=np.int32)
        probe = self._probe(T, c["nlayers"]) if routing else None
        tp = self._taps(T, c["nlayers"]) if taps else None
        self.m.oracle.lib.fnx_o_decoder_verify(C.byref(self.D), ol.ptr(tok), T, pos0, ol.ptr(hidden), ol.ptr(logits), ol.ptr(best), self.threads)
        self.m.oracle.lib.fnx_o_layer_probe(None, None, 0)
        self.m.oracle.lib.fnx_o_layer_taps(None, None, None, None, 0)
        r = dict(hidden=hidden, logits=logits, best=best)
        if routing:
            r["route_logits"], r["route_topi"] = probe
        if taps:
            r["taps"] = tp
        return r

    def layer(self, x, l, pos0):
        """one layer (l: its number, or -1 for the draft layer's) on the rows x, with its rows on their way through it"""
        x = np.array(x, dtype=np.float32, order="C")
        T = x.shape[0]
        tp = self._taps(T, 1)
        lp = C.byref(self.M.layer) if l < 0 else C.cast(C.addressof(self._layer_arr()[l]), C.c_void_p)
        self.m.oracle.lib.fnx_o_decoder_layer(C.byref(self.D), lp, ol.ptr(x), T, pos0, self.threads)
        self.m.oracle.lib.fnx_o_layer_taps(None, None, None, None, 0)
        return dict(x_out=x, att=tp["att"][0], x_mid=tp["x_mid"][0], moe=tp["moe"][0])

    def _layer_arr(self):
        return self._keep[-3]   # the DecLayerO array oracle_structs built

    def draft(self, src, tokens, pos0, routing=False, dv=None, pen=None, par=None):
        """dv = (dv0, dv1): the head's rows for those tokens only; pen = (indexes relative to dv0, counts), par = (repeat, freq,
        present): the last row's penalties (engine.cu:2130-2131)"""
        c = self.m.cfg
        tok = np.ascontiguousarray(tokens, dtype=np.int32)
        src = np.ascontiguousarray(src, dtype=np.float32)
        T = len(tok)
        hidden = np.zeros((T, c["n"]), dtype=np.float32)
        M, keep = self.M, []
        if dv is not None or pen is not None:
            M = MtpO.from_buffer_copy(self.M)
            if dv is not None:
                q, d = self.m.mtp["head"]
                keep = [np.ascontiguousarray(q[dv[0]:dv[1]]), np.ascontiguousarray(d[dv[0]:dv[1]])]
                M.dv0, M.dv1 = dv
                M.head = Q8sO(ol.ptr(keep[0]), ol.ptr(keep[1]), dv[1] - dv[0], c["n"])
            if pen is not None:
                keep += [np.concatenate([[len(pen[0])], pen[0], pen[1]]).astype(np.int32), np.asarray(par, dtype=np.float32)]
                M.pen, M.pen_par = ol.ptr(keep[-2]), ol.ptr(keep[-1])
        logits = np.zeros((T, dv[1] - dv[0] if dv is not None else c["vocab"]), dtype=np.float32)
        best = np.zeros(T, dtype=np.int32)
        probe = self._probe(T, 1) if routing else None
        self.m.oracle.lib.fnx_o_mtp_draft(C.byref(self.D), C.byref(M), ol.ptr(src), ol.ptr(tok), T, pos0, ol.ptr(hidden), ol.ptr(logits),
                                          ol.ptr(best), self.threads)
        self.m.oracle.lib.fnx_o_layer_probe(None, None, 0)
        r = dict(hidden=hidden, logits=logits, best=best)
        if routing:
            r["route_logits"], r["route_topi"] = probe
        return r


def spec_generate(sess, lookup, accept, prompt, max_new, K=4, lk=15, speculate=True, forced=None):
    """The greedy decode round of session.cpp:530-679 over a session with verify(tokens, pos0) / draft(src, tokens, pos0):
    verify [x] + drafts -> accept -> commit -> draft d1 from the kept rows -> prompt lookup, else an MTP chain of K.
    The prompt is read first (windows of up to 16 rows; the draft layer reads the same rows shifted by one, as the
    reference's prompt pass keeps its cells current). Returns the emitted tokens and per-round statistics."""
    ctx = list(prompt)
    pos = 0
    hidden_last = None
    # read the prompt: rows 0 .. len-2 (the last token is the first window's row)
    body = ctx[:-1]
    for i in range(0, len(body), 16):
        w = body[i:i + 16]
        r = sess.verify(w, pos)
        nxt = ctx[i + 1:i + 1 + len(w)]
        sess.draft(r["hidden"], nxt, pos)
        pos += len(w)
    x, drafts, out, rounds = ctx[-1], [], [], []
    while len(out) < max_new:
        rows = [x] + drafts[:15]
        p = pos
        r = sess.verify(rows, p)
        o = [int(t) for t in r["best"]]
        n = accept(rows, o)
        used = min(n, max_new - len(out))
        out.extend(o[:used])
        pos += used
        ctx.extend(o[:used])
        x = o[used - 1]
        rounds.append((len(rows) - 1, used))
        if len(out) >= max_new:
            break
        d = sess.draft(r["hidden"][:used], o[:used], p)
        d1 = int(d["best"][used - 1])
        if not speculate:
            drafts = []
            continue
        if forced is not None:
            drafts = [int(t) for t in forced(len(out), d1)]
            continue
        drafts, _ = lookup(ctx, lk, d1)
        drafts = [int(t) for t in drafts]
        if drafts:
            continue
        drafts = [d1]
        src = d["hidden"][used - 1:used]
        for j in range(1, K):
            d = sess.draft(src, [drafts[-1]], p + used - 1 + j)
            drafts.append(int(d["best"][0]))
            src = d["hidden"][:1]
    return out, rounds
