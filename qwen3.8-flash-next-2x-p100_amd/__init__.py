"""Python-side plumbing for the MI355X verify-path library: loads libfnx_mi355x.so and exposes its C ABI.

The product is the C ABI (include/fnx_mi355x.h); this module only carries device pointers of torch tensors across
ctypes for the tests and the benchmark. There is no fallback: if the shared library is missing, import of `lib()`
raises, and every compute call needs a GPU.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FNX_LIB_PATH") or os.path.join(HERE, "libfnx_mi355x.so")

MAXT = 16
PF_JOB = 64
T_IQ3_S = 21
T_IQ3S_UNIT64 = 1021
T_IQ3S_TILE16 = 1022
IQ3S_BLOCK = 110
Q8_1_BLOCK = 36
MOE_SYNC_WORDS = 33568
ARGMAX_WORDS = 32   # FNX_ARGMAX_WORDS: a key and an arrival count a row   # fnx_moe_ws.sync: uint32 words, zeroed once
ERR_BARRIER = 4


class Job(C.Structure):
    _fields_ = [("w", C.c_int), ("n", C.c_int), ("y", C.c_int * MAXT), ("out", C.c_int * MAXT)]


class BigJob(C.Structure):
    _fields_ = [("w", C.c_int), ("n", C.c_int), ("y", C.c_int * PF_JOB), ("out", C.c_int * PF_JOB)]


class DW(C.Structure):
    _fields_ = [("p", C.c_void_p), ("type", C.c_uint32), ("n_in", C.c_int), ("n_out", C.c_int), ("row_bytes", C.c_size_t),
                ("ep", C.c_void_p)]


class Q8S(C.Structure):
    _fields_ = [("q", C.c_void_p), ("d", C.c_void_p), ("n_out", C.c_int), ("n_in", C.c_int), ("tiled", C.c_int)]


class MoeLayer(C.Structure):
    _fields_ = [("n", C.c_int), ("ff", C.c_int), ("nexp", C.c_int), ("topk", C.c_int), ("router", C.c_void_p),
                ("router_bf16", C.c_int), ("gu", DW), ("gu_stride", C.c_size_t), ("down", DW), ("down_stride", C.c_size_t),
                ("sh_gu", DW), ("sh_down", DW), ("sh_gu_q8", Q8S), ("sh_down_q8", Q8S)]


class MoeWs(C.Structure):
    _fields_ = [("xq", C.c_void_p), ("logits", C.c_void_p), ("topi", C.c_void_p), ("topw", C.c_void_p), ("jobs_gu", C.c_void_p),
                ("jobs_dn", C.c_void_p), ("njobs", C.c_void_p), ("gu", C.c_void_p), ("part", C.c_void_p), ("sync", C.c_void_p)]


class PfWs(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in ("logits", "topi", "topw", "cnt", "jbase", "jobs_gu", "jobs_dn", "njobs", "xh", "gu", "h16", "part")]


class Rope(C.Structure):
    _fields_ = [("base", C.c_float), ("scaled", C.c_int), ("c_low", C.c_float), ("c_high", C.c_float), ("inv_scale", C.c_float),
                ("mscale", C.c_float)]


class DecLayer(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p), ("ffn_norm", C.c_void_p), ("wq", Q8S), ("wk", Q8S),
                ("wv", Q8S), ("wo", Q8S), ("moe", MoeLayer), ("kc", C.c_void_p), ("vc", C.c_void_p)]


class Decoder(C.Structure):
    _fields_ = [("n", C.c_int), ("nq", C.c_int), ("nkv", C.c_int), ("nlayers", C.c_int), ("vocab", C.c_int), ("max_ctx", C.c_int),
                ("eps", C.c_float), ("rope", Rope), ("layers", C.c_void_p), ("out_norm", C.c_void_p), ("head", Q8S), ("emb", C.c_void_p)]


class DecWs(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in ("x", "xn", "qg", "k", "v", "att", "o", "attn_scratch", "xq", "hidden", "logits", "best_v", "best_i",
                                          "keys", "err")] + [("moe", MoeWs)]


class Mtp(C.Structure):
    _fields_ = [("norm_emb", C.c_void_p), ("norm_hid", C.c_void_p), ("out_norm", C.c_void_p), ("fc_emb", Q8S), ("fc_hid", Q8S), ("head", Q8S),
                ("layer", DecLayer), ("dv0", C.c_int), ("dv1", C.c_int), ("pen", C.c_void_p), ("pen_par", C.c_void_p)]


class Round(C.Structure):
    _fields_ = [("state", C.c_void_p), ("rows", C.c_void_p), ("ctx", C.c_void_p), ("ctx_cap", C.c_int), ("log", C.c_void_p), ("log_cap", C.c_int),
                ("speculate", C.c_int), ("key_n", C.c_int), ("lk", C.c_int), ("scratch", C.c_void_p), ("chain", C.c_int), ("chain_src", C.c_void_p)]


class Sampling(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float), ("min_p", C.c_float), ("top_k", C.c_int)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("type", C.c_uint32), ("n_dims", C.c_int), ("ne", C.c_int64 * 4), ("data", C.c_void_p), ("nbytes", C.c_size_t),
                ("shard", C.c_int), ("offset", C.c_uint64)]


class MoeBufs(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in ("router", "gu", "down", "sh_gu", "sh_down")] + \
               [(k, C.c_size_t) for k in ("router_bytes", "gu_bytes", "down_bytes", "sh_gu_bytes", "sh_down_bytes")]


RS_NCTX, RS_POS, RS_ROWS, RS_ACCEPTED, RS_POS_PREV, RS_ROUNDS, RS_STOP, RS_CHAIN, RS_CHAIN_POS, RS_WORDS = 0, 1, 2, 3, 4, 5, 6, 7, 8, 24

EXPORTS = {
    # name: (restype, argtypes)
    "fnx_last_error": (C.c_char_p, []),
    "fnx_version": (C.c_char_p, []),
    "fnx_iq3s_repack": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "fnx_iq3s_tile16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "fnx_iq3s_tile16_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int]),
    "fnx_quantize_q8_1": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "fnx_mmvq": (C.c_int, [C.POINTER(DW), C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "fnx_gemv_f32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "fnx_gemv_bf16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "fnx_route": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                            C.c_void_p]),
    "fnx_router_route": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_swiglu_q8_1": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "fnx_swiglu_stacked_q8_1": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "fnx_moe_gate_up": (C.c_int, [C.POINTER(DW), C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "fnx_moe_down": (C.c_int, [C.POINTER(DW), C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_moe_combine": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                  C.c_void_p]),
    "fnx_argmax": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_lookup_drafts": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "fnx_lookup_drafts_dev": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_void_p]),
    "fnx_accept_greedy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "fnx_accept_greedy_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "fnx_layer_profile": (C.c_int, [C.c_int]),
    "fnx_layer_profile_read": (C.c_int, [C.c_void_p]),
    "fnx_stream_read": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "fnx_moe_verify_layer": (C.c_int, [C.POINTER(MoeLayer), C.c_void_p, C.c_int, C.c_void_p, C.POINTER(MoeWs), C.c_void_p]),
    "fnx_moe_verify_layer_static": (C.c_int, [C.POINTER(MoeLayer), C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "fnx_moe_static_status": (C.c_int, [C.c_void_p, C.c_void_p]),
    "fnx_pf_route": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                               C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "fnx_f32_f16": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]),
    "fnx_moe_gate_up_mma": (C.c_int, [C.POINTER(DW), C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_swiglu_h16": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "fnx_moe_down_mma": (C.c_int, [C.POINTER(DW), C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_moe_gate_up_big": (C.c_int, [C.POINTER(DW), C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_moe_down_big": (C.c_int, [C.POINTER(DW), C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_moe_gate_up_h16_mma": (C.c_int, [C.POINTER(DW), C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_rms_norm_rows": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p]),
    "fnx_add_norm_q8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p]),
    "fnx_combine_add_norm_q8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                          C.c_int, C.c_int, C.c_float, C.c_void_p]),
    "fnx_add_rows": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "fnx_embed_rows": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "fnx_q8s_tile": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "fnx_q8s_tile_bytes": (C.c_size_t, [C.c_int, C.c_int]),
    "fnx_q8s_gemv": (C.c_int, [C.POINTER(Q8S), C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "fnx_q8s_gemv_segs": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p]),
    "fnx_attn_prep_append": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                       C.c_int, C.c_void_p, C.c_int, C.c_float, C.POINTER(Rope), C.c_void_p]),
    "fnx_attn_scratch_floats": (C.c_size_t, [C.c_int, C.c_int, C.c_int]),
    "fnx_attn": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                           C.c_void_p]),
    "fnx_decoder_verify": (C.c_int, [C.POINTER(Decoder), C.c_void_p, C.c_int, C.c_void_p, C.POINTER(DecWs), C.c_void_p]),
    "fnx_decoder_layer": (C.c_int, [C.POINTER(Decoder), C.POINTER(DecLayer), C.c_void_p, C.c_int, C.c_void_p, C.POINTER(DecWs), C.c_void_p]),
    "fnx_mtp_draft": (C.c_int, [C.POINTER(Decoder), C.POINTER(Mtp), C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(DecWs), C.c_void_p]),
    "fnx_decode_round": (C.c_int, [C.POINTER(Decoder), C.POINTER(Mtp), C.POINTER(Round), C.POINTER(DecWs), C.c_void_p]),
    "fnx_top_tokens": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                 C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_penalize_row": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "fnx_make_dist": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(Sampling), C.c_void_p, C.c_void_p]),
    "fnx_draw": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_double]),
    "fnx_accept_sampled": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.POINTER(Sampling), C.c_void_p, C.c_void_p, C.c_void_p,
                                     C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(C.c_int)]),
    "fnx_gguf_open": (C.c_void_p, [C.c_char_p]),
    "fnx_gguf_close": (None, [C.c_void_p]),
    "fnx_gguf_shards": (C.c_int, [C.c_void_p]),
    "fnx_gguf_count": (C.c_int, [C.c_void_p]),
    "fnx_gguf_at": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(GgufTensor)]),
    "fnx_gguf_find": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(GgufTensor)]),
    "fnx_gguf_row_bytes": (C.c_size_t, [C.POINTER(GgufTensor)]),
    "fnx_gguf_key_type": (C.c_int, [C.c_void_p, C.c_char_p]),
    "fnx_gguf_int": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_int64)]),
    "fnx_gguf_num": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_double)]),
    "fnx_gguf_str": (C.c_char_p, [C.c_void_p, C.c_char_p]),
    "fnx_gguf_expert_rows2": (C.c_int, [C.POINTER(GgufTensor), C.POINTER(GgufTensor), C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.POINTER(DW),
                                        C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "fnx_gguf_expert_cols": (C.c_int, [C.POINTER(GgufTensor), C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.POINTER(DW), C.POINTER(C.c_size_t),
                                       C.POINTER(C.c_size_t)]),
    "fnx_gguf_moe_layer_bytes": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.POINTER(MoeBufs)]),
    "fnx_gguf_load_moe_layer": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(MoeBufs), C.POINTER(MoeLayer), C.c_void_p]),
    "fnx_moe_prefill_layer": (C.c_int, [C.POINTER(MoeLayer), C.c_void_p, C.c_int, C.c_void_p, C.POINTER(PfWs), C.c_void_p]),
}

_lib = None


class FnxError(RuntimeError):
    pass


def lib():
    """The loaded C-ABI library. Raises if it was not built (run qwen3.8-flash-next-2x-p100_amd/build.py)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FnxError("libfnx_mi355x.so is not built: run __graft_entry__.build() or build.py (no CPU path exists)")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(status):
    if status != 0:
        raise FnxError(lib().fnx_last_error().decode())


def dw(tensor_or_ptr, n_in, n_out, ep=None, packed=False, tile16=False):
    p = tensor_or_ptr if isinstance(tensor_or_ptr, int) or tensor_or_ptr is None else tensor_or_ptr.data_ptr()
    return DW(p, T_IQ3S_TILE16 if tile16 else T_IQ3S_UNIT64 if packed else T_IQ3_S, n_in, n_out, n_in // 256 * IQ3S_BLOCK, ep)


def stream_ptr():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)
