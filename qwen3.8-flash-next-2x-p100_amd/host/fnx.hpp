// C++ host-side mirror of the reference's operator API for the verify path (engine/src/kernels.hpp, namespace fnx):
// the same function names and argument meaning, throwing std::runtime_error on failure as the reference's launch
// wrappers do (ck_launch, kernels.cu:52-55), implemented over the C ABI of libfnx_mi355x.so.
//
// The reference fixes the model shape at compile time (N, NEXP, TOPK in model.hpp:38-43); here the same names are
// template-free constants of a Shape the caller sets once (defaults: the benchmark's hidden 2048, 512 experts, top-10).
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/fnx_mi355x.h"

namespace fnx {

constexpr int MAXT = FNX_MAXT;
using Job = fnx_job;        // kernels.hpp:18-23
using BigJob = fnx_bigjob;  // kernels.hpp:32-37
using DW = fnx_dw;          // model.hpp:84-94

struct Shape {
    int N = 2048, NEXP = 512, TOPK = 10;
};
inline Shape& shape() {
    static Shape s;
    return s;
}

inline void ck(int status) {
    if (status != 0) throw std::runtime_error(fnx_last_error());
}

constexpr size_t q8_1_bytes(int n) { return (size_t) (n / 32) * 36; }   // kernels.hpp:39

// kernels.hpp:41
inline void quantize_q8_1(const float* x, void* q, int n, int rows, void* st) { ck(fnx_quantize_q8_1(x, q, n, rows, st)); }
// kernels.hpp:49
inline void mmvq(const DW& W, size_t w_stride, const Job* jobs, const int* njobs, int njobs_max, const void* y, float* out, int out_stride,
                 void* st) {
    ck(fnx_mmvq(&W, w_stride, jobs, njobs, njobs_max, y, out, out_stride, st));
}
// kernels.hpp:54-55
inline void gemv_f32(const float* W, const float* x, float* y, int rows, int n, int T, void* st) { ck(fnx_gemv_f32(W, x, y, rows, n, T, st)); }
inline void gemv_bf16(const uint16_t* W, const float* x, float* y, int rows, int n, int T, void* st) { ck(fnx_gemv_bf16(W, x, y, rows, n, T, st)); }
// kernels.hpp:79 (logits rows of NEXP)
inline void route(const float* logits, int T, int* topi, float* topw, Job* jobs_gu, Job* jobs_down, int* njobs, void* st) {
    ck(fnx_route(logits, shape().NEXP, T, shape().NEXP, shape().TOPK, topi, topw, jobs_gu, jobs_down, njobs, st));
}
// kernels.hpp:81, 349
inline void swiglu_q8_1(const float* g, const float* u, void* q, int n, int rows, void* st) { ck(fnx_swiglu_q8_1(g, u, q, n, rows, st)); }
inline void swiglu_stacked_q8_1(const float* gu, void* hq, int ffs, int T, void* st) { ck(fnx_swiglu_stacked_q8_1(gu, hq, ffs, T, st)); }
// kernels.hpp:83
inline void moe_combine(const float* part, const float* topw, const float* sh, const float* sh_logit, float* out, int T, void* st) {
    ck(fnx_moe_combine(part, topw, sh, sh_logit, 1, out, T, shape().N, shape().TOPK, st));
}
// kernels.hpp:294 (the streaming, cache and fold arguments of the reference have no counterpart on one GPU)
inline void router_route(const void* W, bool w_bf16, const float* x, float* logits, int T, int* topi, float* topw, Job* jobs_gu, Job* jobs_dn,
                         int* njobs, void* st) {
    ck(fnx_router_route(W, w_bf16 ? 1 : 0, x, logits, T, shape().N, shape().NEXP, shape().TOPK, topi, topw, jobs_gu, jobs_dn, njobs, st));
}
// kernels.hpp:319, 343
inline void moe_gate_up(const DW& A, size_t sa, const Job* jobs, const int* njobs, int njobs_max, const void* xq, float* gu, void* st) {
    ck(fnx_moe_gate_up(&A, sa, jobs, njobs, njobs_max, xq, gu, shape().TOPK, st));
}
inline void moe_down(const DW& A, size_t sa, const Job* jobs, const int* njobs, int njobs_max, const float* gu, float* part, void* st) {
    ck(fnx_moe_down(&A, sa, jobs, njobs, njobs_max, gu, part, st));
}
// kernels.hpp:433
inline void argmax(const float* logits, int rows, int T, int v0, float* best_v, int* best_i, unsigned long long* keys, unsigned* err, void* st) {
    ck(fnx_argmax(logits, rows, T, v0, best_v, best_i, keys, err, st));
}
// session.hpp:55-58
inline std::vector<int> lookup_drafts(const std::vector<int>& ctx, int lk, int d1, int* match = nullptr) {
    std::vector<int> r((size_t) (lk > 0 ? lk : 0));
    const int n = fnx_lookup_drafts(ctx.data(), (int) ctx.size(), 3, lk, d1, r.data(), match);
    if (n < 0) throw std::runtime_error(fnx_last_error());
    r.resize((size_t) n);
    return r;
}
// session.cpp:573
inline int accept_greedy(const std::vector<int>& rows, const std::vector<int>& o) {
    const int n = fnx_accept_greedy(rows.data(), o.data(), (int) rows.size());
    if (n < 0) throw std::runtime_error(fnx_last_error());
    return n;
}
// load-time re-laying of an IQ3_S tensor (no counterpart in the reference's API; its own load-time layouts are model.hpp:78-82)
inline void iq3s_repack(const void* src, void* dst, size_t n_weights, void* st) { ck(fnx_iq3s_repack(src, dst, n_weights, st)); }

// ---- the prompt path (prefill.cu:288-377, kernels.hpp:328-330)
using BigJob = fnx_bigjob;
inline void pf_route(const float* logits, int C, int* topi, float* topw, int* cnt, int* jbase, BigJob* jobs_gu, BigJob* jobs_dn, int njobs_cap,
                     int* njobs, void* st) {
    ck(fnx_pf_route(logits, shape().NEXP + 1, C, shape().NEXP, shape().TOPK, topi, topw, cnt, jbase, jobs_gu, jobs_dn, njobs_cap, njobs, st));
}
inline void p100_f32_f16(const float* x, size_t n, uint16_t* out, void* st) { ck(fnx_f32_f16(x, n, out, st)); }
// kernels.hpp:324-325
inline void moe_gate_up_big(const DW& A, size_t sa, const BigJob* jobs, const int* njobs, int njobs_cap, const void* xq, float* gu, void* st) {
    ck(fnx_moe_gate_up_big(&A, sa, jobs, njobs, njobs_cap, xq, gu, st));
}
inline void moe_down_big(const DW& A, size_t sa, const BigJob* jobs, const int* njobs, int njobs_cap, const float* gu, float* part, void* st) {
    ck(fnx_moe_down_big(&A, sa, jobs, njobs, njobs_cap, gu, part, st));
}
inline void moe_gate_up_mma(const DW& A, size_t sa, const BigJob* jobs, const int* njobs, int njobs_cap, const uint16_t* xh, float* gu, void* st) {
    ck(fnx_moe_gate_up_mma(&A, sa, jobs, njobs, njobs_cap, xh, gu, st));
}
inline void swiglu_h16(const float* gu, int ffs, int P, uint16_t* h16, void* st) { ck(fnx_swiglu_h16(gu, ffs, P, h16, st)); }
// moe_gate_up_mma and swiglu_h16 as one launch that writes h only (no counterpart of its own in kernels.hpp: lines 328 + 329)
inline void moe_gate_up_h16_mma(const DW& A, size_t sa, const BigJob* jobs, const int* njobs, int njobs_cap, const uint16_t* xh, uint16_t* h16, void* st) {
    ck(fnx_moe_gate_up_h16_mma(&A, sa, jobs, njobs, njobs_cap, xh, h16, st));
}
inline void moe_down_mma(const DW& A, size_t sa, const BigJob* jobs, const int* njobs, int njobs_cap, const uint16_t* h16, float* part, void* st) {
    ck(fnx_moe_down_mma(&A, sa, jobs, njobs, njobs_cap, h16, part, st));
}
// ---- around the MoE half (kernels.hpp:238, 259, 406, 414-418)
using Q8S = fnx_q8s;
using Rope = fnx_rope;
inline void rms_norm_rows(const float* x, const float* w, float* y, int rows, int n, float eps, void* st) { ck(fnx_rms_norm_rows(x, w, y, rows, n, eps, st)); }
// the hand-over between two layers: moe_combine of the partial sums, the residual add, rms_norm_rows and quantize_q8_1 in one pass
inline void combine_add_norm_q8(const float* part, const float* topw, const float* sh, const float* sh_logit, float* x, const float* w, float* xn,
                                void* xq, int T, float eps, void* st) {
    ck(fnx_combine_add_norm_q8(part, topw, sh, sh_logit, 1, shape().TOPK, x, w, xn, xq, T, shape().N, eps, st));
}
// the load-time tile-major layout of a dense matrix's int8 values (no counterpart in kernels.hpp: model.hpp:78-82 is the reference's load-time split)
inline void q8s_tile(const int8_t* src, int8_t* dst, int rows, int cols, void* st) { ck(fnx_q8s_tile(src, dst, rows, cols, st)); }
inline void q8s_gemv(const Q8S& w, const void* y, float* out, int out_stride, int T, void* st) { ck(fnx_q8s_gemv(&w, y, out, out_stride, T, st)); }
inline void q8s_gemv_segs(const Q8S* w, float* const* out, const int* out_stride, int n, const void* y, int T, void* st) {
    const Q8S* p[3] = {&w[0], n > 1 ? &w[1] : nullptr, n > 2 ? &w[2] : nullptr};
    ck(fnx_q8s_gemv_segs(p, out, out_stride, n, y, T, st));
}
inline void attn_prep_append(float* qg, float* k, const float* v, const float* q_norm, const float* k_norm, uint16_t* kc, uint16_t* vc, int nq,
                             int nkv, int T, const int* pos0, int max_ctx, float eps, const Rope& base, void* st) {
    ck(fnx_attn_prep_append(qg, k, v, q_norm, k_norm, kc, vc, nq, nkv, T, pos0, max_ctx, eps, &base, st));
}
inline void attn(const float* qg, const uint16_t* kc, const uint16_t* vc, float* out, int nq, int nkv, const int* pos0, int T, int max_ctx,
                 float* scratch, void* st) {
    ck(fnx_attn(qg, kc, vc, out, nq, nkv, pos0, T, max_ctx, scratch, st));
}

// ---- the sampler (kernels.hpp:434-447; session.hpp:17-26, 41-48)
constexpr int TOPK_N = FNX_TOPK_N;
inline void penalize_row(float* row, int n, const int* pen, const float* par, void* st) { ck(fnx_penalize_row(row, n, pen, par, st)); }
inline void top_tokens(float* logits, int n, int T, int v0, const int* pen_tok, const int* pen_cnt, const int* pen_n, int pen_stride,
                       const float* pen_par, const int* bias_tok, const float* bias_val, const int* bias_off, const int* bias_n, float* out_v,
                       int* out_i, unsigned* err, void* st) {
    ck(fnx_top_tokens(logits, n, T, v0, pen_tok, pen_cnt, pen_n, pen_stride, pen_par, bias_tok, bias_val, bias_off, bias_n, out_v, out_i, err, st));
}
struct Sampling {   // the values of session.hpp:17-26 a distribution is made from
    float temperature = 1.f, top_p = 1.f, min_p = 0.f;
    int top_k = 0;
};
struct Dist {
    std::vector<int> ids;
    std::vector<double> p;
    double prob(int id) const {
        for (size_t i = 0; i < ids.size(); ++i)
            if (ids[i] == id) return p[i];
        return 0.0;
    }
};
inline Dist make_dist(const std::vector<std::pair<float, int>>& cand, const Sampling& s) {
    std::vector<float> v(cand.size());
    std::vector<int> id(cand.size());
    for (size_t i = 0; i < cand.size(); ++i) {
        v[i] = cand[i].first;
        id[i] = cand[i].second;
    }
    const fnx_sampling fs{s.temperature, s.top_p, s.min_p, s.top_k};
    Dist d;
    d.ids.resize(cand.size());
    d.p.resize(cand.size());
    const int k = fnx_make_dist(v.data(), id.data(), (int) cand.size(), &fs, d.ids.data(), d.p.data());
    if (k < 0) throw std::runtime_error(fnx_last_error());
    d.ids.resize((size_t) k);
    d.p.resize((size_t) k);
    return d;
}
inline int draw(const Dist& d, double u) {
    const int t = fnx_draw(d.ids.data(), d.p.data(), (int) d.ids.size(), u);
    if (t < 0) throw std::runtime_error(fnx_last_error());
    return t;
}

// ---- GGUF files (gguf.hpp:25-45): the handle closes with the object
class Gguf {
public:
    explicit Gguf(const std::string& first_shard) : g_(fnx_gguf_open(first_shard.c_str())) {
        if (!g_) throw std::runtime_error(fnx_last_error());
    }
    ~Gguf() { fnx_gguf_close(g_); }
    Gguf(const Gguf&) = delete;
    Gguf& operator=(const Gguf&) = delete;
    fnx_gguf_tensor t(const std::string& name) const {   // throws when missing
        fnx_gguf_tensor out;
        ck(fnx_gguf_find(g_, name.c_str(), &out));
        return out;
    }
    bool has_key(const std::string& key) const { return fnx_gguf_key_type(g_, key.c_str()) >= 0; }
    int64_t i(const std::string& key) const {
        int64_t v;
        ck(fnx_gguf_int(g_, key.c_str(), &v));
        return v;
    }
    double num(const std::string& key) const {
        double v;
        ck(fnx_gguf_num(g_, key.c_str(), &v));
        return v;
    }
    std::string s(const std::string& key) const {
        const char* v = fnx_gguf_str(g_, key.c_str());
        if (!v) throw std::runtime_error("gguf: no string key " + key);
        return v;
    }
    int shards() const { return fnx_gguf_shards(g_); }
    int count() const { return fnx_gguf_count(g_); }
    const fnx_gguf* handle() const { return g_; }

private:
    fnx_gguf* g_;
};

}  // namespace fnx
