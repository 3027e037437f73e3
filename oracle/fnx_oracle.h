/* CPU oracle for the speculative-decode verify path.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference engine's arithmetic for the path
 * (IQ3_S x q8_1 expert mat-vec, router top-k, SwiGLU, combine, argmax, prompt-lookup drafting, greedy acceptance).
 * Only the test-suite, the smoke check and the benchmark's CPU-baseline leg may link or call it. The device library
 * never does: it has no CPU fallback and fails loudly when its HIP code object is missing.
 *
 * Every function cites the reference lines it follows (paths relative to the reference's root).
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   pinned:   h2f/f2h, iq3s_dequant (reference's own tensor_convert.hpp compiled as oracle/_ref + closed forms),
 *             dp4a (selftest.cu's generator), vec_dot/mmvq (vs dequant in f64), q8_1 (closed forms, round trip),
 *             route/topk (two in-tree definitions agree; brute-force sort), jobs (two in-tree builders' invariants),
 *             argmax (brute force + tie/NaN cases), lookup (second in-tree implementation + brute force), accept
 *             (speculative == greedy invariant), swiglu/combine (f64 closed forms), top_tokens (numpy lexsort on
 *             (-key, id) incl. wide ties and signed zeros; penalties as a numpy f32 closed form), make_dist (numpy
 *             vectorised softmax / cumulative cut, limiting cases), accept_sampled (the window's first token is
 *             distributed as the target p whatever q is: exact measure over a grid of uniforms; fixed-draft closed form).
 *   pinned:   the other expert types' decoders (fnx_o_dequant: Q4_0, Q8_0, Q4_K, Q5_K, IQ4_NL, IQ4_XS) against the reference's
 *             own conv::dequantize through oracle/_ref and against numpy restatements; their dots (fnx_o_vec_dot_type)
 *             against the decoded values times the q8_1 values in f64 (the Q4_0 form through the block's sum field to
 *             within that field's f16 rounding).
 *   parity unpinned: the Q5_1 decoder (type 7): the reference's host code has no dequantiser for it; the block layout is
 *             ggml's published one, checked against a numpy restatement only.
 *   parity unpinned: the float-operation order of ggml's vec_dot_<type>_q8_1 for those types (third-party, fetched at
 *             build time, absent from the tree): the per-32-value terms follow its published form, the sums this build's
 *             own fixed order.
 *   parity unpinned: fnx_o_iq3s_quantize_row (the encoder). ggml's quantize_row_iq3_s is not in the reference tree
 *             (third_party/ggml holds only a commit hash) and nothing in the reference calls or tests it. The encoder
 *             here is this build's own; parity of the path is defined from the quantised bytes onward.
 *   parity unpinned: ggml's CPU kernel ggml_vec_dot_iq3_s_q8_K (256-wide Q8_K activations). Not in the tree, never
 *             called by the reference. The oracle follows the reference's own arithmetic (q8_1, 32-wide blocks).
 */
#ifndef FNX_ORACLE_H
#define FNX_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FNX_O_MAXT 16

/* engine/src/kernels.hpp:18-23 */
typedef struct {
    int w;
    int n;
    int y[FNX_O_MAXT];
    int out[FNX_O_MAXT];
} fnx_o_job;

/* half <-> float, engine/src/tensor_convert.hpp:23-50 */
float fnx_o_h2f(uint16_t h);
uint16_t fnx_o_f2h(float x);
/* IEEE round to nearest even, subnormal results included (the device's __float2half) */
uint16_t fnx_o_f2h_rn(float x);

/* p100_compat.h:18-22 (the scalar definition of the 4-way signed byte dot) */
int fnx_o_dp4a(int a, int b, int c);
/* exp as include/fnx_expf.h fixes it (the one exp behind sigm, silu_ and the routing weights on both sides) over n values;
 * pinned against numpy's float64 exp in tests/test_oracle_routing.py */
void fnx_o_expf(const float* x, size_t n, float* y);

/* IQ3_S: 110-byte blocks of 256 weights. tensor_convert.hpp:295-322 */
void fnx_o_iq3s_dequant(const uint8_t* src, size_t n, float* y);
/* this build's own encoder (parity unpinned, see header) */
void fnx_o_iq3s_quantize(const float* w, size_t n, uint8_t* dst);

/* q8_1 activation rows: 36-byte blocks {half d; half sum; int8 qs[32]}. kernels.cu:131-145 */
void fnx_o_quantize_q8_1(const float* x, uint8_t* q, int n, int rows);

/* one lane's share of a super-block: iq3s_x.cuh:4-41. blk: the 110-byte block; q8: the super-block's 8 q8_1 blocks */
float fnx_o_vec_dot_iq3s_q8_1(const uint8_t* blk, const uint8_t* q8, int iqs);

/* out[job.out[j]][r] = W[job.w][r] . y[job.y[j]]   (kernels.cu:192-229, moe.cuh:519-548: lane order and butterfly) */
void fnx_o_mmvq_iq3s(const uint8_t* wbase, size_t w_stride, const uint8_t* const* ep, int nrows, int ncols,
                     const fnx_o_job* jobs, int njobs, const uint8_t* y, float* out, int out_stride, int threads);

/* exact variant: dequantised weights x f32 activations summed in double */
void fnx_o_gemv_exact(const uint8_t* w, int nrows, int ncols, const float* x, int T, double* out);

/* y[t][r] = W[r] . x[t], f32 or bf16 weights. Semantics of kernels.cu:239-287 (k_gemv_f32); the summation order is
 * this build's fixed one, shared bit for bit with the device kernel: 64 lanes, lane l takes float4 chunks l, l+64, ...
 * in order with fmaf on x,y,z,w, then an xor-butterfly 32,16,8,4,2,1 of plain adds. */
void fnx_o_gemv_f32(const float* W, const float* x, float* y, int rows, int n, int T);
void fnx_o_gemv_bf16(const uint16_t* W, const float* x, float* y, int rows, int n, int T);

/* top-k by logit, ties to the lower index, w_k = exp(l_k - l_0) / sum (pick order). moe.cuh:382-411
 * A row with fewer than topk logits above -inf (masked or NaN entries) is filled up with the lowest indexes not yet
 * picked, at weight 0, so that a row's picks stay distinct (the reference emits the index NEXP there, which its callers
 * do not define); a row with no such logit at all gets weights 0. This build's rule, shared with the device. */
void fnx_o_topk_logits(const float* logits, int stride, int T, int nexp, int topk, int* topi, float* topw);
/* softmax over all experts, top-k of the probabilities, renormalised. kernels.cu:338-378 */
void fnx_o_topk_softmax(const float* logits, int stride, int T, int nexp, int topk, int* topi, float* topw);
/* distinct experts in first-pick order. kernels.cu:381-398. returns the job count */
int fnx_o_jobs(const int* topi, int T, int topk, fnx_o_job* gu, fnx_o_job* dn);

/* h = silu(g) * u -> q8_1, rows of n. kernels.cu:400-410 */
void fnx_o_swiglu_q8_1(const float* g, const float* u, uint8_t* q, int n, int rows);
/* rows of [gate (ffs) | up (ffs)] -> q8_1 rows of ffs. moe.cuh:597-608, kernels.cu:2475-2490 */
void fnx_o_swiglu_stacked_q8_1(const float* gu, uint8_t* hq, int ffs, int rows);
/* out[t] = sum_k topw[t][k] part[t*topk+k] (fmaf, k ascending) + sigmoid(sh_logit[t]) sh[t]. kernels.cu:412-419 */
void fnx_o_moe_combine(const float* part, const float* topw, const float* sh, const float* sh_logit, int sh_logit_stride,
                       float* out, int T, int n, int topk);

/* greatest value, lowest index on ties; returns the error word (bit 16: NaN or inf). kernels.cu:1045-1083 */
unsigned fnx_o_argmax(const float* logits, int rows, int T, int v0, float* best_v, int* best_i);

/* session.cpp:428-447 with the key length as a parameter (3 = the reference's LOOKUP_N). returns the draft count */
int fnx_o_lookup_drafts(const int* ctx, int n_ctx, int key_n, int lk, int d1, int* out, int* match);
/* tools/fnx_run.cpp:1046-1059: the fixed-length form */
int fnx_o_lookup_fixed(const int* ctx, int n_ctx, int key_n, int lk, int d1, int* out);
/* session.cpp:573 */
int fnx_o_accept_greedy(const int* rows, const int* o, int R);
/* other expert types at the boundary (kernels.cu:2454-2471): Q4_0 (2), Q5_1 (7), Q8_0 (8), Q4_K (12), Q5_K (13), IQ4_NL (20), IQ4_XS (23) */
int fnx_o_type_block(uint32_t type, int* values, int* bytes);
void fnx_o_dequant(uint32_t type, const uint8_t* src, size_t n, float* y);
float fnx_o_vec_dot_type(uint32_t type, const uint8_t* row, int kb, const uint8_t* q8);
void fnx_o_mmvq_type(uint32_t type, const uint8_t* w, size_t w_stride, int nrows, int ncols, const fnx_o_job* jobs, int njobs, const uint8_t* y,
                     float* out, int out_stride, int threads);
/* kernels.hpp:434-447, topk.cuh: the sampler's candidates (64 a row), logits changed in place; returns the err bits */
unsigned fnx_o_top_tokens(float* logits, int n, int T, int v0, const int* pen_tok, const int* pen_cnt, const int* pen_n, int pen_stride,
                          const float* pen_par, const int* bias_tok, const float* bias_val, const int* bias_off, const int* bias_n, float* out_v,
                          int* out_i);
void fnx_o_penalize_row(float* row, int n, const int* pen, const float* par);
/* session.cpp:41-84, 574-613: a row's distribution, a draw, speculative sampling over a window (ncand <= 64) */
int fnx_o_make_dist(const float* cv, const int* ci, int ncand, float temperature, float top_p, float min_p, int top_k, int* ids, double* p);
int fnx_o_draw(const int* ids, const double* p, int n, double u);
int fnx_o_accept_sampled(const float* cv, const int* ci, int ncand, int T, const int* rows, float temperature, float top_p, float min_p, int top_k,
                         const int* q_ids, const double* q_p, const int* q_n, int q_stride, const double* u, int* o, int* used_u);

/* prefill routing: top-k per row, histogram, jobs of <= pf_job rows per expert, pairs in ascending order.
 * prefill.cu:288-377. jobs: arrays of {w, n, y[pf_job], out[pf_job]} ints. returns the job count */
int fnx_o_pf_jobs(const int* topi, int C, int topk, int nexp, int pf_job, int* jobs_gu, int* jobs_dn, int* cnt);

/* one MoE verify layer (engine.cu:1569-1757 without the cards/streaming): router -> top-k -> jobs -> gate|up ->
 * swiglu q8_1 -> down -> shared expert -> combine. Weights IQ3_S; experts at base + e*stride. */
typedef struct {
    int n, ff, nexp, topk;           /* hidden, expert width, experts, picks */
    const float* router;             /* [nexp + 1][n] f32: the router's rows, then the shared expert's gate */
    const uint8_t* gu;               /* [nexp][2 ff][n] IQ3_S */
    const uint8_t* down;             /* [nexp][n][ff] IQ3_S */
    const uint8_t* sh_gu;            /* [2 ff][n] IQ3_S */
    const uint8_t* sh_down;          /* [n][ff] IQ3_S */
    /* the shared expert as dense split Q8_0 instead (engine.cu:1600-1604: q8s_gemv -> swiglu_stacked_q8_1 -> q8s_gemv):
     * when sh_gu_q is not null these four are used and sh_gu / sh_down are not read (the verify layer only) */
    const int8_t* sh_gu_q;           /* [2 ff][n] */
    const uint16_t* sh_gu_d;         /* [2 ff][n / 32] f16 bits */
    const int8_t* sh_down_q;         /* [n][ff] */
    const uint16_t* sh_down_d;       /* [n][ff / 32] */
} fnx_o_moe_layer;
/* out [T][n]; optional outputs (may be null): logits [T][nexp+1], topi/topw [T][topk], njobs */
void fnx_o_moe_verify_layer(const fnx_o_moe_layer* L, const float* x, int T, float* out, float* logits, int* topi,
                            float* topw, int* njobs, int threads);

/* ---- the prompt path's routed experts on the matrix cores (moe_mma.cuh:1-11, 300-498; moe_mma_iq.cuh:108-152):
 * each weight is the f32 product d * (1 + 2 s) * grid * sign rounded once to f16, activations are f16, products are
 * accumulated in fp32 (the order is the hardware's; this restatement sums in double and rounds once) */
void fnx_o_iq3s_dequant_f16(const uint8_t* src, size_t n, uint16_t* y);
void fnx_o_f32_f16(const float* x, size_t n, uint16_t* y);
/* jobs: {w, n, y[pf_job], out[pf_job]} ints; out[jobs.out[j] * nrows + row] = sum_k W_e[row][k] * x[jobs.y[j] * ldx + k] */
void fnx_o_moe_mma(const uint8_t* wbase, size_t w_stride, int nrows, int ncols, const int* jobs, int njobs, int pf_job,
                   const uint16_t* x, int ldx, float* out, int threads);
/* h = silu(gate) * up of stacked rows [gate (ffs) | up (ffs)], rounded to f16 (moe_mma.cuh:500-507) */
void fnx_o_swiglu_h16(const float* gu, int ffs, int P, uint16_t* h);
/* one MoE layer over a prompt chunk of C rows (prefill.cu:1990-2083 on one card, IQ3_S shared expert run as jobs of
 * all rows): router -> top-k -> BigJobs -> gate|up -> swiglu f16 -> down -> shared expert -> combine.
 * optional outputs may be null: topi/topw [C][topk], njobs */
void fnx_o_moe_prefill_layer(const fnx_o_moe_layer* L, const float* x, int C, int pf_job, float* out, float* logits, int* topi,
                             float* topw, int* njobs, int threads);

/* ---- around the MoE half (benchmark config 4): norms, dense Q8_0 projections, attention, the draft layer */
/* kernels.cu:2818-2826; the mean of squares summed in double */
void fnx_o_rms_norm_rows(const float* x, const float* w, float* y, int rows, int n, float eps);
/* ggml's Q8_0 in the reference's split layout (model.hpp:78-82): d = max|x| / 127 as f16, q = round(x / d) */
void fnx_o_quantize_q8_0_split(const float* w, int rows, int cols, int8_t* q, uint16_t* d);
/* dense.cuh:79-214: out[t * out_stride + r] = (s0 + s1) + (s2 + s3), s_q the q-th quarter of the columns with its
 * 32-column blocks folded in ascending order, acc = fmaf(d_w * d_x, (float) dot, acc) (the reference's term,
 * dense.cuh:196-200, in this build's fixed order, which the device follows bit for bit) */
void fnx_o_q8s_gemv(const int8_t* q, const uint16_t* d, int rows, int cols, const uint8_t* yq, float* out, int out_stride, int T);
typedef struct {
    float base;
    int scaled;
    float c_low, c_high, inv_scale, mscale;
} fnx_o_rope;
/* kernels.cu:513-537, 1878-1910: q and k heads RMS-normed (weights qn, kn) and NEOX-rotated on the first nrot dims at
 * positions pos0 + t, in place; k and v rounded to f16 into the cache rows [pos][nkv][hd] */
void fnx_o_attn_prep_append(float* qg, float* k, const float* v, const float* qn, const float* kn, uint16_t* kc, uint16_t* vc, int nq,
                            int nkv, int hd, int nrot, int T, int pos0, float eps, const fnx_o_rope* rope);
/* kernels.cu:541-643, 786-803 as textbook attention in double: row t over positions [0, pos0 + t], scores q.k / sqrt(hd),
 * out = softmax . v * sigmoid(gate); qg [T][nq][q | gate] */
void fnx_o_attn(const float* qg, const uint16_t* kc, const uint16_t* vc, float* out, int nq, int nkv, int hd, int T, int pos0);
typedef struct {
    const int8_t* q;
    const uint16_t* d;
    int n_out, n_in;
} fnx_o_q8s;
typedef struct {
    const float *attn_norm, *q_norm, *k_norm, *ffn_norm;
    fnx_o_q8s wq, wk, wv, wo;
    fnx_o_moe_layer moe;
    uint16_t *kc, *vc;
} fnx_o_dec_layer;
typedef struct {
    int n, nq, nkv, nlayers, vocab, max_ctx;
    float eps;
    fnx_o_rope rope;
    const fnx_o_dec_layer* layers;
    const float* out_norm;
    fnx_o_q8s head;
    const uint16_t* emb;
} fnx_o_decoder;
typedef struct {
    const float *norm_emb, *norm_hid, *out_norm;
    fnx_o_q8s fc_emb, fc_hid, head;
    fnx_o_dec_layer layer;
    /* engine.cu:2130-2131: the head's rows are the tokens [dv0, dv1) (both 0: the whole vocabulary); pen / pen_par (null: none):
     * the last row's penalty list (fnx_o_penalize_row's format, indexes relative to dv0), applied before the picks */
    int dv0, dv1;
    const int* pen;
    const float* pen_par;
} fnx_o_mtp;
/* the reduced decoder's window (engine.cu Engine::enqueue without streams, cards, GDN layers): hidden [T][n], logits
 * [T][vocab] (may be null), best [T] = argmax rows */
/* test probe: the next `layers` decoder layers run (by either function below) copy their router logits [T][nexp + 1] and
 * picks [T][topk] into consecutive slots of the two arrays; null pointers switch it off */
void fnx_o_layer_probe(float* logits, int* topi, int layers);
/* the next `layers` layers copy, to slot 0, 1, ... of the arrays given (any may be null): the rows going into the layer
 * [T][n], the attention's rows before the output projection [T][nq * 256], the rows after the attention half [T][n], the
 * MoE half's rows [T][n]. layers = 0 switches it off */
void fnx_o_layer_taps(float* x_in, float* att, float* x_mid, float* moe, int layers);
/* one layer (engine.cu: the body of the layer loop, attention half then MoE half) on the caller's rows, in place; L may be
 * one of D's layers or the draft layer's */
void fnx_o_decoder_layer(const fnx_o_decoder* D, const fnx_o_dec_layer* L, float* x, int T, int pos0, int threads);
void fnx_o_decoder_verify(const fnx_o_decoder* D, const int* tokens, int T, int pos0, float* hidden, float* logits, int* best, int threads);
/* engine.cu:2095-2133 without streams: R = fc_hid(rms(src)) + fc_emb(rms(emb[tokens])), one layer, norm, head, argmax */
void fnx_o_mtp_draft(const fnx_o_decoder* D, const fnx_o_mtp* M, const float* src, const int* tokens, int T, int pos0, float* hidden,
                     float* logits, int* best, int threads);

/* xorshift generator of the reference's self-test (selftest.cu:29-40) */
typedef struct { unsigned long long s; } fnx_o_rng;
void fnx_o_rng_init(fnx_o_rng* r, unsigned long long seed);
unsigned fnx_o_rng_next(fnx_o_rng* r);

int fnx_o_threads(void);

#ifdef __cplusplus
}
#endif
#endif
