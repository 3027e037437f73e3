/* fnx_mi355x.h - C ABI of the MI355X (gfx950) verify-path library.
 *
 * Every entry point replaces one operator of the reference engine's launch-wrapper API
 * (engine/src/kernels.hpp, namespace fnx) or one host function of its session loop (engine/src/session.cpp), cited
 * per declaration. Conventions kept from the reference:
 *   - activations are device float rows, one row per token or per routed pair t*topk+k; the shared expert's rows sit
 *     at T*topk+t (kernels.hpp:1-2, 277-282);
 *   - quantised weights are raw ggml blocks, row-major over output rows, expert e at p + e*stride or ep[e]
 *     (model.hpp:84-94);
 *   - work lists are device arrays of fnx_job with a device-resident count; the grid is sized without reading it;
 *   - `st` is a hipStream_t; every device call is asynchronous on it, allocates nothing and never synchronises, so a
 *     caller may capture a whole window into a graph (engine_common.cu:993-1007);
 *   - the caller owns every buffer.
 * Differences: functions return an int status (0 = ok) instead of throwing, the message is in fnx_last_error()
 * (thread-local); the reference's compile-time model constants (N, NEXP, TOPK) are run-time arguments.
 * Data faults go to a device error word as in the reference (bit 16: a non-finite logit seen by argmax).
 */
#ifndef FNX_MI355X_H
#define FNX_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FNX_MAXT 16        /* rows per verify window (model.hpp:43) */
#define FNX_PF_JOB 64      /* rows per prefill job (kernels.hpp:27-30) */
#define FNX_T_IQ3_S 21u    /* ggml type id (gguf.hpp:22-27) */
#define FNX_T_IQ3S_UNIT64 1021u /* this library's load-time re-laying of IQ3_S (fnx_iq3s_repack); not a ggml type */
#define FNX_T_IQ3S_TILE16 1022u /* the prompt path's own re-laying of IQ3_S (fnx_iq3s_tile16); not a ggml type */
#define FNX_IQ3S_BLOCK 110 /* bytes per 256 weights */
#define FNX_Q8_1_BLOCK 36  /* bytes per 32 activations: half d, half sum, int8 qs[32] */
#define FNX_ERR_BARRIER 4u    /* error-word bit (engine_impl.hpp:211-218: "a grid barrier timed out"): a block of the verify window gave up
                              * waiting for the blocks of its row (fnx_moe_ws.sync word 0) */
#define FNX_ERR_NONFINITE 16u /* error-word bit (engine_impl.hpp:211-218) */
#define FNX_ERR_WINDOW 32u    /* error-word bit: a window at a position outside its cache (below 0, or its last row past max_ctx);
                              * the attention then reads only cells that exist and the results mean nothing. No counterpart in the
                              * reference, whose positions are host integers that it checks before launching */

/* kernels.hpp:18-23 */
typedef struct fnx_job {
    int w;             /* matrix index: an expert, or 0 */
    int n;             /* rows of the job */
    int y[FNX_MAXT];   /* activation rows (q8_1) */
    int out[FNX_MAXT]; /* output rows */
} fnx_job;

/* kernels.hpp:32-37 */
typedef struct fnx_bigjob {
    int w;
    int n;
    int y[FNX_PF_JOB];
    int out[FNX_PF_JOB];
} fnx_bigjob;

/* model.hpp:84-94 (DW) without the split-Q8_0 twin, which this path does not use */
typedef struct fnx_dw {
    const void* p;          /* raw ggml blocks, row-major over output rows */
    uint32_t type;          /* FNX_T_IQ3_S (raw ggml blocks) or FNX_T_IQ3S_UNIT64 (after fnx_iq3s_repack); the decode
                             * operators (fnx_mmvq, fnx_moe_gate_up, fnx_moe_down, and fnx_moe_verify_layer operator by
                             * operator) also take ggml's Q4_0 (2), Q5_1 (7), Q8_0 (8), Q4_K (12), Q5_K (13), IQ4_NL (20) and IQ4_XS (23) rows, the
                             * other types of kernels.cu:2454-2471 that the reference's host code can decode; the
                             * prompt path's grouped GEMM and the one-launch window are IQ3_S only */
    int n_in, n_out;        /* columns, rows */
    size_t row_bytes;       /* n_in / 256 * 110 for IQ3_S; whole blocks of the type otherwise */
    const void* const* ep;  /* optional device table: expert e's matrix; null: expert e at p + e * stride */
} fnx_dw;

/* message of the calling thread's last failed call ("" if none) */
const char* fnx_last_error(void);
/* library build id, and whether a usable GPU is present (no device work is started) */
const char* fnx_version(void);

/* Load-time re-laying of IQ3_S weights, the counterpart of the reference's own load-time layouts (the split Q8_0
 * twin, model.hpp:78-82; tensor_convert.hpp): raw ggml block_iq3_s -> "unit64", the same 110 bytes per 256 weights
 * with each 32-weight sub-block's codes, high bits and signs merged into eight 13-bit codebook indexes. A tensor of
 * n_weights (a multiple of 2048) in memory order; dst may equal src. Afterwards describe the tensor with
 * fnx_dw.type = FNX_T_IQ3S_UNIT64: every operator below takes both types and gives the same results; the re-laid
 * type is the fast path. Rows must have 256, 512, 1024 or 2048 columns and expert strides must be multiples of 880. */
int fnx_iq3s_repack(const void* src, void* dst, size_t n_weights, void* st);
/* A second load-time layout, for the prompt path's matrix-core kernels (fnx_moe_gate_up_h16_mma over stacked gate|up
 * matrices, fnx_moe_down_mma over rows of 512 columns, fnx_moe_prefill_layer's gate|up and down) and the mat-vec operators'
 * jobs of many rows; no counterpart in the reference, whose prompt kernels read raw blocks: nmat matrices of nrows x ncols
 * (rows in 16s, columns in 512s) from the unit64 layout into tiles of 16 rows x 512 columns in which the 64 lanes of a
 * wave find their shares side by side (3,584 bytes a tile: 1.8 % more than the blocks). src: the matrices one after the
 * other in unit64 form; dst: another buffer of fnx_iq3s_tile16_bytes(nrows, ncols, nmat) bytes, expert e at
 * e * fnx_iq3s_tile16_bytes(nrows, ncols, 1). A fnx_dw over dst has type FNX_T_IQ3S_TILE16 (row_bytes as for IQ3_S). A
 * model served with both paths keeps both copies (288 GB hold them). */
int fnx_iq3s_tile16(const void* src, void* dst, int nrows, int ncols, int nmat, void* st);
size_t fnx_iq3s_tile16_bytes(int nrows, int ncols, int nmat);

/* kernels.hpp:41  quantize_q8_1: f32 rows of n -> q8_1 blocks, ggml's rounding (kernels.cu:131-145) */
int fnx_quantize_q8_1(const float* x, void* q, int n, int rows, void* st);

/* kernels.hpp:49  mmvq: out[job.out[j]][r] = W[job.w][r] . y[job.y[j]] for every job in jobs[0..*njobs)
 * (njobs null: njobs_max jobs). y: q8_1 rows of W->n_in. W (here and in fnx_moe_gate_up / fnx_moe_down): IQ3_S as ggml
 * blocks, as unit64, or as tile16 (rows in 16s, 512 .. 2048 columns in 512s; w_stride then counts that layout's bytes):
 * tile16 is the layout for jobs of many rows, whose weights go decoded straight into matrix-core operands, unit64 the
 * one for jobs of one or two rows. */
int fnx_mmvq(const fnx_dw* W, size_t w_stride, const fnx_job* jobs, const int* njobs, int njobs_max, const void* y,
             float* out, int out_stride, void* st);

/* kernels.hpp:54-55  gemv_f32 / gemv_bf16: y[t][r] = W[r] . x[t], W [rows][n], n % 256 == 0. The reference calls it
 * with T <= 16; any T is taken here (the prompt path's router logits are one call over a chunk's rows), every sum in
 * the same order of operations whatever T is. */
int fnx_gemv_f32(const float* W, const float* x, float* y, int rows, int n, int T, void* st);
int fnx_gemv_bf16(const uint16_t* W, const float* x, float* y, int rows, int n, int T, void* st);

/* kernels.hpp:79  route: logits [T][nexp] -> top-k (softmax, renormalised; ties to the lower index), the gate|up
 * jobs (rows = tokens, outputs = pairs t*topk+k) and the down jobs (rows = outputs = pairs); njobs[0] = njobs[1] =
 * the count. logits_stride: floats between rows (nexp, or nexp + 1 when the rows carry the shared gate's logit) */
int fnx_route(const float* logits, int logits_stride, int T, int nexp, int topk, int* topi, float* topw, fnx_job* jobs_gu,
              fnx_job* jobs_dn, int* njobs, void* st);

/* kernels.hpp:294  router_route: logits rows of nexp + 1 = W [nexp + 1][n] . x (the router's rows, then the shared
 * expert's gate), top-k per token by logit, weights the selected softmax renormalised, jobs as route. W: f32
 * (w_bf16 = 0) or bf16 bits (w_bf16 = 1). njobs[0] = the count; njobs[1] is left at zero as in the reference. */
int fnx_router_route(const void* W, int w_bf16, const float* x, float* logits, int T, int n, int nexp, int topk, int* topi,
                     float* topw, fnx_job* jobs_gu, fnx_job* jobs_dn, int* njobs, void* st);

/* kernels.hpp:81   swiglu_q8_1: h[r] = silu(g[r]) * u[r] -> q8_1, rows of n */
int fnx_swiglu_q8_1(const float* g, const float* u, void* q, int n, int rows, void* st);
/* kernels.hpp:349  swiglu_stacked_q8_1: T rows of [gate (ffs) | up (ffs)] -> q8_1 rows of ffs */
int fnx_swiglu_stacked_q8_1(const float* gu, void* hq, int ffs, int T, void* st);

/* kernels.hpp:319  moe_gate_up: gu rows of 2*ffs = A->n_out: [gate | up]; expert stride sa; xq: q8_1 rows of A->n_in,
 * one per row of the window: njobs_max / topk of them (njobs_max is the window's pairs, as in the reference, whose
 * launcher takes T = njobs_max / TOPK, kernels.cu:2449); the jobs' y index them */
int fnx_moe_gate_up(const fnx_dw* A, size_t sa, const fnx_job* jobs, const int* njobs, int njobs_max, const void* xq, float* gu,
                    int topk, void* st);
/* kernels.hpp:343  moe_down: part rows of A->n_out from silu(gate) * up of the gu rows (rows of 2 * A->n_in).
 * Like the reference (moe.cuh:592-594) the q8_1 rows of h live in one library-owned device buffer, so one MoE may be
 * in flight per device; njobs_max (the window's pairs) <= 176. */
int fnx_moe_down(const fnx_dw* A, size_t sa, const fnx_job* jobs, const int* njobs, int njobs_max, const float* gu, float* part,
                 void* st);
/* kernels.hpp:83   moe_combine: out[t] = sum_k topw[t][k] * part[t*topk + k] + sigmoid(sh_logit[t * stride]) * sh[t] */
int fnx_moe_combine(const float* part, const float* topw, const float* sh, const float* sh_logit, int sh_logit_stride, float* out,
                    int T, int n, int topk, void* st);

/* kernels.hpp:433  argmax: best[t] = (value, index + v0), the lowest index on ties. One launch: a row's last block to
 * arrive decodes the row's key. keys: FNX_ARGMAX_WORDS words, zeroed once (left at zero): a key a row, then a count of
 * arrived blocks a row - twice the reference's MAXT words (engine.cu:314). err bit 16: a logit was NaN or inf */
#define FNX_ARGMAX_WORDS (2 * FNX_MAXT)
int fnx_argmax(const float* logits, int rows, int T, int v0, float* best_v, int* best_i, unsigned long long* keys, unsigned* err,
               void* st);

/* session.hpp:55-58  lookup_drafts (host memory): the tokens after the latest earlier place of ctx's last key_n
 * tokens, if the first of them is d1 (d1 < 0: whatever it is), as many as the match is long, 3 to lk. key_n = 3 is
 * the reference's LOOKUP_N; 2 and 4 are this build's parameterisation. Returns the draft count (<= lk) or -1 on a
 * bad argument; *match (may be null) = the run's start or -1. */
int fnx_lookup_drafts(const int* ctx, int n_ctx, int key_n, int lk, int d1, int* out, int* match);
/* the same on device memory, asynchronous: ctx, d1, out (lk ints), n_out, match are device pointers; lk <= 64 */
int fnx_lookup_drafts_dev(const int* ctx, int n_ctx, int key_n, int lk, const int* d1, int* out, int* n_out, int* match, void* st);

/* session.cpp:573  greedy acceptance: n = 1; while (n < R && rows[n] == o[n-1]) ++n  (host memory) */
int fnx_accept_greedy(const int* rows, const int* o, int R);
/* the same on device memory, asynchronous: n_accept[0] = n */
int fnx_accept_greedy_dev(const int* rows, const int* o, int R, int* n_accept, void* st);

/* ---- the whole MoE half of a verify window (engine.cu:1569-1757 Engine::ffn_half without cards and streaming):
 * quantize -> router_route -> gate|up (routed + shared) -> swiglu q8_1 -> down (routed + shared) -> combine.
 * Same results as the calls above made one by one (up to the order of a few float additions). With unit64 experts,
 * n = 2048 and ff of 256, 512 or 1024 (and a GPU of at least 16 CUs a window row) the window is one launch: a window
 * row's blocks compute its router logits, rank it, run its gate|up sweeps (SwiGLU -> q8_1 rows of h) and its down trips
 * with the combine's chains, handing over within the row through the workspace's sync words (fnx_moe_ws.sync, zeroed
 * once); a block of the launch also writes the job lists for the caller. It touches only the caller's workspace, so
 * windows with workspaces of their own may run on different streams at once. Other shapes run operator by operator through the library's one pair buffer per device, like moe_down: the
 * library puts such calls in order across streams (not under graph capture). A row with fewer than topk logits above
 * -inf (masked or NaN entries) takes the lowest experts not yet taken for its remaining picks, at weight 0, so its picks
 * stay distinct and no job exceeds 16 rows (the reference's result is undefined there); fnx_router_route and
 * fnx_pf_route follow the same rule. */
/* model.hpp:78-82  Q8S: dense Q8_0 in the split layout: int8 values [n_out][n_in], f16 scale bits [n_out][n_in / 32] */
typedef struct fnx_q8s {
    const int8_t* q;
    const uint16_t* d;
    int n_out, n_in;
    int tiled;   /* 0: q is [n_out][n_in] as the reference's split layout (model.hpp:78-82); 1: q was re-laid by fnx_q8s_tile */
} fnx_q8s;
typedef struct fnx_moe_layer {
    int n, ff, nexp, topk;   /* hidden, expert width, experts, picks per token */
    const void* router;      /* [nexp + 1][n]: the router's rows, then the shared expert's gate */
    int router_bf16;         /* 0: f32, 1: bf16 bits */
    fnx_dw gu;               /* routed gate|up: n_out = 2 ff, n_in = n */
    size_t gu_stride;        /* bytes between experts */
    fnx_dw down;             /* routed down: n_out = n, n_in = ff */
    size_t down_stride;
    fnx_dw sh_gu;            /* shared expert gate|up */
    fnx_dw sh_down;          /* shared expert down */
    /* the shared expert as dense split Q8_0 (model.hpp:84-94, DW::s; engine.cu:1600-1604 runs it as q8s_gemv ->
     * swiglu_stacked_q8_1 -> q8s_gemv): when both q pointers are set these are used and sh_gu / sh_down are not read */
    fnx_q8s sh_gu_q8;        /* n_out = 2 ff, n_in = n */
    fnx_q8s sh_down_q8;      /* n_out = n, n_in = ff */
} fnx_moe_layer;
/* caller-owned scratch for one window; sizes from fnx_moe_ws_bytes */
typedef struct fnx_moe_ws {
    void* xq;        /* q8_1 rows of x: T * n/32 * 36 bytes */
    float* logits;   /* [T][nexp + 1] */
    int* topi;       /* [T][topk] */
    float* topw;     /* [T][topk] */
    fnx_job* jobs_gu;/* [T * topk + 1] (the last one is the shared expert's) */
    fnx_job* jobs_dn;/* [T * topk + 1] */
    int* njobs;      /* [2], zeroed once */
    float* gu;       /* [T * topk + T][2 ff] floats. Operator by operator: the gate|up outputs. The one-launch window keeps
                      * the pairs' h there instead, as q8_1 rows of its own record size, and never writes f32 gate|up rows */
    float* part;     /* [T * topk + T][n] floats. Operator by operator: the down outputs. The one-launch window uses it only
                      * as scratch for a split-Q8_0 shared expert */
    unsigned* sync;  /* [FNX_MOE_SYNC_WORDS], 8-byte aligned, zeroed once: the arrival counters and the marked words through which
                      * the blocks of the one-launch window hand over within a window row (every window leaves them zero), and
                      * in word 0 the window's error bits:
                      * FNX_ERR_BARRIER if a block gave up waiting for its row (kernels.cu:884, 899 bound the reference's device waits
                      * the same way). After that error the results mean nothing and the words must be zeroed again */
} fnx_moe_ws;
#define FNX_MOE_SYNC_WORDS 33568
int fnx_moe_verify_layer(const fnx_moe_layer* L, const float* x, int T, float* out, const fnx_moe_ws* ws, void* st);
/* The same window without a workspace argument and without any allocation: no counterpart in the reference. For callers
 * that cannot allocate device memory (code under graph capture, serving loops and harnesses that forbid it): the scratch
 * of fnx_moe_ws lives in one array of FNX_MOE_STATIC_WS_BYTES in the library's device image, which each GPU the library
 * runs on holds until the process ends. Only the one-launch window runs on it: unit64 experts, hidden 2048, ff 256,
 * 512 or 1024, up to 1024 experts, up to 16 picks a row, T x topk <= 160; anything else is refused with a message. x and
 * out are the caller's, as above; results are those of fnx_moe_verify_layer bit for bit. All calls on a GPU share that
 * GPU's array: two of them in flight at once (two streams, two threads) race. */
#define FNX_MOE_STATIC_WS_BYTES (576 * 1024)
int fnx_moe_verify_layer_static(const fnx_moe_layer* L, const float* x, int T, float* out, void* st);
/* The error word of that array's windows (fnx_moe_ws.sync word 0 of the library's own workspace on the current device),
 * for the caller who cannot see it otherwise: waits for the stream, copies the word to *err and, if FNX_ERR_BARRIER is set
 * there, zeroes the array's sync words so that the next window starts clean. Not for the hot path (it synchronises). */
int fnx_moe_static_status(unsigned* err, void* st);
/* Profiling aid, the counterpart of the reference's FNX_PROF stamps in its window graph (engine.cu:1382-1530):
 * fnx_layer_profile(1) makes the one-launch window record events on its stream around its launch (not to be used under
 * graph capture), fnx_layer_profile(0) stops that; fnx_layer_profile_read waits for the last recorded window and returns two
 * durations in milliseconds: [0] what runs before the window's launch (the three dense launches of a split-Q8_0 shared
 * expert; next to nothing otherwise), [1] the window's launch (router, top-k, gate|up, SwiGLU, down, combine). One profiled
 * window at a time per process. */
int fnx_layer_profile(int on);
int fnx_layer_profile_read(float* ms2);
/* Calibration aid (no counterpart in the reference): one read-only pass over `bytes` of device memory, nothing decoded,
 * so that the expert mat-vec launches can be judged against what the memory system gives a plain read of the same shape.
 * variant: 0 / 1 / 7 / 8: 16-byte loads a lane, 4 / 8 / 16 / 2 in flight, every wave one contiguous range; 2 / 3: the same 4 / 8
 * with the 1 KiB chunks dealt round-robin to the waves; 4: 8-byte loads, 8 in flight; 5: as 1 with nontemporal loads;
 * 6: the unit64 planes as the expert kernels load them (five loads a unit and lane, a group of four units in flight), every
 * wave one contiguous range; 9: the groups dealt round-robin to the grid's waves; 10: every block one contiguous range,
 * its waves taking the groups in turn; 11 / 12 / 13: as 6 / 9 / 10 with nontemporal loads; 14 / 15: four units as one lane-interleaved
 * record of 3,520 bytes (six loads a lane of 16, 16, 16, 4, 4 and 8 bytes), the records dealt round-robin to the grid's waves, plain / nontemporal; 1000 s + K (s = 1 .. 8, K = 1 .. 64
 * dividing 64 s): the buffer as matrices of 256 s units (s = 4: a gate|up matrix of the benchmark's shape, 2: a down matrix)
 * read in a shuffled order, a wave staying with a matrix for K trips of four units. sink: one device word (never written in
 * practice; it keeps the loads alive). */
int fnx_stream_read(const void* p, size_t bytes, int variant, int blocks, int threads, void* sink, void* st);

/* ---- the prompt path's MoE over a chunk of C rows (prefill.cu:1990-2083) */
/* prefill.cu:288-377  k_pf_top10 / k_pf_count / k_pf_jobbase / k_pf_fill in one call: top-k and weights per row,
 * cnt [nexp] pairs per expert, jbase [nexp] each expert's first job, jobs of up to FNX_PF_JOB rows per expert with
 * the pairs in ascending order (gate|up: y = row, out = pair; down: y = out = pair), njobs[0] = the job count.
 * njobs_cap = capacity of the job arrays; C * topk / FNX_PF_JOB + nexp is always enough. */
int fnx_pf_route(const float* logits, int logits_stride, int C, int nexp, int topk, int* topi, float* topw, int* cnt, int* jbase,
                 fnx_bigjob* jobs_gu, fnx_bigjob* jobs_dn, int njobs_cap, int* njobs, void* st);
/* kernels.hpp (p100_f32_f16): f32 -> f16, round to nearest even */
int fnx_f32_f16(const float* x, size_t n, uint16_t* out, void* st);
/* kernels.hpp:324-325  moe_gate_up_big, moe_down_big: the prompt path's jobs over q8_1 activations (the reference's moe_q8
 * mode of the prompt pass, prefill.cu:1842-1844) - fnx_moe_gate_up's and fnx_moe_down's terms (mmvq semantics: integer dot
 * products of a sub-block, then d_w (1 + 2 s) d_x) for jobs of up to FNX_PF_JOB rows. gate_up: gu[jobs.out][2 ffs] from the
 * q8_1 rows xq[jobs.y] of A->n_in values; down: part[jobs.out][n] from h = silu(gate) * up of the rows gu[jobs.y] ([gate |
 * up] of 2 * A->n_in floats), quantised to q8_1 on the way (moe.cuh:597-608). tile16 matrices (rows in 16s, 512 .. 2048
 * columns in 512s), 1 .. 4096 jobs a launch; a job's rows go sixteen at a time through the int8 matrix cores. The two
 * families of prompt kernels - these and the f16 ones below - differ by the activations' q8_1 rounding: a caller's choice,
 * as the reference's. */
int fnx_moe_gate_up_big(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const void* xq, float* gu,
                        void* st);
int fnx_moe_down_big(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const float* gu, float* part,
                     void* st);
/* kernels.hpp:328  moe_gate_up_mma: gu[jobs.out][2 ffs] = W_e[2 ffs][n] . xh[jobs.y] with f16 weights (each the f32
 * value rounded once), f16 activations, fp32 accumulation, on the matrix cores. xh rows of A->n_in halves. Raw blocks and
 * unit64 (tile16 gate|up matrices go through fnx_moe_gate_up_h16_mma, which leaves h). */
int fnx_moe_gate_up_mma(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const uint16_t* xh, float* gu,
                        void* st);
/* kernels.hpp:329  swiglu_h16: h16[p][ffs] = f16(silu(gate) * up) of the P stacked rows [gate | up] */
int fnx_swiglu_h16(const float* gu, int ffs, int P, uint16_t* h16, void* st);
/* kernels.hpp:328 + 329 in one launch: h16[jobs.out][ffs] = f16(silu(gate) * up) of the products, which are not written.
 * For tile16 matrices (2 ffs rows in 32s, columns in 512s; an error otherwise); fnx_moe_prefill_layer uses it where it
 * can. The products are fnx_moe_gate_up_mma's up to the order in which a row's f16 products are added. */
int fnx_moe_gate_up_h16_mma(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const uint16_t* xh,
                            uint16_t* h16, void* st);
/* kernels.hpp:330  moe_down_mma: part[jobs.out][n] = W_e[n][ffs] . h16[jobs.y]. Raw blocks, unit64, or tile16 with
 * ffs = 512 */
int fnx_moe_down_mma(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const uint16_t* h16, float* part,
                     void* st);
/* caller-owned scratch for one chunk; P = C * topk, J = P / FNX_PF_JOB + nexp, S = ceil(C / FNX_PF_JOB) */
typedef struct fnx_pf_ws {
    float* logits;        /* [C][nexp + 1] */
    int* topi;            /* [C][topk] */
    float* topw;          /* [C][topk] */
    int* cnt;             /* [nexp] */
    int* jbase;           /* [nexp] */
    fnx_bigjob* jobs_gu;  /* [J + S]: the routed jobs, then (at J) the shared expert's */
    fnx_bigjob* jobs_dn;  /* [J + S] */
    int* njobs;           /* [2]: routed jobs, shared jobs */
    uint16_t* xh;         /* [C][n] f16 */
    float* gu;            /* [P + C][2 ff] */
    uint16_t* h16;        /* [P + C][ff] */
    float* part;          /* [P + C][n] */
} fnx_pf_ws;
/* the MoE half of a prompt chunk on one GPU (prefill.cu:1990-2083: router -> top-k -> jobs -> gate|up -> swiglu ->
 * down -> shared expert -> weighted sum); the shared expert (IQ3_S) runs as jobs over all rows through the same
 * kernels. out [C][n]. */
int fnx_moe_prefill_layer(const fnx_moe_layer* L, const float* x, int C, float* out, const fnx_pf_ws* ws, void* st);

/* ---- the rest of a verify step around the MoE half: norms, dense projections, attention, the draft layer
 * (benchmark config 4: a reduced decoder of attention + MoE layers and the MTP draft layer). Head width 256, the first
 * 64 dims rotated (model.hpp:41). */
/* kernels.hpp:406  rms_norm_rows: y[r] = x[r] / sqrt(mean(x[r]^2) + eps) * w */
int fnx_rms_norm_rows(const float* x, const float* w, float* y, int rows, int n, float eps, void* st);
/* x[r] += add[r] (add may be null); xn[r] = rms_norm(x[r]) * w; xq[r] = q8_1 of xn[r] (xn, xq may be null): the residual
 * add, rms_norm_rows and quantize_q8_1 that follow one another between a layer's halves (engine.cu's hc_read takes
 * the same place in the reference), one pass over each row; the values are the three operators' bit for bit. n <= 4096 */
int fnx_add_norm_q8(float* x, const float* add, const float* w, float* xn, void* xq, int rows, int n, float eps, void* st);
/* the same with the MoE half's combine (kernels.hpp's moe_combine, kernels.cu:412-419) as what is added: x[r] += sum_k
 * topw[r][k] part[r topk + k] + sigmoid(sh_logit[r]) sh[r], then norm and q8_1 as above - fnx_moe_combine followed by
 * fnx_add_norm_q8 in one launch, their values bit for bit (the decoder's layers hand over this way) */
int fnx_combine_add_norm_q8(const float* part, const float* topw, const float* sh, const float* sh_logit, int sh_logit_stride, int topk, float* x,
                            const float* w, float* xn, void* xq, int rows, int n, float eps, void* st);
/* y = a + b over n floats */
int fnx_add_rows(const float* a, const float* b, float* y, size_t n, void* st);
/* rows tokens[t] of an f16 table [vocab][n] as f32 (the window's input rows) */
int fnx_embed_rows(const uint16_t* emb, const int* tokens, int T, int vocab, int n, float* y, void* st);
/* A load-time layout of a dense matrix's int8 values, the counterpart of the reference's own load-time split (model.hpp:
 * 78-82): tiles of 16 rows, a tile its 64-column steps one after another (1 KiB each, a wave's lanes' 16-byte shares side
 * by side), so that the mat-vec below streams whole cache lines (the output head: 4.7 against 4.1 TB/s). src [rows][cols]
 * int8 -> dst, another buffer of fnx_q8s_tile_bytes(rows, cols) bytes (rows padded to 16); the scales stay as they are; a
 * fnx_q8s over dst has tiled = 1. Both layouts give the same bits. cols a multiple of 256. */
int fnx_q8s_tile(const int8_t* src, int8_t* dst, int rows, int cols, void* st);
size_t fnx_q8s_tile_bytes(int rows, int cols);
/* dense.cuh:79-214 (q8s_gemv): out[t * out_stride + r] = W[r] . y[t] for T <= 16 q8_1 rows; n_in a multiple of 256. The
 * result is (s0 + s1) + (s2 + s3), s_q the q-th quarter of the columns, its 32-column blocks folded in ascending order with
 * acc = fmaf(d_w * d_x, (float) dot, acc) */
int fnx_q8s_gemv(const fnx_q8s* W, const void* yq, float* out, int out_stride, int T, void* st);
/* kernels.hpp:414-418 (q8s_gemv_segs): n (1..3) matrices of the same columns over the same rows in one launch, each
 * output as q8s_gemv of that matrix alone gives it; all but the last matrix hold a multiple of 16 rows */
int fnx_q8s_gemv_segs(const fnx_q8s* const* W, float* const* out, const int* out_stride, int n, const void* yq, int T, void* st);
/* rope.hpp:22-39  the rotary's constants (scaled = 0: plain frequencies base^(-2 i / 64), mscale 1) */
typedef struct fnx_rope {
    float base;
    int scaled;
    float c_low, c_high, inv_scale, mscale;
} fnx_rope;
/* kernels.hpp:259  attn_prep_append: q heads (qg [T][nq][q | gate], 2 x 256 each) and k heads RMS-normed with their
 * weights and rotated at positions *pos0 + t, in place; k and v appended to the f16 caches of max_ctx positions (a
 * multiple of 8, under 4 GiB a cache): K is [position][nkv][256]; V is this library's own layout [position / 8][nkv][256][position % 8]
 * (eight positions of a dimension together: 16 bytes, the matrix-core attention's operand of one lane). */
int fnx_attn_prep_append(float* qg, float* k, const float* v, const float* q_norm, const float* k_norm, uint16_t* kc, uint16_t* vc, int nq,
                         int nkv, int T, const int* pos0, int max_ctx, float eps, const fnx_rope* rope, void* st);
/* kernels.hpp:238  attn: row t attends positions [0, *pos0 + t]; out [T][nq][256] = softmax(q k / 16) v * sigmoid(gate).
 * On the matrix cores: q and the probabilities enter as two f16 terms each (hi + lo), the cache is f16, sums are fp32. max_ctx: the caches' capacity (the grid
 * covers it; *pos0 + T <= max_ctx). scratch: fnx_attn_scratch_floats(nq, T, max_ctx) floats (the splits' partial sums) */
size_t fnx_attn_scratch_floats(int nq, int T, int max_ctx);
int fnx_attn(const float* qg, const uint16_t* kc, const uint16_t* vc, float* out, int nq, int nkv, const int* pos0, int T, int max_ctx,
             float* scratch, void* st);
/* one decoder layer of the reduced model: x += wo . attn(norm(x)); x += moe(norm(x)) */
typedef struct fnx_dec_layer {
    const float *attn_norm, *q_norm, *k_norm, *ffn_norm;   /* [n], [256], [256], [n] */
    fnx_q8s wq, wk, wv, wo;                                 /* [nq * 512][n], [nkv * 256][n], [nkv * 256][n], [n][nq * 256] */
    fnx_moe_layer moe;
    uint16_t *kc, *vc;                                      /* this layer's caches, max_ctx x nkv x 256 f16 each (layouts: attn_prep_append) */
} fnx_dec_layer;
typedef struct fnx_decoder {
    int n, nq, nkv, nlayers, vocab, max_ctx;
    float eps;
    fnx_rope rope;
    const fnx_dec_layer* layers;   /* host array of nlayers */
    const float* out_norm;         /* [n] */
    fnx_q8s head;                  /* [vocab][n] */
    const uint16_t* emb;           /* [vocab][n] f16 */
} fnx_decoder;
/* caller-owned scratch for windows of up to 16 rows */
typedef struct fnx_dec_ws {
    float *x, *xn, *qg, *k, *v, *att, *o;   /* [T][n], [T][n], [T][nq*512], [T][nkv*256] x2, [T][nq*256], [T][n] */
    float* attn_scratch;                    /* fnx_attn_scratch_floats(nq, T, max_ctx) */
    void* xq;                               /* q8_1 rows of max(n, nq * 256) values */
    float *hidden, *logits, *best_v;        /* [T][n] (the rows before the output norm), [T][vocab], [T] */
    int* best_i;                            /* [T] */
    unsigned long long* keys;               /* [FNX_ARGMAX_WORDS], zero */
    unsigned* err;                          /* [1] */
    fnx_moe_ws moe;
} fnx_dec_ws;
/* engine.cu (Engine::enqueue, reduced): the window's rows through every layer, the output norm, the head and argmax:
 * ws->hidden, ws->logits, ws->best_i. tokens: device, T ids; their K/V go to positions *pos0 + t. */
int fnx_decoder_verify(const fnx_decoder* D, const int* tokens, int T, const int* pos0, const fnx_dec_ws* ws, void* st);
/* engine.cu (Engine::enqueue): the body of its layer loop, one layer on rows the caller gives (x: device, [T][n]; L: one of D's
 * layers or the draft layer's). Leaves in the workspace what the layer loop hands on: ws->x = x + the attention half's
 * rows, ws->xq = the attention's rows in q8_1 form (what the output projection read), ws->xn = the normed rows the MoE
 * half read, ws->o = the MoE half's rows (the next layer's first pass adds them); the layer's K and V rows go into its
 * caches at *pos0 + t. For callers that drive the layers themselves, and for layer-by-layer comparisons. */
int fnx_decoder_layer(const fnx_decoder* D, const fnx_dec_layer* L, const float* x, int T, const int* pos0, const fnx_dec_ws* ws, void* st);
/* engine.cu:2095-2133 (mtp_enqueue, without hyper-connection streams): R = fc_hid(rms(src)) + fc_emb(rms(emb[tokens])),
 * one decoder layer (its own cache), the output norm, the head, argmax. src: [T][n] hidden rows (the verify's, or the
 * draft layer's own for a chain). ws->hidden receives the layer's output rows. */
typedef struct fnx_mtp {
    const float *norm_emb, *norm_hid, *out_norm;   /* [n] each */
    fnx_q8s fc_emb, fc_hid, head;                  /* [n][n], [n][n], [dv1 - dv0][n] */
    fnx_dec_layer layer;
    /* model.hpp:233-243, engine.cu:2130-2131: the head's rows are the tokens [dv0, dv1) of the vocabulary (a card's share of
     * the draft head); dv0 == dv1 == 0: all of it. Rows of ws->logits then have dv1 - dv0 values, and the picks are token ids
     * (dv0 added, as argmax's v0). pen / pen_par (null: none): the LAST row's penalty list in fnx_penalize_row's format, its
     * indexes relative to dv0 (engine_common.cu:1602), applied to that row's logits in place before the picks. */
    int dv0, dv1;
    const int* pen;
    const float* pen_par;
} fnx_mtp;
int fnx_mtp_draft(const fnx_decoder* D, const fnx_mtp* M, const float* src, const int* tokens, int T, const int* pos0, const fnx_dec_ws* ws,
                  void* st);

/* ---- a greedy decode round that the host only enqueues. session.cpp:530-679 (Session::generate) drives these steps
 * from the host and waits for each; the reference's captured windows (engine_common.cu:993-1021) still hand the picks to
 * the host for acceptance. Here the acceptance (session.cpp:565-573), the commit, the draft layer's pass over the rows
 * kept (engine.cu:2095-2133) and the prompt lookup (session.cpp:428-447) read and leave their results in device words,
 * so no argument of a round changes from one round to the next: rounds can be enqueued back to back, or captured once in
 * a graph and replayed. When the lookup finds nothing the MTP chain follows (session.cpp:666-678, at a fixed length
 * fnx_round.chain; the reference's adaptive length and its min_p cut are the host's): each further draft is the draft
 * layer's pick for the draft before, from its own hidden row. Its launches are always enqueued; in a round whose lookup
 * found drafts their kernels leave at once on a device word. */
enum {
    FNX_RS_NCTX = 0,     /* tokens in ctx: the prompt and everything emitted */
    FNX_RS_POS = 1,      /* cache position of the window's first row (= FNX_RS_NCTX - 1) */
    FNX_RS_ROWS = 2,     /* rows of the window that count: 1 + the drafts */
    FNX_RS_ACCEPTED = 3, /* tokens the last round kept */
    FNX_RS_POS_PREV = 4, /* the last window's position */
    FNX_RS_ROUNDS = 5,   /* rounds done */
    FNX_RS_STOP = 6,     /* set once the next window would not fit the caches or ctx: later rounds change nothing */
    FNX_RS_CHAIN = 7,    /* 1 while this round's MTP chain runs (the lookup found nothing), else 0 */
    FNX_RS_CHAIN_POS = 8, /* FNX_MAXT words: the cache positions of the chain's steps */
    FNX_RS_WORDS = 24
};
typedef struct fnx_round {
    int* state;    /* device, FNX_RS_WORDS ints (the caller sets NCTX, POS, ROWS and zeroes the others) */
    int* rows;     /* device, FNX_MAXT ints: the window: the context's last token, then the drafts, then zeros */
    int* ctx;      /* device, ctx_cap ints: the prompt, then every token emitted */
    int ctx_cap;
    int* log;      /* device, log_cap x 2 ints (drafts offered, tokens kept) a round, or null */
    int log_cap;
    int speculate; /* 0: plain greedy decoding, one row a round (no draft layer, no lookup) */
    int key_n, lk; /* prompt lookup: tokens in the key (3 in the reference), most drafts (<= FNX_MAXT - 1) */
    int* scratch;  /* device, FNX_MAXT ints */
    int chain;     /* drafts of an MTP chain (the reference's K), 1 .. FNX_MAXT - 1; 0 counts as 1 */
    float* chain_src; /* device, n floats (the hidden row the chain starts from); may be null when chain <= 1 */
} fnx_round;
/* one round: fnx_decoder_verify over the window -> acceptance and commit -> fnx_mtp_draft over the rows kept -> lookup
 * -> the next window. Expert weights must be in the unit64 layout and hidden = 2048 (the one-launch window), since only
 * that routes a row count held on the device. The draft layer uses the same workspace after the verify. */
int fnx_decode_round(const fnx_decoder* D, const fnx_mtp* M, const fnx_round* R, const fnx_dec_ws* ws, void* st);

/* ---- the sampler: the non-greedy half of acceptance.
 * kernels.hpp:434-447 + topk.cuh (top_tokens): per row t < T of logits (n of the vocabulary from token v0) the row's
 * logit_bias (bias_n[t] of them from bias_off[t] in bias_tok / bias_val, each token once) and penalties (pen_n[t] tokens
 * and their counts at row t * pen_stride; pen_par: per row repeat, freq, present: a non-positive logit times repeat, a
 * positive one divided by it, then minus count * freq and minus present) applied IN PLACE, then the row's FNX_TOPK_N
 * highest into out_v / out_i (logit descending, token id ascending on ties, however many tie). err bit 16: a logit was NaN
 * or inf before the penalties. pen_n and bias_n may be null (no such lists). n >= FNX_TOPK_N, n <= 327,680. The slices'
 * candidates pass between the two launches in one library-owned device buffer: one top_tokens in flight per device. */
#define FNX_TOPK_N 64
int fnx_top_tokens(float* logits, int n, int T, int v0, const int* pen_tok, const int* pen_cnt, const int* pen_n, int pen_stride,
                   const float* pen_par, const int* bias_tok, const float* bias_val, const int* bias_off, const int* bias_n, float* out_v,
                   int* out_i, unsigned* err, void* st);
/* kernels.hpp:434-436 penalize_row: pen = {k, k indexes into the row, their k counts}, par = {repeat, freq, present};
 * k <= 4096 (engine.hpp:73 PEN_CAP; a greater count is cut there, as is a bias list's) */
int fnx_penalize_row(float* row, int n, const int* pen, const float* par, void* st);
/* session.hpp:17-26 Sampling, the values the distribution is made from (temperature > 0: greedy rows do not come here) */
typedef struct fnx_sampling {
    float temperature, top_p, min_p;
    int top_k;   /* 0: no cut */
} fnx_sampling;
/* session.cpp:41-75 make_dist (host): a row's distribution from its candidates in top_tokens' order: top_k, then top_p
 * over the untempered softmax of those (in double), then min_p as a logit threshold, then the temperature's softmax over
 * the survivors. Returns how many survive (ids, p filled; both hold ncand), or -1. */
int fnx_make_dist(const float* cand_v, const int* cand_i, int ncand, const fnx_sampling* s, int* ids, double* p);
/* session.cpp:77-84 draw (host): the token at u in [0, 1) */
int fnx_draw(const int* ids, const double* p, int n, double u);
/* session.cpp:574-613 (host): speculative sampling over a window. cand_v / cand_i: T rows of ncand candidates; rows[0] the
 * window's first token, rows[j + 1] draft j, drawn from q_j = (q_ids, q_p)[j * q_stride ..][q_n[j]] (q_n null or
 * q_n[j] = 0: a fixed draft, all of q_j on it). Draft j stands with probability min(1, p_j / q_j); else row j's token is
 * drawn from max(0, p_j - q_j) normalized and the window ends there; all standing: one more from the last row. The
 * uniforms come from u in the order they are used (the reference draws them from its mt19937_64 as it goes); *used_u =
 * how many were. Returns the tokens emitted n (o[0 .. n)), or -1. */
int fnx_accept_sampled(const float* cand_v, const int* cand_i, int ncand, int T, const int* rows, const fnx_sampling* s, const int* q_ids,
                       const double* q_p, const int* q_n, int q_stride, const double* u, int nu, int* o, int* used_u);

/* ---- GGUF ingestion of a layer's experts (host code; the file format either side of the path).
 * gguf.hpp:25-45 (Tensor, Gguf), gguf.cpp:219-320 (load_shard: the header walk and its checks, exercised by
 * tools/gguf_test.cpp): a file, and the "-0000N-of-0000M" shards beside it, mapped read-only and indexed by tensor
 * name; metadata of the first shard. A header that does not add up is refused with a message naming the tensor. */
typedef struct fnx_gguf fnx_gguf;
typedef struct fnx_gguf_tensor {
    const char* name;   /* lives as long as the handle */
    uint32_t type;      /* ggml type id (21 = IQ3_S, 0 = F32, 30 = BF16, 8 = Q8_0 ...) */
    int n_dims;
    int64_t ne[4];      /* ne[0] = values a row; unused dimensions are 1 */
    const void* data;   /* in the mapping */
    size_t nbytes;
    int shard;          /* which file, and where in it */
    uint64_t offset;
} fnx_gguf_tensor;
fnx_gguf* fnx_gguf_open(const char* first_shard);   /* null on failure: fnx_last_error() */
void fnx_gguf_close(fnx_gguf* g);
int fnx_gguf_shards(const fnx_gguf* g);
int fnx_gguf_count(const fnx_gguf* g);                                        /* tensors over all shards */
int fnx_gguf_at(const fnx_gguf* g, int i, fnx_gguf_tensor* t);                /* the i-th in name order */
int fnx_gguf_find(const fnx_gguf* g, const char* name, fnx_gguf_tensor* t);   /* 0: found; 1: no such tensor */
size_t fnx_gguf_row_bytes(const fnx_gguf_tensor* t);                          /* bytes of one ne[0] row; 0 for an unknown type */
int fnx_gguf_key_type(const fnx_gguf* g, const char* key);                    /* the GGUF value type of a key of the first shard, or -1 */
int fnx_gguf_int(const fnx_gguf* g, const char* key, int64_t* v);             /* 0: ok; 1: no such integer key */
int fnx_gguf_num(const fnx_gguf* g, const char* key, double* v);              /* a number, integer or float as writers differ */
const char* fnx_gguf_str(const fnx_gguf* g, const char* key);                 /* null: no such string key */
/* model.cpp:722-741 expert_rows2: per expert, rows [r0, r1) of gate then of up, expert-major, into host memory dst
 * (null: only *w's shape, *stride and the byte count are worked out). Returns 0 and fills w (w->p = dst) and stride. */
int fnx_gguf_expert_rows2(const fnx_gguf_tensor* gate, const fnx_gguf_tensor* up, int r0, int r1, void* dst, size_t dst_bytes, fnx_dw* w,
                          size_t* stride, size_t* bytes);
/* model.cpp:768-790 expert_cols: per expert, every row's columns [c0, c1) (whole blocks of the tensor's type: multiples
 * of 256 for IQ3_S; the reference counts 32-value blocks and so cannot slice an IQ3_S row at all) */
int fnx_gguf_expert_cols(const fnx_gguf_tensor* down, int c0, int c1, void* dst, size_t dst_bytes, fnx_dw* w, size_t* stride, size_t* bytes);
/* one layer's MoE block from "blk.<layer>.": ffn_gate_inp(.weight) + ffn_gate_inp_shexp -> router rows (F32 or BF16 in the
 * file, f32 on the device); ffn_gate_exps / ffn_up_exps rows [ff0, ff1) -> gate|up; ffn_down_exps columns [ff0, ff1) ->
 * down; the _shexp tensors likewise (model.cpp:988-989, 1063-1068 without the card split's other half). Experts in
 * IQ3_S are uploaded into the caller's device buffers and re-laid there (fnx_iq3s_repack), so *L is ready for
 * fnx_moe_verify_layer / fnx_moe_prefill_layer; a layer with any tensor in Q4_0, Q5_1, Q8_0, IQ4_NL, IQ4_XS, Q4_K or Q5_K is left as the
 * file has it (fnx_moe_verify_layer then runs operator by operator; the prompt path needs IQ3_S). The upload is synchronous; the re-laying runs on st.
 * topk <= 0: taken from "<general.architecture>.expert_used_count". */
typedef struct fnx_moe_bufs {
    void *router, *gu, *down, *sh_gu, *sh_down;   /* device */
    size_t router_bytes, gu_bytes, down_bytes, sh_gu_bytes, sh_down_bytes;
} fnx_moe_bufs;
int fnx_gguf_moe_layer_bytes(const fnx_gguf* g, int layer, int ff0, int ff1, fnx_moe_bufs* sizes);
int fnx_gguf_load_moe_layer(const fnx_gguf* g, int layer, int ff0, int ff1, int topk, const fnx_moe_bufs* dev, fnx_moe_layer* L, void* st);
#ifdef __cplusplus
}
#endif
#endif
