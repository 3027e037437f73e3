/* CPU oracle: see fnx_oracle.h. TEST INFRASTRUCTURE ONLY - never linked into the device library.
 * Build: gcc -O2 -ffp-contract=off -fopenmp -fPIC -shared (oracle/Makefile). -ffp-contract=off matters: every fused
 * multiply-add below is written as fmaf() on purpose, everything else must stay an unfused multiply and add. */
#include "fnx_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#include "../include/fnx_expf.h" /* the one exp both sides use, fixed operation by operation */
#include "iq3s_grid.h"

#define IQ3S_BLOCK 110
#define Q8_1_BLOCK 36

int fnx_o_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---------------------------------------------------------------- half <-> float (tensor_convert.hpp:23-50) */
float fnx_o_h2f(uint16_t h) {
    const uint32_t sign = (h >> 15) & 1u, ex = (h >> 10) & 31u, man = h & 1023u;
    float f;
    if (ex == 0) f = ldexpf((float) man, -24);
    else if (ex == 31) f = man ? NAN : INFINITY;
    else f = ldexpf((float) (man + 1024u), (int) ex - 25);
    return sign ? -f : f;
}

uint16_t fnx_o_f2h(float x) { /* round to nearest even */
    uint32_t b;
    memcpy(&b, &x, 4);
    const uint32_t sign = (b >> 16) & 0x8000u, ex = (b >> 23) & 0xFFu, man = b & 0x7FFFFFu;
    if (ex == 0xFF) return (uint16_t) (sign | 0x7C00u | (man ? 0x200u : 0u));
    const int ne = (int) ex - 127 + 15;
    if (ne >= 31) return (uint16_t) (sign | 0x7C00u);
    if (ne <= 0) {
        if (ne < -10) return (uint16_t) sign;
        const uint32_t mm = (man | 0x800000u) >> (1 - ne);
        uint32_t r = mm >> 13;
        const uint32_t rem = mm & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r;
        return (uint16_t) (sign | r);
    }
    uint32_t r = ((uint32_t) ne << 10) | (man >> 13);
    const uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r;
    return (uint16_t) (sign | r);
}

/* IEEE round-to-nearest-even for every input, subnormal results included: what the device conversions (__float2half,
 * kernels.cu:131-145, moe_mma.cuh:500-507, moe_mma_iq.cuh) do. The host routine above (tensor_convert.hpp:31-49) drops
 * the bits it shifts out before it rounds a subnormal result, so the two differ on a few subnormal inputs. */
uint16_t fnx_o_f2h_rn(float x) {
    uint32_t b;
    memcpy(&b, &x, 4);
    const uint32_t sign = (b >> 16) & 0x8000u, ex = (b >> 23) & 0xFFu, man = b & 0x7FFFFFu;
    if (ex == 0xFF) return (uint16_t) (sign | 0x7C00u | (man ? 0x200u : 0u));
    const int ne = (int) ex - 127 + 15;
    if (ne >= 31) return (uint16_t) (sign | 0x7C00u);
    if (ne <= 0) {
        if (ne < -10) return (uint16_t) sign;
        const int shift = 14 - ne; /* 14..24 */
        const uint32_t full = man | 0x800000u, half = 1u << (shift - 1), rem = full & ((1u << shift) - 1u);
        uint32_t r = full >> shift;
        if (rem > half || (rem == half && (r & 1u))) ++r;
        return (uint16_t) (sign | r);
    }
    uint32_t r = ((uint32_t) ne << 10) | (man >> 13);
    const uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r;
    return (uint16_t) (sign | r);
}

static float bf16_to_f32(uint16_t b) {
    const uint32_t u = (uint32_t) b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ---------------------------------------------------------------- dp4a (p100_compat.h:18-22) */
int fnx_o_dp4a(int a, int b, int c) {
    return c + (int) (signed char) a * (int) (signed char) b + (int) (signed char) (a >> 8) * (int) (signed char) (b >> 8) +
           (int) (signed char) (a >> 16) * (int) (signed char) (b >> 16) + (a >> 24) * (b >> 24);
}

/* ---------------------------------------------------------------- IQ3_S decode (tensor_convert.hpp:295-322) */
void fnx_o_iq3s_dequant(const uint8_t* src, size_t n, float* y) {
    for (size_t b = 0; b < n / 256; ++b) {
        const uint8_t* p = src + b * IQ3S_BLOCK;
        uint16_t dh;
        memcpy(&dh, p, 2);
        const float d = fnx_o_h2f(dh);
        const uint8_t *qs = p + 2, *qh = p + 66, *signs = p + 74, *scales = p + 106;
        float* o = y + b * 256;
        for (int ib = 0; ib < 8; ++ib) { /* sub-block ib: qs[8 ib..], qh[ib], signs[4 ib..], nibble ib & 1 of scales[ib / 2] */
            const int s4 = (scales[ib / 2] >> (4 * (ib & 1))) & 0xF;
            const float db = d * (float) (1 + 2 * s4);
            for (int l = 0; l < 4; ++l) {
                const uint32_t g1 = fnx_o_iq3s_grid[qs[8 * ib + 2 * l] | ((qh[ib] << (8 - 2 * l)) & 256)];
                const uint32_t g2 = fnx_o_iq3s_grid[qs[8 * ib + 2 * l + 1] | ((qh[ib] << (7 - 2 * l)) & 256)];
                const uint8_t sg = signs[4 * ib + l];
                for (int j = 0; j < 4; ++j) {
                    o[32 * ib + 8 * l + j] = db * (float) ((g1 >> (8 * j)) & 255) * ((sg >> j) & 1 ? -1.f : 1.f);
                    o[32 * ib + 8 * l + 4 + j] = db * (float) ((g2 >> (8 * j)) & 255) * ((sg >> (j + 4)) & 1 ? -1.f : 1.f);
                }
            }
        }
    }
}

/* ---------------------------------------------------------------- IQ3_S encoder (this build's own; parity unpinned)
 * Per 32-weight sub-block: try five candidate scales amax / c, c in {15, 13.5, 12, 10.5, 9}; for each, every 4-group
 * takes the nearest codebook entry (squared error on magnitudes, ties to the lower index); keep the scale with the
 * least error. Block scale d = max sub-block scale / 31 (stored as half); sub-block code s = round((scale/d - 1)/2)
 * clamped to 0..15; the groups are then re-coded against the final d (1 + 2 s). Signs are the weights' own. */
static int nearest_grid(const float a[4]) { /* a: magnitudes in codebook units */
    int best = 0;
    float be = INFINITY;
    for (int g = 0; g < 512; ++g) {
        const uint32_t v = fnx_o_iq3s_grid[g];
        float e = 0.f;
        for (int j = 0; j < 4; ++j) {
            const float df = a[j] - (float) ((v >> (8 * j)) & 255);
            e = e + df * df;
        }
        if (e < be) {
            be = e;
            best = g;
        }
    }
    return best;
}
static float group_err(const float a[4], int g) {
    const uint32_t v = fnx_o_iq3s_grid[g];
    float e = 0.f;
    for (int j = 0; j < 4; ++j) {
        const float df = a[j] - (float) ((v >> (8 * j)) & 255);
        e = e + df * df;
    }
    return e;
}
void fnx_o_iq3s_quantize(const float* w, size_t n, uint8_t* dst) {
    static const float cand[5] = {15.0f, 13.5f, 12.0f, 10.5f, 9.0f};
    for (size_t b = 0; b < n / 256; ++b) {
        const float* x = w + b * 256;
        uint8_t* p = dst + b * IQ3S_BLOCK;
        memset(p, 0, IQ3S_BLOCK);
        float sc[8], smax = 0.f;
        for (int ib = 0; ib < 8; ++ib) {
            float amax = 0.f;
            for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[32 * ib + j]));
            sc[ib] = 0.f;
            if (amax > 0.f) {
                float beste = INFINITY;
                for (int c = 0; c < 5; ++c) {
                    const float s = amax / cand[c];
                    float err = 0.f;
                    for (int g = 0; g < 8; ++g) {
                        float a[4];
                        for (int j = 0; j < 4; ++j) a[j] = fabsf(x[32 * ib + 4 * g + j]) / s;
                        err = err + group_err(a, nearest_grid(a));
                    }
                    err = err * s * s;
                    if (err < beste) {
                        beste = err;
                        sc[ib] = s;
                    }
                }
            }
            smax = fmaxf(smax, sc[ib]);
        }
        const uint16_t dh = fnx_o_f2h(smax / 31.0f);
        memcpy(p, &dh, 2);
        const float d = fnx_o_h2f(dh);
        uint8_t *qs = p + 2, *qh = p + 66, *signs = p + 74, *scales = p + 106;
        for (int ib = 0; ib < 8; ++ib) {
            int s4 = 0;
            if (d > 0.f) {
                s4 = (int) roundf((sc[ib] / d - 1.0f) * 0.5f);
                s4 = s4 < 0 ? 0 : s4 > 15 ? 15 : s4;
            }
            scales[ib / 2] |= (uint8_t) (s4 << (4 * (ib & 1)));
            const float db = d * (float) (1 + 2 * s4);
            for (int g = 0; g < 8; ++g) {
                float a[4];
                uint8_t sg = 0;
                for (int j = 0; j < 4; ++j) {
                    const float v = x[32 * ib + 4 * g + j];
                    a[j] = db > 0.f ? fabsf(v) / db : 0.f;
                    if (v < 0.f) sg |= (uint8_t) (1u << j);
                }
                const int gi = nearest_grid(a);
                qs[8 * ib + g] = (uint8_t) (gi & 255);
                qh[ib] |= (uint8_t) ((gi >> 8) << g);
                signs[4 * ib + g / 2] |= (uint8_t) (sg << (4 * (g & 1)));
            }
        }
    }
}

/* ---------------------------------------------------------------- q8_1 (kernels.cu:131-145)
 * one warp per 32 values: amax and the sum by xor-butterfly over the 32 lanes (16, 8, 4, 2, 1) */
static float butterfly_sum(float* v, int n) { /* v[l] += v[l ^ o] for o = n/2 .. 1; every lane ends with the same value */
    float t[64];
    for (int o = n / 2; o; o >>= 1) {
        for (int l = 0; l < n; ++l) t[l] = v[l] + v[l ^ o];
        memcpy(v, t, (size_t) n * sizeof(float));
    }
    return v[0];
}
static void q8_1_block(const float* xi, uint8_t* blk) {
    float amax = 0.f, lanes[32];
    for (int j = 0; j < 32; ++j) {
        amax = fmaxf(amax, fabsf(xi[j]));
        lanes[j] = xi[j];
    }
    const float sum = butterfly_sum(lanes, 32);
    const float d = amax / 127.0f;
    const uint16_t dh = fnx_o_f2h_rn(d), sh = fnx_o_f2h_rn(sum);
    memcpy(blk, &dh, 2);
    memcpy(blk + 2, &sh, 2);
    for (int j = 0; j < 32; ++j) blk[4 + j] = (uint8_t) (int8_t) (amax == 0.0f ? 0 : (int) roundf(xi[j] / d));
}
void fnx_o_quantize_q8_1(const float* x, uint8_t* q, int n, int rows) {
    for (int r = 0; r < rows; ++r)
        for (int b = 0; b < n / 32; ++b) q8_1_block(x + (size_t) r * n + 32 * b, q + ((size_t) r * (n / 32) + b) * Q8_1_BLOCK);
}

/* ---------------------------------------------------------------- the integer dot (iq3s_x.cuh:4-41) */
static int ld32(const uint8_t* p) { /* get_int_b2 / get_int_b4: a little-endian 32-bit load */
    uint32_t v;
    memcpy(&v, p, 4);
    return (int) v;
}
static int vcmpne4_zero(uint32_t a) { /* __vcmpne4(a, 0): 0xff in every byte of a that is not zero */
    uint32_t r = 0;
    for (int k = 0; k < 4; ++k)
        if ((a >> (8 * k)) & 0xFFu) r |= 0xFFu << (8 * k);
    return (int) r;
}
static int vsub4(uint32_t a, uint32_t b) { /* __vsub4: per-byte a - b, wrapping */
    uint32_t r = 0;
    for (int k = 0; k < 4; ++k) r |= (((a >> (8 * k)) - (b >> (8 * k))) & 0xFFu) << (8 * k);
    return (int) r;
}
float fnx_o_vec_dot_iq3s_q8_1(const uint8_t* blk, const uint8_t* q8, int iqs) {
    const uint8_t *bqs = blk + 2, *bqh = blk + 66, *bsigns = blk + 74, *bscales = blk + 106;
    const uint8_t* qs = bqs + 4 * iqs; /* the two ints at iqs, iqs + 1 */
    const int qh = bqh[iqs / 2];
    const uint8_t* sp = bsigns + 4 * (iqs / 2);
    const uint8_t* yb = q8 + (size_t) (iqs / 2) * Q8_1_BLOCK;
    int sumi = 0;
    for (int l0 = 0; l0 < 8; l0 += 2) {
        const uint32_t gx = fnx_o_iq3s_grid[qs[l0] | ((qh << (8 - l0)) & 0x100)];
        const uint32_t gy = fnx_o_iq3s_grid[qs[l0 + 1] | ((qh << (7 - l0)) & 0x100)];
        const uint32_t sb = sp[l0 / 2];
        const int signs0 = vcmpne4_zero(((sb & 0x03u) << 7) | ((sb & 0x0Cu) << 21));
        const int signs1 = vcmpne4_zero(((sb & 0x30u) << 3) | ((sb & 0xC0u) << 17));
        const int grid_l = vsub4(gx ^ (uint32_t) signs0, (uint32_t) signs0);
        const int grid_h = vsub4(gy ^ (uint32_t) signs1, (uint32_t) signs1);
        const int u0 = ld32(yb + 4 + 4 * l0), u1 = ld32(yb + 4 + 4 * (l0 + 1));
        sumi = fnx_o_dp4a(grid_l, u0, sumi);
        sumi = fnx_o_dp4a(grid_h, u1, sumi);
    }
    sumi *= 1 + 2 * ((bscales[iqs / 4] >> ((iqs << 1) & 0x04)) & 0x0F);
    uint16_t dw, dx;
    memcpy(&dw, blk, 2);
    memcpy(&dx, yb, 2);
    const float d = fnx_o_h2f(dw) * fnx_o_h2f(dx);
    return d * (float) sumi;
}

/* lanes per row as moe_g picks them (moe.cuh:664-670): 8 lanes a super-block, doubled up to 32 */
static int lanes_per_row(int ncols) {
    const int lanes = ncols / 256 * 8;
    int G = 8;
    while (G < lanes && G < 32) G *= 2;
    return G;
}
/* one weight row against one q8_1 row: lane gl takes super-blocks gl / 8, + G / 8, ... with its sub-block 2 (gl % 8);
 * the lanes' sums then meet in a butterfly (kernels.cu:209-228) */
static float row_dot(const uint8_t* wr, int ncols, const uint8_t* yq) {
    const int G = lanes_per_row(ncols), bpi = G / 8, bpr = ncols / 256;
    float tmp[32];
    for (int gl = 0; gl < G; ++gl) {
        float t = 0.f;
        for (int kbx = gl / 8; kbx < bpr; kbx += bpi)
            t += fnx_o_vec_dot_iq3s_q8_1(wr + (size_t) kbx * IQ3S_BLOCK, yq + (size_t) kbx * 8 * Q8_1_BLOCK, 2 * (gl % 8));
        tmp[gl] = t;
    }
    return butterfly_sum(tmp, G);
}
void fnx_o_mmvq_iq3s(const uint8_t* wbase, size_t w_stride, const uint8_t* const* ep, int nrows, int ncols,
                     const fnx_o_job* jobs, int njobs, const uint8_t* y, float* out, int out_stride, int threads) {
    const size_t row_bytes = (size_t) (ncols / 256) * IQ3S_BLOCK, y_row = (size_t) (ncols / 32) * Q8_1_BLOCK;
    const long total = (long) njobs * nrows;
    (void) threads;
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
    for (long q = 0; q < total; ++q) {
        const int ji = (int) (q / nrows), r = (int) (q % nrows);
        const fnx_o_job* jb = jobs + ji;
        const uint8_t* we = ep ? ep[jb->w] : wbase + (size_t) jb->w * w_stride;
        for (int j = 0; j < jb->n; ++j)
            out[(size_t) jb->out[j] * out_stride + r] = row_dot(we + (size_t) r * row_bytes, ncols, y + (size_t) jb->y[j] * y_row);
    }
}

void fnx_o_gemv_exact(const uint8_t* w, int nrows, int ncols, const float* x, int T, double* out) {
    const size_t row_bytes = (size_t) (ncols / 256) * IQ3S_BLOCK;
    float* wf = (float*) malloc((size_t) ncols * sizeof(float));
    for (int r = 0; r < nrows; ++r) {
        fnx_o_iq3s_dequant(w + (size_t) r * row_bytes, (size_t) ncols, wf);
        for (int t = 0; t < T; ++t) {
            double s = 0.0;
            for (int i = 0; i < ncols; ++i) s += (double) wf[i] * (double) x[(size_t) t * ncols + i];
            out[(size_t) t * nrows + r] = s;
        }
    }
    free(wf);
}

/* ---------------------------------------------------------------- f32 / bf16 mat-vec in the fixed 64-lane order */
static float dot64(const float* w, const uint16_t* wb, const float* x, int n) {
    float lane[64];
    const int chunks = n / 4;
    for (int l = 0; l < 64; ++l) {
        float a = 0.f;
        for (int c = l; c < chunks; c += 64)
            for (int k = 0; k < 4; ++k) {
                const float wv = w ? w[4 * c + k] : bf16_to_f32(wb[4 * c + k]);
                a = fmaf(wv, x[4 * c + k], a);
            }
        lane[l] = a;
    }
    return butterfly_sum(lane, 64);
}
void fnx_o_gemv_f32(const float* W, const float* x, float* y, int rows, int n, int T) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r)
        for (int t = 0; t < T; ++t) y[(size_t) t * rows + r] = dot64(W + (size_t) r * n, NULL, x + (size_t) t * n, n);
}
void fnx_o_gemv_bf16(const uint16_t* W, const float* x, float* y, int rows, int n, int T) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r)
        for (int t = 0; t < T; ++t) y[(size_t) t * rows + r] = dot64(NULL, W + (size_t) r * n, x + (size_t) t * n, n);
}

void fnx_o_expf(const float* x, size_t n, float* y) {
    for (size_t i = 0; i < n; ++i) y[i] = fnx_expf(x[i]);
}

/* ---------------------------------------------------------------- routing */
void fnx_o_topk_logits(const float* logits, int stride, int T, int nexp, int topk, int* topi, float* topw) {
    unsigned char* taken = (unsigned char*) malloc((size_t) nexp);
    for (int t = 0; t < T; ++t) {
        const float* v = logits + (size_t) t * stride;
        memset(taken, 0, (size_t) nexp);
        float top0 = 0.f, z = 0.f, e[64];
        for (int k = 0; k < topk; ++k) {
            float bv = -INFINITY;
            int bi = nexp;
            for (int i = 0; i < nexp; ++i) /* ascending index with a strict compare: the lower index wins a tie */
                if (!taken[i] && v[i] > bv) {
                    bv = v[i];
                    bi = i;
                }
            const int found = bi < nexp;
            if (!found) /* no logit above -inf is left (masked or NaN): the lowest index not yet picked, at weight 0 */
                for (int i = 0; i < nexp; ++i)
                    if (!taken[i]) {
                        bi = i;
                        break;
                    }
            if (bi < nexp) taken[bi] = 1;
            if (k == 0) top0 = bv;
            e[k] = found ? fnx_expf(bv - top0) : 0.f;
            z += e[k];
            topi[t * topk + k] = bi < nexp ? bi : nexp - 1;
        }
        for (int k = 0; k < topk; ++k) topw[t * topk + k] = z > 0.f ? e[k] / z : 0.f;
    }
    free(taken);
}
void fnx_o_topk_softmax(const float* logits, int stride, int T, int nexp, int topk, int* topi, float* topw) {
    float* p = (float*) malloc((size_t) nexp * sizeof(float));
    for (int t = 0; t < T; ++t) {
        const float* l = logits + (size_t) t * stride;
        float m = -INFINITY, z = 0.f;
        for (int i = 0; i < nexp; ++i) m = fmaxf(m, l[i]);
        for (int i = 0; i < nexp; ++i) {
            p[i] = fnx_expf(l[i] - m);
            z += p[i];
        }
        for (int i = 0; i < nexp; ++i) p[i] = p[i] / z;
        float sel = 0.f;
        for (int k = 0; k < topk; ++k) {
            float bv = p[0];
            int bi = 0;
            for (int i = 1; i < nexp; ++i)
                if (p[i] > bv) {
                    bv = p[i];
                    bi = i;
                }
            topi[t * topk + k] = bi;
            topw[t * topk + k] = bv;
            p[bi] = -1.0f;
        }
        for (int k = 0; k < topk; ++k) sel += topw[t * topk + k];
        for (int k = 0; k < topk; ++k) topw[t * topk + k] /= sel;
    }
    free(p);
}
int fnx_o_jobs(const int* topi, int T, int topk, fnx_o_job* gu, fnx_o_job* dn) {
    int nj = 0;
    for (int t = 0; t < T; ++t)
        for (int k = 0; k < topk; ++k) {
            const int e = topi[t * topk + k], pair = t * topk + k;
            int j = 0;
            while (j < nj && gu[j].w != e) ++j;
            if (j == nj) {
                gu[j].w = e;
                gu[j].n = 0;
                dn[j].w = e;
                dn[j].n = 0;
                ++nj;
            }
            gu[j].y[gu[j].n] = t;
            gu[j].out[gu[j].n] = pair;
            ++gu[j].n;
            dn[j].y[dn[j].n] = pair;
            dn[j].out[dn[j].n] = pair;
            ++dn[j].n;
        }
    return nj;
}

/* ---------------------------------------------------------------- swiglu, combine (kernels.cu:67-68, 400-419) */
/* kernels.cu:67-68, with exp as include/fnx_expf.h fixes it (the reference's __expf is the CUDA toolkit's: its bits cannot be
 * restated; any exp within a few units in the last place is "the reference's" to the tolerance its own tests use) */
static float sigm(float x) { return 1.0f / (1.0f + fnx_expf(-x)); }
static float silu(float x) { return x / (1.0f + fnx_expf(-x)); }
void fnx_o_swiglu_q8_1(const float* g, const float* u, uint8_t* q, int n, int rows) {
    float h[32];
    for (int r = 0; r < rows; ++r)
        for (int b = 0; b < n / 32; ++b) {
            for (int j = 0; j < 32; ++j) {
                const size_t i = (size_t) r * n + 32 * b + j;
                h[j] = silu(g[i]) * u[i];
            }
            q8_1_block(h, q + ((size_t) r * (n / 32) + b) * Q8_1_BLOCK);
        }
}
void fnx_o_swiglu_stacked_q8_1(const float* gu, uint8_t* hq, int ffs, int rows) {
    float h[32];
    for (int r = 0; r < rows; ++r) {
        const float* g = gu + (size_t) r * 2 * ffs;
        for (int b = 0; b < ffs / 32; ++b) {
            for (int j = 0; j < 32; ++j) h[j] = silu(g[32 * b + j]) * g[ffs + 32 * b + j];
            q8_1_block(h, hq + ((size_t) r * (ffs / 32) + b) * Q8_1_BLOCK);
        }
    }
}
void fnx_o_moe_combine(const float* part, const float* topw, const float* sh, const float* sh_logit, int sh_logit_stride,
                       float* out, int T, int n, int topk) {
    for (int t = 0; t < T; ++t) {
        const float gate = sigm(sh_logit[(size_t) t * sh_logit_stride]);
        for (int i = 0; i < n; ++i) {
            float s = 0.f;
            for (int k = 0; k < topk; ++k) s = fmaf(topw[t * topk + k], part[((size_t) t * topk + k) * n + i], s);
            out[(size_t) t * n + i] = s + gate * sh[(size_t) t * n + i];
        }
    }
}

/* ---------------------------------------------------------------- argmax (kernels.cu:1045-1083) */
static uint32_t fkey(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
static float fkey_inv(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
unsigned fnx_o_argmax(const float* logits, int rows, int T, int v0, float* best_v, int* best_i) {
    unsigned err = 0;
    for (int t = 0; t < T; ++t) {
        const float* r = logits + (size_t) t * rows;
        uint64_t best = 0;
        for (int i = 0; i < rows; ++i) {
            if (!isfinite(r[i])) err |= 16u;
            const uint64_t k = (uint64_t) fkey(r[i]) << 32 | (uint32_t) ~(uint32_t) i;
            if (k > best) best = k;
        }
        best_v[t] = fkey_inv((uint32_t) (best >> 32));
        best_i[t] = (int) ~(uint32_t) best + v0;
    }
    return err;
}

/* ---------------------------------------------------------------- other expert types at the boundary (kernels.cu:2454-2471)
 * Decoders as tensor_convert.hpp:152-265 dequantises the types (the reference's own host code; pinned against it through
 * oracle/_ref). The dot with q8_1 rows is ggml's vec_dot_<type>_q8_1 (ggml-cuda/vecdotq.cuh of llama.cpp @
 * 3cf03257f219afbe7334045ff7c6a06ac68c627d, third_party/ggml/VERSION.txt - a fetched dependency, not in the tree):
 * restated from its published form per 32 values; its per-thread split of a block and its warp order cannot be pinned, so
 * the sums here run in this build's order (lane l of 64 takes sub-blocks l, l + 64, ...; then the xor butterfly). */
#define T_Q4_0 2u
#define T_Q5_1 7u
#define T_Q8_0 8u
#define T_Q4_K 12u
#define T_Q5_K 13u
#define T_IQ4_NL 20u
#define T_IQ4_XS 23u
static const int8_t KV_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
int fnx_o_type_block(uint32_t type, int* values, int* bytes) {
    switch (type) {
        case T_Q4_0: *values = 32; *bytes = 18; return 0;
        case T_Q5_1: *values = 32; *bytes = 24; return 0;
        case T_Q8_0: *values = 32; *bytes = 34; return 0;
        case T_IQ4_NL: *values = 32; *bytes = 18; return 0;
        case T_Q4_K: *values = 256; *bytes = 144; return 0;
        case T_IQ4_XS: *values = 256; *bytes = 136; return 0;
        case T_Q5_K: *values = 256; *bytes = 176; return 0;
    }
    return 1;
}
/* get_scale_min_k4 (ggml; tensor_convert.hpp scale_min_k4): sub-block j's 6-bit scale and min out of the 12 bytes */
static void k4_scale_min(int j, const uint8_t* q, int* sc, int* m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
        *m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}
/* sub-block kb (32 values) of a row: its integers q[32] with value = scale * q - offset */
typedef struct {
    int q[32];
    float d, dmin; /* the block's scales as floats (dmin: K-quants only) */
    int sc, m;     /* K-quants: the sub-block's 6-bit scale and min */
} sub_t;
static void sub_decode(uint32_t type, const uint8_t* row, int kb, sub_t* o) {
    uint16_t h;
    o->dmin = 0.f;
    o->sc = 1;
    o->m = 0;
    if (type == T_Q8_0) {
        const uint8_t* p = row + (size_t) kb * 34;
        memcpy(&h, p, 2);
        o->d = fnx_o_h2f(h);
        for (int j = 0; j < 32; ++j) o->q[j] = (int8_t) p[2 + j];
    } else if (type == T_Q5_1) { /* ggml block_q5_1 {half d; half m; u32 qh; u8 qs[16]}: value = d * q + m, q = nibble | bit << 4 (not
                                    in tensor_convert.hpp: the layout is ggml's published one) */
        const uint8_t* p = row + (size_t) kb * 24;
        uint32_t qh;
        memcpy(&h, p, 2);
        o->d = fnx_o_h2f(h);
        memcpy(&h, p + 2, 2);
        o->dmin = fnx_o_h2f(h); /* the block's m (added, not subtracted) */
        memcpy(&qh, p + 4, 4);
        for (int j = 0; j < 16; ++j) {
            o->q[j] = (p[8 + j] & 0xF) | (int) (((qh >> j) & 1u) << 4);
            o->q[j + 16] = (p[8 + j] >> 4) | (int) (((qh >> (j + 16)) & 1u) << 4);
        }
    } else if (type == T_Q4_0 || type == T_IQ4_NL) {
        const uint8_t* p = row + (size_t) kb * 18;
        memcpy(&h, p, 2);
        o->d = fnx_o_h2f(h);
        for (int j = 0; j < 16; ++j) {
            const int lo = p[2 + j] & 0xF, hi = p[2 + j] >> 4;
            o->q[j] = type == T_Q4_0 ? lo : KV_IQ4NL[lo];      /* Q4_0: the - 8 is applied through the q8_1 sum */
            o->q[j + 16] = type == T_Q4_0 ? hi : KV_IQ4NL[hi];
        }
    } else if (type == T_IQ4_XS) { /* {half d; u16 scales_h; u8 scales_l[4]; u8 qs[128]}: sub-block ib has a 6-bit scale - 32 */
        const int ib = kb & 7;
        const uint8_t* p = row + (size_t) (kb >> 3) * 136;
        uint16_t sh;
        memcpy(&h, p, 2);
        o->d = fnx_o_h2f(h);
        memcpy(&sh, p + 2, 2);
        o->sc = (((p[4 + ib / 2] >> (4 * (ib % 2))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4)) - 32;
        const uint8_t* qs = p + 8 + 16 * ib;
        for (int j = 0; j < 16; ++j) {
            o->q[j] = KV_IQ4NL[qs[j] & 0xF];
            o->q[j + 16] = KV_IQ4NL[qs[j] >> 4];
        }
    } else { /* Q4_K, Q5_K: super-block kb / 8, sub-block kb % 8 */
        const int sb = kb & 7, five = type == T_Q5_K;
        const uint8_t* p = row + (size_t) (kb >> 3) * (five ? 176 : 144);
        memcpy(&h, p, 2);
        o->d = fnx_o_h2f(h);
        memcpy(&h, p + 2, 2);
        o->dmin = fnx_o_h2f(h);
        k4_scale_min(sb, p + 4, &o->sc, &o->m);
        const uint8_t *qh = p + 16, *ql = p + (five ? 48 : 16) + 32 * (sb >> 1);
        for (int l = 0; l < 32; ++l) {
            int v = (sb & 1) ? ql[l] >> 4 : ql[l] & 0xF;
            if (five && ((qh[l] >> sb) & 1)) v += 16;
            o->q[l] = v;
        }
    }
}
void fnx_o_dequant(uint32_t type, const uint8_t* src, size_t n, float* y) {
    for (size_t kb = 0; kb < n / 32; ++kb) {
        sub_t s;
        sub_decode(type, src, (int) kb, &s);
        for (int j = 0; j < 32; ++j) {
            if (type == T_Q4_0) y[kb * 32 + j] = s.d * (float) (s.q[j] - 8);
            else if (type == T_Q5_1) y[kb * 32 + j] = s.d * (float) s.q[j] + s.dmin;
            else if (type == T_IQ4_XS) y[kb * 32 + j] = (s.d * (float) s.sc) * (float) s.q[j];
            else if (type == T_Q4_K || type == T_Q5_K) y[kb * 32 + j] = (s.d * (float) s.sc) * (float) s.q[j] - s.dmin * (float) s.m;
            else y[kb * 32 + j] = s.d * (float) s.q[j];
        }
    }
}
/* one sub-block's term of the dot with a q8_1 block {half d; half sum; int8 qs[32]} */
float fnx_o_vec_dot_type(uint32_t type, const uint8_t* row, int kb, const uint8_t* q8) {
    sub_t s;
    uint16_t h;
    sub_decode(type, row, kb, &s);
    memcpy(&h, q8, 2);
    const float dx = fnx_o_h2f(h);
    memcpy(&h, q8 + 2, 2);
    const float sx = fnx_o_h2f(h);
    int dot = 0, qsum = 0;
    for (int j = 0; j < 32; ++j) {
        const int x = (int8_t) q8[4 + j];
        dot += s.q[j] * x;
        qsum += x;
    }
    if (type == T_Q4_0) return s.d * ((float) dot * dx - 8.0f * sx);                      /* vec_dot_q4_0_q8_1_impl */
    if (type == T_Q5_1) return (float) dot * (s.d * dx) + s.dmin * sx;                    /* vec_dot_q5_1_q8_1_impl */
    if (type == T_IQ4_XS) return (s.d * dx) * (float) (dot * s.sc);                       /* vec_dot_iq4_xs_q8_1 */
    if (type == T_Q4_K || type == T_Q5_K)                                               /* vec_dot_q4_K_q8_1_impl_vmmq */
        return s.d * (dx * (float) (dot * s.sc)) - s.dmin * (dx * (float) (qsum * s.m));
    return (s.d * dx) * (float) dot;                                                      /* vec_dot_q8_0_q8_1_impl, vec_dot_iq4_nl_q8_1 */
}
void fnx_o_mmvq_type(uint32_t type, const uint8_t* w, size_t w_stride, int nrows, int ncols, const fnx_o_job* jobs, int njobs, const uint8_t* y,
                     float* out, int out_stride, int threads) {
    int values, bytes;
    if (fnx_o_type_block(type, &values, &bytes)) return;
    const int sbr = ncols / 32;
    const size_t row_bytes = (size_t) (ncols / values) * bytes;
    (void) threads;
#pragma omp parallel for collapse(2) num_threads(threads > 0 ? threads : 1)
    for (int ji = 0; ji < njobs; ++ji)
        for (int r = 0; r < nrows; ++r) {
            const fnx_o_job* jb = jobs + ji;
            const uint8_t* row = w + (size_t) jb->w * w_stride + (size_t) r * row_bytes;
            for (int t = 0; t < jb->n; ++t) {
                float lanes[64];
                for (int l = 0; l < 64; ++l) {
                    float acc = 0.f;
                    for (int kb = l; kb < sbr; kb += 64) acc += fnx_o_vec_dot_type(type, row, kb, y + ((size_t) jb->y[t] * sbr + kb) * Q8_1_BLOCK);
                    lanes[l] = acc;
                }
                out[(size_t) jb->out[t] * out_stride + r] = butterfly_sum(lanes, 64);
            }
        }
}

/* ---------------------------------------------------------------- the sampler's candidates (topk.cuh, kernels.hpp:434-447) */
static int cmp_desc_u64(const void* a, const void* b) {
    const uint64_t x = *(const uint64_t*) a, y = *(const uint64_t*) b;
    return x < y ? 1 : x > y ? -1 : 0;
}
/* kernels.cu:1771-1781 k_penalize_row; the same arithmetic as topk.cuh:40-46 */
static float penalized(float l, int cnt, float repeat, float freq, float present) {
    l = l <= 0.f ? l * repeat : l / repeat;
    return l - (float) cnt * freq - present;
}
void fnx_o_penalize_row(float* row, int n, const int* pen, const float* par) {
    const int k = pen[0];
    for (int i = 0; i < k; ++i) {
        const int j = pen[1 + i], cnt = pen[1 + k + i];
        if (j < 0 || j >= n || cnt <= 0) continue;
        row[j] = penalized(row[j], cnt, par[0], par[1], par[2]);
    }
}
/* topk.cuh:18-156 k_topk_rows: the finite check on the head's logits, the row's logit_bias, then its penalties (in
 * place), then the 64 greatest by (order-preserving key of the logit's bits descending, id ascending). The reference's
 * radix select and its wide-tie pass are a way to that set; here every (key, id) pair is sorted. */
unsigned fnx_o_top_tokens(float* logits, int n, int T, int v0, const int* pen_tok, const int* pen_cnt, const int* pen_n, int pen_stride,
                          const float* pen_par, const int* bias_tok, const float* bias_val, const int* bias_off, const int* bias_n, float* out_v,
                          int* out_i) {
    unsigned err = 0;
    uint64_t* keys = (uint64_t*) malloc((size_t) n * sizeof(uint64_t));
    for (int t = 0; t < T; ++t) {
        float* L = logits + (size_t) t * n;
        for (int j = 0; j < n; ++j)
            if (!isfinite(L[j])) err |= 16u;
        for (int i = 0; bias_n && i < bias_n[t]; ++i) {
            const int at = bias_off[t] + i, tok = bias_tok[at] - v0;
            if (tok >= 0 && tok < n) L[tok] += bias_val[at];
        }
        for (int i = 0; pen_n && i < pen_n[t]; ++i) {
            const int tok = pen_tok[t * pen_stride + i] - v0, cnt = pen_cnt[t * pen_stride + i];
            if (tok < 0 || tok >= n || cnt <= 0) continue;
            L[tok] = penalized(L[tok], cnt, pen_par[t * 3], pen_par[t * 3 + 1], pen_par[t * 3 + 2]);
        }
        for (int j = 0; j < n; ++j) keys[j] = (uint64_t) fkey(L[j]) << 32 | (uint32_t) (0xffffffffu - (uint32_t) j);
        qsort(keys, (size_t) n, sizeof(uint64_t), cmp_desc_u64);
        for (int r = 0; r < 64; ++r) {
            const int j = (int) (0xffffffffu - (uint32_t) keys[r]);
            out_i[t * 64 + r] = v0 + j;
            out_v[t * 64 + r] = L[j];
        }
    }
    free(keys);
    return err;
}

/* ---------------------------------------------------------------- the sampler's draw (session.cpp:34-84, 574-613) */
static double dist_prob(const int* ids, const double* p, int n, int id) { /* session.cpp:34-39 */
    for (int i = 0; i < n; ++i)
        if (ids[i] == id) return p[i];
    return 0.0;
}
/* session.cpp:41-75 make_dist */
int fnx_o_make_dist(const float* cv, const int* ci, int ncand, float temperature, float top_p, float min_p, int top_k, int* ids, double* p) {
    const int k = (top_k <= 0 || top_k > ncand) ? ncand : top_k;
    int keep = k;
    const double mx = cv[0];
    if (top_p < 1.f) {
        double sum = 0.0, cum = 0.0;
        for (int i = 0; i < k; ++i) sum += exp((double) cv[i] - mx);
        for (int i = 0; i < k; ++i) {
            cum += exp((double) cv[i] - mx) / sum;
            if (cum >= (double) top_p) {
                keep = i + 1;
                break;
            }
        }
    }
    if (min_p > 0.f) {
        const float thresh = cv[0] + logf(min_p);
        for (int i = 1; i < keep; ++i)
            if (cv[i] < thresh) {
                keep = i;
                break;
            }
    }
    const double inv_t = 1.0 / temperature, smx = cv[0] * inv_t;
    double sum = 0.0;
    for (int i = 0; i < keep; ++i) {
        ids[i] = ci[i];
        p[i] = exp(cv[i] * inv_t - smx);
        sum += p[i];
    }
    for (int i = 0; i < keep; ++i) p[i] /= sum;
    return keep;
}
/* session.cpp:77-84 draw */
int fnx_o_draw(const int* ids, const double* p, int n, double u) {
    double cum = 0.0;
    for (int i = 0; i < n; ++i) {
        cum += p[i];
        if (u < cum) return ids[i];
    }
    return ids[n - 1];
}
/* session.cpp:574-613: speculative sampling over a window of T rows; uniforms taken from u in the order of use */
int fnx_o_accept_sampled(const float* cv, const int* ci, int ncand, int T, const int* rows, float temperature, float top_p, float min_p, int top_k,
                         const int* q_ids, const double* q_p, const int* q_n, int q_stride, const double* u, int* o, int* used_u) {
    int ids[64], n, at = 0;
    double p[64], p0[64];
    for (n = 0; n < T; ++n) {
        int m = fnx_o_make_dist(cv + (size_t) n * ncand, ci + (size_t) n * ncand, ncand, temperature, top_p, min_p, top_k, ids, p);
        if (n + 1 < T) {
            const int dr = rows[n + 1], qn = q_n ? q_n[n] : 0, fixed = qn == 0;
            const int* qi = q_ids ? q_ids + (size_t) n * q_stride : NULL;
            const double* qp = q_p ? q_p + (size_t) n * q_stride : NULL;
            if (u[at++] * (fixed ? 1.0 : dist_prob(qi, qp, qn, dr)) < dist_prob(ids, p, m, dr)) {
                o[n] = dr;
                continue;
            }
            double rest = 0.0;
            memcpy(p0, p, sizeof(double) * (size_t) m);
            for (int i = 0; i < m; ++i) {
                const double q = fixed ? (ids[i] == dr ? 1.0 : 0.0) : dist_prob(qi, qp, qn, ids[i]);
                p[i] = p[i] - q > 0.0 ? p[i] - q : 0.0;
                rest += p[i];
            }
            if (rest > 1e-12)
                for (int i = 0; i < m; ++i) p[i] /= rest;
            else
                memcpy(p, p0, sizeof(double) * (size_t) m);
        }
        o[n] = fnx_o_draw(ids, p, m, u[at++]);
        ++n;
        break;
    }
    if (used_u) *used_u = at;
    return n;
}

/* ---------------------------------------------------------------- prompt lookup, acceptance */
#define LOOKUP_MIN 3       /* session.cpp:18 */
#define IMAGE_TOK (1 << 30) /* engine.hpp:84 */
int fnx_o_lookup_drafts(const int* ctx, int n_ctx, int key_n, int lk, int d1, int* out, int* match) {
    int nr = 0;
    if (match) *match = -1;
    if (lk == 0 || n_ctx <= key_n) return 0;
    const long n0 = (long) n_ctx - key_n;
    for (long s = n0; s-- > 0;)
        if (memcmp(ctx + s, ctx + n0, (size_t) key_n * sizeof(int)) == 0) {
            if (s + key_n < n_ctx && (d1 < 0 || ctx[s + key_n] == d1)) {
                int m = key_n;
                while (m < lk && (long) (m - key_n) < s && ctx[s - 1 - (m - key_n)] == ctx[n0 - 1 - (m - key_n)]) ++m;
                int k = m > LOOKUP_MIN ? m : LOOKUP_MIN;
                if (k > lk) k = lk;
                long end = s + key_n + k;
                if (end > n_ctx) end = n_ctx;
                for (long i = s + key_n; i < end; ++i) out[nr++] = ctx[i];
                if (match) *match = (int) s;
            }
            break;
        }
    for (int i = 0; i < nr; ++i)
        if (out[i] >= IMAGE_TOK) {
            nr = i;
            break;
        }
    return nr;
}
int fnx_o_lookup_fixed(const int* ctx, int n_ctx, int key_n, int lk, int d1, int* out) {
    int nr = 0;
    if (lk == 0 || n_ctx <= key_n) return 0;
    const long n0 = (long) n_ctx - key_n;
    for (long st = n0; st-- > 0;)
        if (memcmp(ctx + st, ctx + n0, (size_t) key_n * sizeof(int)) == 0) {
            if (st + key_n < n_ctx && ctx[st + key_n] == d1) {
                long end = st + key_n + lk;
                if (end > n_ctx) end = n_ctx;
                for (long i = st + key_n; i < end; ++i) out[nr++] = ctx[i];
            }
            break;
        }
    return nr;
}
int fnx_o_accept_greedy(const int* rows, const int* o, int R) {
    int n = 1;
    while (n < R && rows[n] == o[n - 1]) ++n;
    return n;
}

/* ---------------------------------------------------------------- prefill jobs (prefill.cu:320-377)
 * jobs are arrays of ints {w, n, y[pf_job], out[pf_job]} */
int fnx_o_pf_jobs(const int* topi, int C, int topk, int nexp, int pf_job, int* jobs_gu, int* jobs_dn, int* cnt) {
    const int P = C * topk, js = 2 + 2 * pf_job;
    int* jbase = (int*) malloc((size_t) nexp * sizeof(int));
    int* fill = (int*) calloc((size_t) nexp, sizeof(int));
    memset(cnt, 0, (size_t) nexp * sizeof(int));
    for (int p = 0; p < P; ++p) ++cnt[topi[p]];
    int nj = 0;
    for (int e = 0; e < nexp; ++e) {
        jbase[e] = nj;
        nj += (cnt[e] + pf_job - 1) / pf_job;
    }
    for (int p = 0; p < P; ++p) { /* ascending pair index: a pair always lands in the same job and slot */
        const int e = topi[p], s = fill[e]++, j = jbase[e] + s / pf_job, k = s % pf_job;
        int *g = jobs_gu + (size_t) j * js, *d = jobs_dn + (size_t) j * js;
        g[2 + k] = p / topk;
        g[2 + pf_job + k] = p;
        d[2 + k] = p;
        d[2 + pf_job + k] = p;
        if (k == 0) {
            const int left = cnt[e] - (s / pf_job) * pf_job;
            g[0] = d[0] = e;
            g[1] = d[1] = left < pf_job ? left : pf_job;
        }
    }
    free(jbase);
    free(fill);
    return nj;
}

/* ---------------------------------------------------------------- one MoE verify layer */
void fnx_o_moe_verify_layer(const fnx_o_moe_layer* L, const float* x, int T, float* out, float* logits_out, int* topi_out,
                            float* topw_out, int* njobs_out, int threads) {
    const int n = L->n, ff = L->ff, nexp = L->nexp, topk = L->topk, P = T * topk;
    const size_t gu_stride = (size_t) 2 * ff * (n / 256) * IQ3S_BLOCK, dn_stride = (size_t) n * (ff / 256) * IQ3S_BLOCK;
    if (threads <= 0) threads = 1;
#ifdef _OPENMP
    const int prev = omp_get_max_threads();
    omp_set_num_threads(threads);
#endif
    uint8_t* xq = (uint8_t*) malloc((size_t) T * (n / 32) * Q8_1_BLOCK);
    float* logits = (float*) malloc((size_t) T * (nexp + 1) * sizeof(float));
    float* lt = (float*) malloc((size_t) T * (nexp + 1) * sizeof(float));
    int* topi = (int*) malloc((size_t) P * sizeof(int));
    float* topw = (float*) malloc((size_t) P * sizeof(float));
    fnx_o_job* jgu = (fnx_o_job*) calloc((size_t) P + 1, sizeof(fnx_o_job));
    fnx_o_job* jdn = (fnx_o_job*) calloc((size_t) P + 1, sizeof(fnx_o_job));
    float* gu = (float*) malloc((size_t) (P + T) * 2 * ff * sizeof(float));
    uint8_t* hq = (uint8_t*) malloc((size_t) (P + T) * (ff / 32) * Q8_1_BLOCK);
    float* part = (float*) malloc((size_t) (P + T) * n * sizeof(float));

    fnx_o_quantize_q8_1(x, xq, n, T);
    fnx_o_gemv_f32(L->router, x, lt, nexp + 1, n, T); /* lt[t][row] with stride nexp + 1 */
    memcpy(logits, lt, (size_t) T * (nexp + 1) * sizeof(float));
    fnx_o_topk_logits(logits, nexp + 1, T, nexp, topk, topi, topw);
    const int nj = fnx_o_jobs(topi, T, topk, jgu, jdn);
    /* routed experts */
    fnx_o_mmvq_iq3s(L->gu, gu_stride, NULL, 2 * ff, n, jgu, nj, xq, gu, 2 * ff, threads);
    /* shared expert: one job of all T rows, outputs at rows P + t (kernels.hpp:277-282) */
    fnx_o_job sh;
    sh.w = 0;
    sh.n = T;
    for (int t = 0; t < T; ++t) {
        sh.y[t] = t;
        sh.out[t] = P + t;
    }
    if (L->sh_gu_q) fnx_o_q8s_gemv(L->sh_gu_q, L->sh_gu_d, 2 * ff, n, xq, gu + (size_t) P * 2 * ff, 2 * ff, T); /* engine.cu:1601 */
    else fnx_o_mmvq_iq3s(L->sh_gu, 0, NULL, 2 * ff, n, &sh, 1, xq, gu, 2 * ff, threads);
    fnx_o_swiglu_stacked_q8_1(gu, hq, ff, P + T);
    fnx_o_mmvq_iq3s(L->down, dn_stride, NULL, n, ff, jdn, nj, hq, part, n, threads);
    for (int t = 0; t < T; ++t) sh.y[t] = P + t;
    if (L->sh_gu_q) /* engine.cu:1603: the rows P + t of hq and of part */
        fnx_o_q8s_gemv(L->sh_down_q, L->sh_down_d, n, ff, hq + (size_t) P * (ff / 32) * Q8_1_BLOCK, part + (size_t) P * n, n, T);
    else fnx_o_mmvq_iq3s(L->sh_down, 0, NULL, n, ff, &sh, 1, hq, part, n, threads);
    fnx_o_moe_combine(part, topw, part + (size_t) P * n, logits + nexp, nexp + 1, out, T, n, topk);

    if (logits_out) memcpy(logits_out, logits, (size_t) T * (nexp + 1) * sizeof(float));
    if (topi_out) memcpy(topi_out, topi, (size_t) P * sizeof(int));
    if (topw_out) memcpy(topw_out, topw, (size_t) P * sizeof(float));
    if (njobs_out) *njobs_out = nj;
    free(xq);
    free(logits);
    free(lt);
    free(topi);
    free(topw);
    free(jgu);
    free(jdn);
    free(gu);
    free(hq);
    free(part);
#ifdef _OPENMP
    omp_set_num_threads(prev);
#endif
}

/* ---------------------------------------------------------------- prompt path: f16 tiles (moe_mma_iq.cuh:108-152) */
void fnx_o_iq3s_dequant_f16(const uint8_t* src, size_t n, uint16_t* y) {
    float f[256];
    for (size_t b = 0; b < n / 256; ++b) {
        fnx_o_iq3s_dequant(src + b * IQ3S_BLOCK, 256, f); /* d * (1 + 2 s) * grid * sign: exact in f32 */
        for (int i = 0; i < 256; ++i) y[b * 256 + i] = fnx_o_f2h_rn(f[i]);
    }
}
void fnx_o_f32_f16(const float* x, size_t n, uint16_t* y) {
    for (size_t i = 0; i < n; ++i) y[i] = fnx_o_f2h_rn(x[i]);
}
void fnx_o_moe_mma(const uint8_t* wbase, size_t w_stride, int nrows, int ncols, const int* jobs, int njobs, int pf_job,
                   const uint16_t* x, int ldx, float* out, int threads) {
    const int js = 2 + 2 * pf_job;
    const size_t row_bytes = (size_t) (ncols / 256) * IQ3S_BLOCK;
    if (threads <= 0) threads = 1;
#pragma omp parallel num_threads(threads)
    {
        uint16_t* wh = (uint16_t*) malloc((size_t) ncols * sizeof(uint16_t));
        float* wf = (float*) malloc((size_t) ncols * sizeof(float));
        float* xf = (float*) malloc((size_t) pf_job * ncols * sizeof(float));
        for (int ji = 0; ji < njobs; ++ji) {
            const int* jb = jobs + (size_t) ji * js;
            const uint8_t* we = wbase + (size_t) jb[0] * w_stride;
            const int n = jb[1];
            for (int j = 0; j < n; ++j)
                for (int k = 0; k < ncols; ++k) xf[(size_t) j * ncols + k] = fnx_o_h2f(x[(size_t) jb[2 + j] * ldx + k]);
#pragma omp for schedule(static)
            for (int row = 0; row < nrows; ++row) {
                fnx_o_iq3s_dequant_f16(we + (size_t) row * row_bytes, (size_t) ncols, wh);
                for (int k = 0; k < ncols; ++k) wf[k] = fnx_o_h2f(wh[k]);
                for (int j = 0; j < n; ++j) {
                    double s = 0.0;
                    const float* xr = xf + (size_t) j * ncols;
                    for (int k = 0; k < ncols; ++k) s += (double) wf[k] * (double) xr[k];
                    out[(size_t) jb[2 + pf_job + j] * nrows + row] = (float) s;
                }
            }
        }
        free(wh);
        free(wf);
        free(xf);
    }
}
void fnx_o_swiglu_h16(const float* gu, int ffs, int P, uint16_t* h) {
    for (int r = 0; r < P; ++r)
        for (int i = 0; i < ffs; ++i) h[(size_t) r * ffs + i] = fnx_o_f2h_rn(silu(gu[(size_t) r * 2 * ffs + i]) * gu[(size_t) r * 2 * ffs + ffs + i]);
}
void fnx_o_moe_prefill_layer(const fnx_o_moe_layer* L, const float* x, int C, int pf_job, float* out, float* logits_out, int* topi_out,
                             float* topw_out, int* njobs_out, int threads) {
    const int n = L->n, ff = L->ff, nexp = L->nexp, topk = L->topk, P = C * topk, js = 2 + 2 * pf_job;
    const size_t gu_stride = (size_t) 2 * ff * (n / 256) * IQ3S_BLOCK, dn_stride = (size_t) n * (ff / 256) * IQ3S_BLOCK;
    const int maxjobs = P / pf_job + nexp + 1, shjobs = (C + pf_job - 1) / pf_job;
    float* logits = (float*) malloc((size_t) C * (nexp + 1) * sizeof(float));
    int* topi = (int*) malloc((size_t) P * sizeof(int));
    float* topw = (float*) malloc((size_t) P * sizeof(float));
    int* cnt = (int*) malloc((size_t) nexp * sizeof(int));
    int* jgu = (int*) calloc((size_t) maxjobs * js, sizeof(int));
    int* jdn = (int*) calloc((size_t) maxjobs * js, sizeof(int));
    int* jsh = (int*) calloc((size_t) shjobs * js, sizeof(int));
    uint16_t* xh = (uint16_t*) malloc((size_t) C * n * sizeof(uint16_t));
    float* gu = (float*) malloc((size_t) (P + C) * 2 * ff * sizeof(float));
    uint16_t* h16 = (uint16_t*) malloc((size_t) (P + C) * ff * sizeof(uint16_t));
    float* part = (float*) malloc((size_t) (P + C) * n * sizeof(float));
    if (threads <= 0) threads = 1;
#ifdef _OPENMP
    const int prev = omp_get_max_threads();
    omp_set_num_threads(threads);
#endif
    for (int t0 = 0; t0 < C; t0 += 16) { /* the same sums whatever the grouping: each (row, token) sum stands alone */
        const int T = C - t0 < 16 ? C - t0 : 16;
        fnx_o_gemv_f32(L->router, x + (size_t) t0 * n, logits + (size_t) t0 * (nexp + 1), nexp + 1, n, T);
    }
    fnx_o_topk_logits(logits, nexp + 1, C, nexp, topk, topi, topw);
    const int nj = fnx_o_pf_jobs(topi, C, topk, nexp, pf_job, jgu, jdn, cnt);
    fnx_o_f32_f16(x, (size_t) C * n, xh);
    fnx_o_moe_mma(L->gu, gu_stride, 2 * ff, n, jgu, nj, pf_job, xh, n, gu, threads);
    for (int j = 0; j < shjobs; ++j) { /* the shared expert: every row, outputs at rows P + t */
        int* jb = jsh + (size_t) j * js;
        jb[0] = 0;
        jb[1] = C - j * pf_job < pf_job ? C - j * pf_job : pf_job;
        for (int i = 0; i < jb[1]; ++i) {
            jb[2 + i] = j * pf_job + i;
            jb[2 + pf_job + i] = P + j * pf_job + i;
        }
    }
    fnx_o_moe_mma(L->sh_gu, 0, 2 * ff, n, jsh, shjobs, pf_job, xh, n, gu, threads);
    fnx_o_swiglu_h16(gu, ff, P + C, h16);
    fnx_o_moe_mma(L->down, dn_stride, n, ff, jdn, nj, pf_job, h16, ff, part, threads);
    for (int j = 0; j < shjobs; ++j) {
        int* jb = jsh + (size_t) j * js;
        for (int i = 0; i < jb[1]; ++i) jb[2 + i] = P + j * pf_job + i;
    }
    fnx_o_moe_mma(L->sh_down, 0, n, ff, jsh, shjobs, pf_job, h16, ff, part, threads);
    fnx_o_moe_combine(part, topw, part + (size_t) P * n, logits + nexp, nexp + 1, out, C, n, topk);
    if (logits_out) memcpy(logits_out, logits, (size_t) C * (nexp + 1) * sizeof(float));
    if (topi_out) memcpy(topi_out, topi, (size_t) P * sizeof(int));
    if (topw_out) memcpy(topw_out, topw, (size_t) P * sizeof(float));
    if (njobs_out) *njobs_out = nj;
    free(logits); free(topi); free(topw); free(cnt); free(jgu); free(jdn); free(jsh); free(xh); free(gu); free(h16); free(part);
#ifdef _OPENMP
    omp_set_num_threads(prev);
#endif
}

/* ---------------------------------------------------------------- around the MoE half */
void fnx_o_rms_norm_rows(const float* x, const float* w, float* y, int rows, int n, float eps) {
    for (int r = 0; r < rows; ++r) {
        double s = 0.0;
        for (int i = 0; i < n; ++i) s += (double) x[(size_t) r * n + i] * x[(size_t) r * n + i];
        const float sc = (float) (1.0 / sqrt(s / n + (double) eps));
        for (int i = 0; i < n; ++i) y[(size_t) r * n + i] = x[(size_t) r * n + i] * sc * w[i];
    }
}
void fnx_o_quantize_q8_0_split(const float* w, int rows, int cols, int8_t* q, uint16_t* d) {
    const int nb = cols / 32;
    for (int r = 0; r < rows; ++r)
        for (int b = 0; b < nb; ++b) {
            const float* x = w + (size_t) r * cols + 32 * b;
            float amax = 0.f;
            for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[j]));
            const float dd = amax / 127.0f, id = dd != 0.f ? 1.0f / dd : 0.f;
            d[(size_t) r * nb + b] = fnx_o_f2h_rn(dd);
            for (int j = 0; j < 32; ++j) q[(size_t) r * cols + 32 * b + j] = (int8_t) roundf(x[j] * id);
        }
}
void fnx_o_q8s_gemv(const int8_t* q, const uint16_t* d, int rows, int cols, const uint8_t* yq, float* out, int out_stride, int T) {
    const int nb = cols / 32, qb = nb / 4 > 0 ? nb / 4 : nb; /* blocks per quarter (fewer than 4 blocks: one part) */
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r)
        for (int t = 0; t < T; ++t) {
            float part[4] = {0.f, 0.f, 0.f, 0.f};
            for (int b = 0; b < nb; ++b) { /* each quarter: ascending blocks, one fmaf each; the order is part of the definition */
                const uint8_t* blk = yq + ((size_t) t * nb + b) * Q8_1_BLOCK;
                uint16_t dxh;
                memcpy(&dxh, blk, 2);
                const int8_t* xs = (const int8_t*) blk + 4;
                int s = 0;
                for (int j = 0; j < 32; ++j) s += (int) q[(size_t) r * cols + 32 * b + j] * (int) xs[j];
                part[b / qb] = fmaf(fnx_o_h2f(d[(size_t) r * nb + b]) * fnx_o_h2f(dxh), (float) s, part[b / qb]);
            }
            out[(size_t) t * out_stride + r] = (part[0] + part[1]) + (part[2] + part[3]);
        }
}
static float rope_unit_freq(const fnx_o_rope* r, int pair, int nrot) { /* rope.hpp:33-39 */
    const float fe = powf(r->base, -2.0f * (float) pair / (float) nrot);
    if (!r->scaled) return fe;
    const float y = ((float) pair - r->c_low) / fmaxf(0.001f, r->c_high - r->c_low);
    const float ramp = 1.0f - fminf(1.0f, fmaxf(0.0f, y));
    return fe * (ramp + (1.0f - ramp) * r->inv_scale);
}
static void norm_rope(float* x, const float* w, int pos, int hd, int nrot, float eps, const fnx_o_rope* r) { /* kernels.cu:513-530 */
    double ms = 0.0;
    for (int i = 0; i < hd; ++i) ms += (double) x[i] * x[i];
    const float sc = (float) (1.0 / sqrt(ms / hd + (double) eps));
    for (int i = 0; i < hd; ++i) x[i] = x[i] * sc * w[i];
    for (int i = 0; i < nrot / 2; ++i) {
        const float theta = (float) pos * rope_unit_freq(r, i, nrot);
        const float sn = sinf(theta) * r->mscale, cs = cosf(theta) * r->mscale;
        const float x0 = x[i], x1 = x[i + nrot / 2];
        x[i] = x0 * cs - x1 * sn;
        x[i + nrot / 2] = x0 * sn + x1 * cs;
    }
}
void fnx_o_attn_prep_append(float* qg, float* k, const float* v, const float* qn, const float* kn, uint16_t* kc, uint16_t* vc, int nq,
                            int nkv, int hd, int nrot, int T, int pos0, float eps, const fnx_o_rope* rope) {
    for (int t = 0; t < T; ++t) {
        for (int h = 0; h < nq; ++h) norm_rope(qg + ((size_t) t * nq + h) * 2 * hd, qn, pos0 + t, hd, nrot, eps, rope);
        for (int h = 0; h < nkv; ++h) {
            float* kr = k + ((size_t) t * nkv + h) * hd;
            norm_rope(kr, kn, pos0 + t, hd, nrot, eps, rope);
            for (int i = 0; i < hd; ++i) {
                kc[((size_t) (pos0 + t) * nkv + h) * hd + i] = fnx_o_f2h_rn(kr[i]);
                vc[((size_t) (pos0 + t) * nkv + h) * hd + i] = fnx_o_f2h_rn(v[((size_t) t * nkv + h) * hd + i]);
            }
        }
    }
}
void fnx_o_attn(const float* qg, const uint16_t* kc, const uint16_t* vc, float* out, int nq, int nkv, int hd, int T, int pos0) {
    const int qpk = nq / nkv;
#pragma omp parallel for schedule(dynamic) collapse(2)
    for (int t = 0; t < T; ++t)
        for (int h = 0; h < nq; ++h) {
            const int ctx = pos0 + t + 1, kvh = h / qpk;
            const float* q = qg + ((size_t) t * nq + h) * 2 * hd;
            double* sc = (double*) malloc((size_t) ctx * sizeof(double));
            double* acc = (double*) calloc((size_t) hd, sizeof(double));
            double mx = -INFINITY, z = 0.0;
            for (int p = 0; p < ctx; ++p) {
                const uint16_t* kr = kc + ((size_t) p * nkv + kvh) * hd;
                double s = 0.0;
                for (int i = 0; i < hd; ++i) s += (double) q[i] * (double) fnx_o_h2f(kr[i]);
                sc[p] = s / sqrt((double) hd);
                if (sc[p] > mx) mx = sc[p];
            }
            for (int p = 0; p < ctx; ++p) {
                const double w = exp(sc[p] - mx);
                const uint16_t* vr = vc + ((size_t) p * nkv + kvh) * hd;
                z += w;
                for (int i = 0; i < hd; ++i) acc[i] += w * (double) fnx_o_h2f(vr[i]);
            }
            for (int i = 0; i < hd; ++i)
                out[((size_t) t * nq + h) * hd + i] = (float) (acc[i] / z * (1.0 / (1.0 + exp(-(double) q[hd + i]))));
            free(sc);
            free(acc);
        }
}
static void embed_rows(const uint16_t* emb, const int* tokens, int T, int n, float* y) {
    for (int t = 0; t < T; ++t)
        for (int i = 0; i < n; ++i) y[(size_t) t * n + i] = fnx_o_h2f(emb[(size_t) tokens[t] * n + i]);
}
static void dense_q8s(const fnx_o_q8s* W, const float* x, int T, float* out) { /* quantize_q8_1 then q8s_gemv (engine.cu dense()) */
    uint8_t* xq = (uint8_t*) malloc((size_t) T * (W->n_in / 32) * Q8_1_BLOCK);
    fnx_o_quantize_q8_1(x, xq, W->n_in, T);
    fnx_o_q8s_gemv(W->q, W->d, W->n_out, W->n_in, xq, out, W->n_out, T);
    free(xq);
}
/* a test's view into the layers' routing: when set, the next `layers` calls of dec_layer copy their router logits
 * ([T][nexp + 1]) and picks ([T][topk]) to consecutive slots of these arrays */
static float* g_probe_logits;
static int* g_probe_topi;
static int g_probe_left, g_probe_at;
void fnx_o_layer_probe(float* logits, int* topi, int layers) {
    g_probe_logits = logits;
    g_probe_topi = topi;
    g_probe_left = logits && topi ? layers : 0;
    g_probe_at = 0;
}
/* what a test may ask a layer for besides x: the rows as they go into the layer (x_in), the attention's rows before the output
 * projection (att: [T][nq * 256], the rows whose q8_1 form feeds wo), x after the attention half (x_mid), the MoE half's
 * rows (moe); any of them may be null. The probe below sets the same for the layers of a whole window. */
typedef struct layer_taps {
    float *x_in, *att, *x_mid, *moe;
} layer_taps;
static layer_taps g_taps; /* per layer: slot g_taps_at of each array */
static int g_taps_left, g_taps_at;
void fnx_o_layer_taps(float* x_in, float* att, float* x_mid, float* moe, int layers) {
    g_taps.x_in = x_in;
    g_taps.att = att;
    g_taps.x_mid = x_mid;
    g_taps.moe = moe;
    g_taps_left = layers;
    g_taps_at = 0;
}
static void dec_layer(const fnx_o_decoder* D, const fnx_o_dec_layer* L, float* x, int T, int pos0, int threads) {
    const int n = D->n, nq = D->nq, nkv = D->nkv, hd = 256, nrot = 64;
    float* probe_l = NULL;
    int* probe_i = NULL;
    if (g_probe_left > 0) {
        probe_l = g_probe_logits + (size_t) g_probe_at * T * (L->moe.nexp + 1);
        probe_i = g_probe_topi + (size_t) g_probe_at * T * L->moe.topk;
        --g_probe_left;
        ++g_probe_at;
    }
    layer_taps tap = {NULL, NULL, NULL, NULL};
    if (g_taps_left > 0) {
        const size_t at = (size_t) g_taps_at * T;
        if (g_taps.x_in) tap.x_in = g_taps.x_in + at * n;
        if (g_taps.att) tap.att = g_taps.att + at * nq * hd;
        if (g_taps.x_mid) tap.x_mid = g_taps.x_mid + at * n;
        if (g_taps.moe) tap.moe = g_taps.moe + at * n;
        --g_taps_left;
        ++g_taps_at;
    }
    float* xn = (float*) malloc((size_t) T * n * sizeof(float));
    float* qg = (float*) malloc((size_t) T * nq * 2 * hd * sizeof(float));
    float* k = (float*) malloc((size_t) T * nkv * hd * sizeof(float));
    float* v = (float*) malloc((size_t) T * nkv * hd * sizeof(float));
    float* att = (float*) malloc((size_t) T * nq * hd * sizeof(float));
    float* o = (float*) malloc((size_t) T * n * sizeof(float));
    if (tap.x_in) memcpy(tap.x_in, x, (size_t) T * n * sizeof(float));
    fnx_o_rms_norm_rows(x, L->attn_norm, xn, T, n, D->eps);
    dense_q8s(&L->wq, xn, T, qg);
    dense_q8s(&L->wk, xn, T, k);
    dense_q8s(&L->wv, xn, T, v);
    fnx_o_attn_prep_append(qg, k, v, L->q_norm, L->k_norm, L->kc, L->vc, nq, nkv, hd, nrot, T, pos0, D->eps, &D->rope);
    fnx_o_attn(qg, L->kc, L->vc, att, nq, nkv, hd, T, pos0);
    if (tap.att) memcpy(tap.att, att, (size_t) T * nq * hd * sizeof(float));
    dense_q8s(&L->wo, att, T, o);
    for (size_t i = 0; i < (size_t) T * n; ++i) x[i] += o[i];
    if (tap.x_mid) memcpy(tap.x_mid, x, (size_t) T * n * sizeof(float));
    fnx_o_rms_norm_rows(x, L->ffn_norm, xn, T, n, D->eps);
    fnx_o_moe_verify_layer(&L->moe, xn, T, o, probe_l, probe_i, NULL, NULL, threads);
    if (tap.moe) memcpy(tap.moe, o, (size_t) T * n * sizeof(float));
    for (size_t i = 0; i < (size_t) T * n; ++i) x[i] += o[i];
    free(xn); free(qg); free(k); free(v); free(att); free(o);
}
/* one layer on rows given by the caller (engine.cu's layer loop body): x in place; the layer's K and V go into its cache */
void fnx_o_decoder_layer(const fnx_o_decoder* D, const fnx_o_dec_layer* L, float* x, int T, int pos0, int threads) {
    dec_layer(D, L, x, T, pos0, threads);
}
/* nv head rows for the tokens from v0; pen (may be null): the last row's penalties before the picks (engine.cu:2130-2131) */
static void dec_head(const fnx_o_decoder* D, const float* norm, const fnx_o_q8s* head, const float* x, int T, float* logits_out, int* best,
                     int nv, int v0, const int* pen, const float* pen_par) {
    float* xn = (float*) malloc((size_t) T * D->n * sizeof(float));
    float* logits = logits_out ? logits_out : (float*) malloc((size_t) T * nv * sizeof(float));
    float* bv = (float*) malloc((size_t) T * sizeof(float));
    fnx_o_rms_norm_rows(x, norm, xn, T, D->n, D->eps);
    dense_q8s(head, xn, T, logits);
    if (pen) fnx_o_penalize_row(logits + (size_t) (T - 1) * nv, nv, pen, pen_par);
    fnx_o_argmax(logits, nv, T, v0, bv, best);
    free(xn);
    free(bv);
    if (!logits_out) free(logits);
}
void fnx_o_decoder_verify(const fnx_o_decoder* D, const int* tokens, int T, int pos0, float* hidden, float* logits, int* best, int threads) {
    embed_rows(D->emb, tokens, T, D->n, hidden);
    for (int l = 0; l < D->nlayers; ++l) dec_layer(D, &D->layers[l], hidden, T, pos0, threads);
    dec_head(D, D->out_norm, &D->head, hidden, T, logits, best, D->vocab, 0, NULL, NULL);
}
void fnx_o_mtp_draft(const fnx_o_decoder* D, const fnx_o_mtp* M, const float* src, const int* tokens, int T, int pos0, float* hidden,
                     float* logits, int* best, int threads) {
    const int n = D->n;
    float* xn = (float*) malloc((size_t) T * n * sizeof(float));
    float* e = (float*) malloc((size_t) T * n * sizeof(float));
    float* e2 = (float*) malloc((size_t) T * n * sizeof(float));
    float* x = (float*) malloc((size_t) T * n * sizeof(float));
    fnx_o_rms_norm_rows(src, M->norm_hid, xn, T, n, D->eps);
    dense_q8s(&M->fc_hid, xn, T, x);
    embed_rows(D->emb, tokens, T, n, e);
    fnx_o_rms_norm_rows(e, M->norm_emb, xn, T, n, D->eps);
    dense_q8s(&M->fc_emb, xn, T, e2);
    for (size_t i = 0; i < (size_t) T * n; ++i) x[i] += e2[i];
    dec_layer(D, &M->layer, x, T, pos0, threads);
    memcpy(hidden, x, (size_t) T * n * sizeof(float));
    dec_head(D, M->out_norm, &M->head, x, T, logits, best, M->dv1 > M->dv0 ? M->dv1 - M->dv0 : D->vocab, M->dv0, M->pen, M->pen_par);
    free(xn); free(e); free(e2); free(x);
}

/* ---------------------------------------------------------------- selftest.cu:29-40 */
void fnx_o_rng_init(fnx_o_rng* r, unsigned long long seed) { r->s = seed * 2685821657736338717ull + 1442695040888963407ull; }
unsigned fnx_o_rng_next(fnx_o_rng* r) {
    r->s ^= r->s >> 12;
    r->s ^= r->s << 25;
    r->s ^= r->s >> 27;
    return (unsigned) ((r->s * 2685821657736338717ull) >> 32);
}
