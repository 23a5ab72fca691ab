/*
 * onenew_oracle.c -- CPU restatement of the oneNew x86 Conv / MatMul / Gemm arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP kernels and the timed
 * CPU baseline of the benchmark.  It is never linked into, loaded by or called from the shipped
 * library; only tests/, the smoke check and the benchmark's cpu_baseline leg may use it.
 *
 * It follows the reference pass structure (zero-pad copy -> im2col -> tiled SGEMM -> bias sweep
 * -> activation sweep; direct depthwise; W8A32 quantise -> int8 im2col -> int32 GEMM -> fp32
 * de-quantise) and the reference rounding points: every output element is the sum, in ascending
 * k, of individually rounded products (no fused multiply-add except where the reference uses an
 * explicit FMA intrinsic).  Build with -ffp-contract=off.  Against the reference kernels compiled
 * with their own flags the results are bit-identical for all fp32 and int8 paths whose output is
 * square (OH == OW); see the notes on im2col below.
 *
 * The kernel functions of this file are pinned by tests/test_oracle_*.py: against the compiled
 * reference kernels (golden fixtures made by tests/golden/make_golden.py), against float64
 * brute force and against algebraic invariants.
 *
 * oracle_quant_weight_bias and the oracle_calib_* functions restate tools/optimize/model_quant.hpp,
 * which only builds together with the reference's host runtime, OpenCV and protobuf: there is no
 * reference output for them.  They are pinned by what the mathematics fixes instead
 * (tests/test_oracle_math.py): the quantiser by its closed form (product rounded before the division,
 * truncation), the histogram by numpy's bincount, the percentile by a sort, the KL and MSE searches
 * by float64 brute force of their definitions at every candidate range.  What stays open is the
 * overload of fabs / abs / log the reference gets for floats (left to its include order); the
 * float overloads are used here.
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <omp.h>

#include "onenew_oracle.h"

static int g_threads = 8; /* reference default and maximum: CMakeLists.txt:57-68 */

void oracle_set_threads(int t) { g_threads = t < 1 ? 1 : t; }
int oracle_get_threads(void) { return g_threads; }

static inline int imin(int a, int b) { return a < b ? a : b; }

int oracle_conv_out_shape(const onhip_conv_desc_t *d, int32_t *oh, int32_t *ow) {
    /* host/ops/conv.h:43-50 */
    if (d->stride_h < 1 || d->stride_w < 1 || d->kh < 1 || d->kw < 1) return -1;
    int hh = d->h + d->pad_t + d->pad_b - d->kh, ww = d->w + d->pad_l + d->pad_r - d->kw;
    if (hh < 0 || ww < 0) return -1;
    *oh = hh / d->stride_h + 1;
    *ow = ww / d->stride_w + 1;
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * activation tables
 * ------------------------------------------------------------------------------------------- */

/* host/ops/conv.h:178-194: all-float arithmetic, x = i/512 - 8 */
void oracle_build_silu_lut(float *lut) {
    const float limit = 8.0f;
    const float step = (float) (1.0 / 512);
    for (int i = 0; i < ORACLE_LUT_LEN; ++i) {
        float x = (float) i * step - limit;
        lut[i] = x / (1.0f + expf(-x));
    }
}

/* host/ops/gelu.h:80-96: `x * 0.5 * (1 + erf(x * inv_sqrt2))` in C++: erf resolves to the float
 * overload and `1 + float` stays float; only the two outer multiplications run in double. */
void oracle_build_gelu_lut(float *lut) {
    const float limit = 8.0f;
    const float step = (float) (1.0 / 512);
    const float inv_sqrt2 = 1.0f / 1.4142f;
    for (int i = 0; i < ORACLE_LUT_LEN; ++i) {
        float x = (float) i * step - limit;
        double g = (double) x * 0.5 * (double) (1.0f + erff(x * inv_sqrt2));
        lut[i] = (float) g;
    }
}

/* device/x86/Conv/conv.c:1246-1261 (SiLU) and device/x86/Gelu/gelu.c:22-38 (GELU): same rule */
static inline float lut_apply(float v, const float *lut) {
    if (v < -8.0f) return 0.0f;
    if (v >= 8.0f) return v;
    int idx = (int) ((v + 8.0f) * 512.0f);
    return lut[idx];
}

void oracle_lut_act_f32(const float *x, const float *lut, float *y, int64_t count) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t i = 0; i < count; ++i) y[i] = lut_apply(x[i], lut);
}

/* device/x86/Conv/conv.c:1216-1304.  RELU6 has no branch there: identity. */
static void act_sweep(const onhip_conv_desc_t *d, const float *lut, float *y, int64_t count) {
    switch (d->act_type) {
        case RELU:
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (int64_t i = 0; i < count; ++i) y[i] = y[i] > 0.0f ? y[i] : 0.0f;
            break;
        case SILU:
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (int64_t i = 0; i < count; ++i) y[i] = lut_apply(y[i], lut);
            break;
        case CLIP: {
            const float lo = d->clip_min, hi = d->clip_max;
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (int64_t i = 0; i < count; ++i) {
                float v = y[i] > lo ? y[i] : lo; /* max first, then min: conv.c:1274-1275 */
                y[i] = v < hi ? v : hi;
            }
            break;
        }
        case LEAKYRELU: {
            const float a = d->leaky_relu_alpha;
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (int64_t i = 0; i < count; ++i) y[i] = y[i] > 0.0f ? y[i] : a * y[i];
            break;
        }
        case HARDSILU: {
            const float a = d->hard_sigmoid_alpha, b = d->hard_sigmoid_beta;
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (int64_t i = 0; i < count; ++i) {
                float t = a * y[i] + b; /* two roundings */
                t = t > 0.0f ? t : 0.0f;
                y[i] = y[i] * (t < 1.0f ? t : 1.0f);
            }
            break;
        }
        default:
            break;
    }
}

/* ---------------------------------------------------------------------------------------------
 * SGEMM  C[M,N] = A[M,K] * B[K,N], row-major  (device/x86_utils/opt_gemm.h:17-174)
 *
 * The reference walks (m tile, n tile, k tile) blocks and, inside, adds four separately rounded
 * products at a time to the stored partial sum (:83-92); its tail steps 2-4 (:101-172) continue
 * the same running sums.  For every element this is one ascending-k chain
 *     c = 0; for k: c = c + round(a[m,k] * b[k,n])
 * which is what is computed here, blocked over n (C row chunk stays in L1) and k.
 * ------------------------------------------------------------------------------------------- */
static void sgemm_rows(float *C, const float *A, const float *B, int N, int K, int m_lo, int m_hi) {
    enum { NT = 1024, KT = 8 };
    for (int n0 = 0; n0 < N; n0 += NT) {
        const int nn = imin(NT, N - n0);
        for (int m = m_lo; m < m_hi; ++m) memset(C + (size_t) m * N + n0, 0, sizeof(float) * nn);
        for (int k0 = 0; k0 < K; k0 += KT) {
            const int k1 = imin(K, k0 + KT);
            for (int m = m_lo; m < m_hi; ++m) {
                float *restrict c = C + (size_t) m * N + n0;
                for (int k = k0; k < k1; ++k) {
                    const float a = A[(size_t) m * K + k];
                    const float *restrict b = B + (size_t) k * N + n0;
                    for (int n = 0; n < nn; ++n) c[n] = c[n] + a * b[n];
                }
            }
        }
    }
}

/* parallel over row tiles of at most 32 rows, like conv.c:395-396 / mat_mul.c:88-89 */
static void sgemm_mt(float *C, const float *A, const float *B, int M, int N, int K) {
    int mt = M / 8 > 32 ? 32 : M / 8;
    if (mt == 0) mt = M;
    const int tiles = (M + mt - 1) / mt;
#pragma omp parallel for num_threads(g_threads) schedule(dynamic, 1)
    for (int t = 0; t < tiles; ++t) sgemm_rows(C, A, B, N, K, t * mt, imin(M, (t + 1) * mt));
}

/* ---------------------------------------------------------------------------------------------
 * fp32 convolution, one image
 * ------------------------------------------------------------------------------------------- */

/* conv_pad.h:61-96: zero-padded copy */
static void pad_copy_f32(float *dst, const float *src, int C, int H, int W, int pt, int pl, int pb, int pr) {
    const int PH = H + pt + pb, PW = W + pl + pr;
    memset(dst, 0, sizeof(float) * (size_t) C * PH * PW);
    for (int c = 0; c < C; ++c)
        for (int h = 0; h < H; ++h)
            memcpy(dst + ((size_t) c * PH + h + pt) * PW + pl, src + ((size_t) c * H + h) * W, sizeof(float) * W);
}

/*
 * conv.c:168-258.  col[(c*kh*kw + i*kw + j) * OH*OW + oh*OW + ow] = xpad[c][oh*sh + i][ow*sw + j].
 * The reference spaces the (i, j) planes by OH*OH instead of OH*OW (:189-190) and multiplies ow by
 * strides[0], oh by strides[1] (:186-187,200,205); both coincide with this textbook form whenever
 * OH == OW and the strides are equal, which is every shape the reference models use.
 */
static void im2col_f32(float *col, const float *xp, int C, int PH, int PW, int kh, int kw, int sh, int sw,
                       int OH, int OW) {
    (void) PH;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int c = 0; c < C; ++c)
        for (int i = 0; i < kh; ++i)
            for (int j = 0; j < kw; ++j) {
                float *dst = col + ((size_t) (c * kh + i) * kw + j) * OH * OW;
                for (int oh = 0; oh < OH; ++oh) {
                    const float *src = xp + ((size_t) c * PH + oh * sh + i) * PW + j;
                    for (int ow = 0; ow < OW; ++ow) dst[oh * OW + ow] = src[ow * sw];
                }
            }
}

/* dense convolution with bias: conv.c:300-415 (general) and :68-166 (1x1 stride 1: no im2col) */
static void conv_dense_bias(const onhip_conv_desc_t *d, int OH, int OW, const float *x, const float *w,
                            const float *bias, float *y, float *scratch) {
    const int C = d->cin, H = d->h, W = d->w, M = d->cout, N = OH * OW, K = C * d->kh * d->kw;
    const float *bmat = x;
    const int padded = d->pad_t || d->pad_l || d->pad_b || d->pad_r;
    const int is_1x1s1 = d->kh == 1 && d->kw == 1 && d->stride_h == 1 && d->stride_w == 1;
    float *xp = scratch;
    const int PH = H + d->pad_t + d->pad_b, PW = W + d->pad_l + d->pad_r;
    if (padded) {
        pad_copy_f32(xp, x, C, H, W, d->pad_t, d->pad_l, d->pad_b, d->pad_r);
        bmat = xp;
    }
    if (!is_1x1s1) {
        float *col = scratch + (padded ? (size_t) C * PH * PW : 0);
        im2col_f32(col, bmat, C, PH, PW, d->kh, d->kw, d->stride_h, d->stride_w, OH, OW);
        bmat = col;
    }
    sgemm_mt(y, w, bmat, M, N, K);
    /* bias sweep after the full sum: conv.c:405-412 */
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int m = 0; m < M; ++m) {
        float *row = y + (size_t) m * N;
        const float b = bias[m];
        for (int n = 0; n < N; ++n) row[n] += b;
    }
}

/* dense convolution without bias: conv.c:417-525.  Row GEMM whose 8-wide body uses an explicit
 * fused multiply-add (:515) while the scalar tail (:518-520) rounds the product first. */
static void conv_dense_nobias(const onhip_conv_desc_t *d, int OH, int OW, const float *x, const float *w,
                              float *y, float *scratch) {
    const int C = d->cin, H = d->h, W = d->w, M = d->cout, N = OH * OW, K = C * d->kh * d->kw;
    const int padded = d->pad_t || d->pad_l || d->pad_b || d->pad_r;
    const int PH = H + d->pad_t + d->pad_b, PW = W + d->pad_l + d->pad_r;
    const float *src = x;
    if (padded) {
        pad_copy_f32(scratch, x, C, H, W, d->pad_t, d->pad_l, d->pad_b, d->pad_r);
        src = scratch;
    }
    float *col = scratch + (padded ? (size_t) C * PH * PW : 0);
    im2col_f32(col, src, C, PH, PW, d->kh, d->kw, d->stride_h, d->stride_w, OH, OW);
    const int nvec = N & ~7;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int m = 0; m < M; ++m) {
        float *restrict c = y + (size_t) m * N;
        memset(c, 0, sizeof(float) * N);
        for (int k = 0; k < K; ++k) {
            const float a = w[(size_t) m * K + k];
            const float *restrict b = col + (size_t) k * N;
            for (int n = 0; n < nvec; ++n) c[n] = fmaf(a, b[n], c[n]);
            for (int n = nvec; n < N; ++n) c[n] = c[n] + a * b[n];
        }
    }
}

/*
 * depthwise convolution with bias, any kernel: conv.c:527-615 (full pad, direct loops) and the
 * 3x3 / pad 1 special case :757-899 (pad rows only, edge columns handled apart).  Both add the taps
 * in ascending (i, j) order to a zero-initialised sum and add the bias last; taps that fall on
 * padding contribute +-0.  Rows are evaluated tap by tap so the compiler can vectorise along ow.
 */
static void conv_depthwise_bias(const onhip_conv_desc_t *d, int OH, int OW, const float *x, const float *w,
                                const float *bias, float *y) {
    const int C = d->cout, H = d->h, W = d->w, kh = d->kh, kw = d->kw, sh = d->stride_h, sw = d->stride_w;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int c = 0; c < C; ++c) {
        const float *wc = w + (size_t) c * kh * kw;
        const float *xc = x + (size_t) c * H * W;
        for (int oh = 0; oh < OH; ++oh) {
            float *restrict row = y + ((size_t) c * OH + oh) * OW;
            for (int ow = 0; ow < OW; ++ow) row[ow] = 0.0f;
            for (int i = 0; i < kh; ++i) {
                const int ih = oh * sh + i - d->pad_t;
                if (ih < 0 || ih >= H) continue;
                const float *restrict xr = xc + (size_t) ih * W;
                for (int j = 0; j < kw; ++j) {
                    const float wt = wc[i * kw + j];
                    /* ow range with 0 <= ow*sw + j - pad_l < W */
                    const int off = j - d->pad_l;
                    int lo = off >= 0 ? 0 : (-off + sw - 1) / sw;
                    int hi = (W - 1 - off) >= 0 ? (W - 1 - off) / sw + 1 : 0;
                    if (hi > OW) hi = OW;
                    for (int ow = lo; ow < hi; ++ow) row[ow] = row[ow] + wt * xr[ow * sw + off];
                }
            }
            const float b = bias[c];
            for (int ow = 0; ow < OW; ++ow) row[ow] = row[ow] + b;
        }
    }
}

static size_t conv_f32_scratch_floats(const onhip_conv_desc_t *d, int OH, int OW) {
    const size_t PH = d->h + d->pad_t + d->pad_b, PW = d->w + d->pad_l + d->pad_r;
    return (size_t) d->cin * PH * PW + (size_t) d->cin * d->kh * d->kw * OH * OW + 64;
}

static int check_conv_desc(const onhip_conv_desc_t *d, int32_t *OH, int32_t *OW) {
    if (d->n < 1 || d->cin < 1 || d->cout < 1 || d->h < 1 || d->w < 1) return -1;
    if (oracle_conv_out_shape(d, OH, OW)) return -1;
    if (d->group != 1 && d->cin != d->cout) return -1;
    return 0;
}

/* conv.c:13-66 dispatch, applied to each of the d->n images in turn */
int oracle_conv2d_f32(const onhip_conv_desc_t *d, const float *x, const float *w, const float *bias,
                      const float *silu_lut, float *y) {
    int32_t OH, OW;
    if (check_conv_desc(d, &OH, &OW)) return -1;
    if (d->has_bias && d->act_type == SILU && !silu_lut) return -1;
    float *scratch = NULL;
    if (d->group == 1) {
        scratch = (float *) aligned_alloc(64, ((conv_f32_scratch_floats(d, OH, OW) * 4 + 63) / 64) * 64);
        if (!scratch) return -2;
    }
    const size_t in_sz = (size_t) d->cin * d->h * d->w, out_sz = (size_t) d->cout * OH * OW;
    for (int b = 0; b < d->n; ++b) {
        const float *xb = x + b * in_sz;
        float *yb = y + b * out_sz;
        if (!d->has_bias) {
            /* conv.c:18-27: bias-less convolutions take the dense path whatever the group and
             * return before the activation.  Depthwise without bias is not meaningful there
             * (the weight would be read as [cout, cin, kh, kw]); it is rejected here. */
            if (d->group != 1) { free(scratch); return -1; }
            conv_dense_nobias(d, OH, OW, xb, w, yb, scratch);
            continue;
        }
        if (d->group != 1) conv_depthwise_bias(d, OH, OW, xb, w, bias, yb);
        else conv_dense_bias(d, OH, OW, xb, w, bias, yb, scratch);
        if (d->act_type != NOT_ACT) act_sweep(d, silu_lut, yb, (int64_t) out_sz);
    }
    free(scratch);
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * W8A32 convolution (conv.c:901-1059 dense, :1061-1214 dense without bias, :617-755 depthwise)
 * ------------------------------------------------------------------------------------------- */

/* conv.c:961-973: t = x * (1.0f / scale), clamp to [-128, 127], roundf (ties away from zero) */
void oracle_quantize_s8(const float *x, float scale, int8_t *q, int64_t count) {
    const float r = 1.0f / scale;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t i = 0; i < count; ++i) {
        float t = x[i] * r;
        t = (t < -128.0f) ? -128.0f : (t > 127.0f) ? 127.0f : t;
        q[i] = (int8_t) roundf(t);
    }
}

/* int32 accumulators of one image; zero padding contributes nothing (conv.c:979-1039, :727-738) */
static void conv_s8_acc(const onhip_conv_desc_t *d, int OH, int OW, const int8_t *q, const int8_t *w8,
                        int32_t *acc) {
    const int C = d->cin, H = d->h, W = d->w, M = d->cout, kh = d->kh, kw = d->kw;
    const int depthwise = d->group != 1;
    const int KC = depthwise ? 1 : C;
#pragma omp parallel for num_threads(g_threads) schedule(dynamic, 1)
    for (int m = 0; m < M; ++m) {
        int32_t *am = acc + (size_t) m * OH * OW;
        memset(am, 0, sizeof(int32_t) * (size_t) OH * OW);
        for (int kc = 0; kc < KC; ++kc) {
            const int8_t *qc = q + (size_t) (depthwise ? m : kc) * H * W;
            for (int i = 0; i < kh; ++i)
                for (int j = 0; j < kw; ++j) {
                    const int32_t wt = w8[((size_t) m * KC + kc) * kh * kw + i * kw + j];
                    if (wt == 0) continue;
                    const int off = j - d->pad_l;
                    int lo = off >= 0 ? 0 : (-off + d->stride_w - 1) / d->stride_w;
                    int hi = (W - 1 - off) >= 0 ? (W - 1 - off) / d->stride_w + 1 : 0;
                    if (hi > OW) hi = OW;
                    for (int oh = 0; oh < OH; ++oh) {
                        const int ih = oh * d->stride_h + i - d->pad_t;
                        if (ih < 0 || ih >= H) continue;
                        const int8_t *restrict qr = qc + (size_t) ih * W + off;
                        int32_t *restrict ar = am + (size_t) oh * OW;
                        for (int ow = lo; ow < hi; ++ow) ar[ow] += wt * (int32_t) qr[ow * d->stride_w];
                    }
                }
        }
    }
}

/* conv.c:1041-1056 (and :739,:746-752 depthwise): three separately rounded fp32 operations */
static void dequant_sweep(const onhip_conv_desc_t *d, int OH, int OW, const int32_t *acc, const int32_t *bias32,
                          const float *weight_aux, float *y) {
    const float s = d->input_scale;
    const int N = OH * OW;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int m = 0; m < d->cout; ++m) {
        const float coeff = weight_aux[m] * 1 / 127.0f;
        const int32_t *a = acc + (size_t) m * N;
        float *o = y + (size_t) m * N;
        if (d->has_bias) {
            const float b = (float) bias32[m];
            for (int n = 0; n < N; ++n) {
                float f = (float) a[n] * s;
                f = f + b;
                o[n] = f * coeff;
            }
        } else {
            for (int n = 0; n < N; ++n) {
                float f = (float) a[n] * s;
                o[n] = f * coeff;
            }
        }
    }
}

/* the consumer's input quantisation (conv.c:961-973) applied to this layer's output */
void oracle_requantize_s8(const float *y, float output_scale, int8_t *q, int64_t count) {
    oracle_quantize_s8(y, output_scale, q, count);
}

int oracle_conv2d_w8a32(const onhip_conv_desc_t *d, const float *x, const int8_t *w8, const int32_t *bias32,
                        const float *weight_aux, const float *silu_lut, void *y, int32_t *acc32) {
    int32_t OH, OW;
    if (check_conv_desc(d, &OH, &OW)) return -1;
    /* the reference pads all four sides by pads[0] (conv.c:979-999, :698-719) while the output
     * shape comes from the four individual pads: only uniform padding is self-consistent */
    if (d->pad_t != d->pad_l || d->pad_t != d->pad_b || d->pad_t != d->pad_r) return -1;
    if (!d->has_bias && d->group != 1) return -1;
    if (d->has_bias && d->act_type == SILU && !silu_lut) return -1;
    if (!(d->input_scale > 0.0f)) return -1;
    const size_t in_sz = (size_t) d->cin * d->h * d->w, out_sz = (size_t) d->cout * OH * OW;
    int8_t *q = (int8_t *) malloc(in_sz);
    int32_t *acc = (int32_t *) malloc(sizeof(int32_t) * out_sz);
    float *yf = d->out_s8 ? (float *) malloc(sizeof(float) * out_sz) : NULL;
    if (!q || !acc || (d->out_s8 && !yf)) { free(q); free(acc); free(yf); return -2; }
    for (int b = 0; b < d->n; ++b) {
        oracle_quantize_s8(x + b * in_sz, d->input_scale, q, (int64_t) in_sz);
        conv_s8_acc(d, OH, OW, q, w8, acc);
        if (acc32) memcpy(acc32 + b * out_sz, acc, sizeof(int32_t) * out_sz);
        float *yb = d->out_s8 ? yf : (float *) y + b * out_sz;
        dequant_sweep(d, OH, OW, acc, bias32, weight_aux, yb);
        if (d->has_bias && d->act_type != NOT_ACT) act_sweep(d, silu_lut, yb, (int64_t) out_sz);
        if (d->out_s8) oracle_requantize_s8(yb, d->output_scale, (int8_t *) y + b * out_sz, (int64_t) out_sz);
    }
    free(q); free(acc); free(yf);
    return 0;
}

/* tools/optimize/model_quant.hpp:6-29: per output channel max|w|, truncating conversion */
void oracle_quant_weight_bias(const float *w, const float *bias, int cout, int per_channel, int8_t *w8,
                              int32_t *bias32, float *weight_aux) {
    for (int oc = 0; oc < cout; ++oc) {
        const float *wc = w + (size_t) oc * per_channel;
        float mx = 0.0f;
        for (int i = 0; i < per_channel; ++i) {
            float a = fabsf(wc[i]);
            mx = a > mx ? a : mx;
        }
        weight_aux[oc] = mx;
        /* "w * 127 / max": the product is rounded before the division (model_quant.hpp:22,25) */
        for (int i = 0; i < per_channel; ++i) w8[(size_t) oc * per_channel + i] = (int8_t) ((wc[i] * 127.0f) / mx);
        if (bias) bias32[oc] = (int32_t) ((bias[oc] * 127.0f) / mx);
    }
}

/* ---------------------------------------------------------------------------------------------
 * Activation-scale calibration (tools/optimize/model_quant.hpp:83-185 percentile, :197-435 KL,
 * :437-623 MSE; input_scale = threshold / 127 at :668).  The reference tool only builds with the whole
 * host runtime and OpenCV, so no reference output exists for these; it calls fabs / abs / log on floats
 * without saying which overload it gets, float overloads (the evident intent) are used here.  What pins
 * them instead (tests/test_oracle_math.py): the histogram against numpy's bincount, the percentile against
 * a sort, and the value of the KL and the MSE search at every one of the 1920 candidate ranges against the
 * float64 definition (interval-overlap matrix / nearest-level brute force) on histograms whose winner is
 * inside the range, off the multiples of 128 and has mass beyond it.
 * ------------------------------------------------------------------------------------------- */

/* model_quant.hpp:287-292: running maximum of |x| over the calibration images */
float oracle_calib_abs_max(const float *x, int64_t n, float running_max) {
    float mx = running_max;
    for (int64_t i = 0; i < n; ++i) {
        const float a = fabsf(x[i]);
        mx = mx > a ? mx : a;
    }
    return mx;
}

/* model_quant.hpp:325-332: 2048-bin histogram of |x| over [0, max], zeros skipped, counts kept as floats */
void oracle_calib_histogram(const float *x, int64_t n, float max_abs, float *hist) {
    for (int64_t i = 0; i < n; ++i) {
        if (x[i] == 0.0f) continue;
        int idx = (int) (fabsf(x[i]) * ORACLE_CALIB_BINS * 1.0f / max_abs);
        idx = idx < ORACLE_CALIB_BINS - 1 ? idx : ORACLE_CALIB_BINS - 1;
        hist[idx] += 1.0f;
    }
}

/* model_quant.hpp:345-431, one value per candidate clipping range (128 ... 2047 bins): the KL divergence between
 * the clipped reference distribution (mass beyond the range folded into its last bin, :356-358) and the same range
 * seen through 128 levels (fractional bin edges, :376-392, spread back over the bins, :398-415).  kl has
 * ORACLE_CALIB_BINS - 128 entries. */
void oracle_calib_kl_curve(const float *hist, int64_t elem_count, float *kl_out) {
    enum { TARGET = 128, MIN_BINS = 128 };
    const float kl_eps = 1e-7f;
    static float p[ORACLE_CALIB_BINS], accp[ORACLE_CALIB_BINS], q[TARGET], eq[ORACLE_CALIB_BINS];
    for (int bins = MIN_BINS; bins < ORACLE_CALIB_BINS; ++bins) {
        for (int i = 0; i < bins; ++i) p[i] = accp[i] = kl_eps + hist[i];
        for (int i = bins; i < ORACLE_CALIB_BINS; ++i) accp[bins - 1] += hist[i];
        for (int i = 0; i < bins; ++i) {
            accp[i] = (float) (accp[i] / (double) elem_count);
            p[i] = (float) (p[i] / (double) elem_count);
        }
        const float ratio = (float) bins * 1.0f / TARGET;
        for (int i = 0; i < TARGET; ++i) {
            const float st = i * ratio, ed = (i + 1) * ratio;
            float v = 0.0f;
            if (floorf(st) == floorf(ed)) {
                v += (ed - st) * p[(int) floorf(st)];
            } else {
                v += (ceilf(st) - st) * p[(int) floorf(st)];
                for (int j = (int) ceilf(st); j < (int) floorf(ed); ++j) v += p[j];
                /* the reference reads p_histogram[floor(ed)], one past the end when ed == bins: that slot
                 * is multiplied by ed - floor(ed) == 0 there, so it is skipped here */
                if (ed - floorf(ed) != 0.0f) v += (ed - floorf(ed)) * p[(int) floorf(ed)];
            }
            q[i] = v / (ed - st);
        }
        for (int i = 0; i < bins; ++i) eq[i] = kl_eps;
        for (int i = 0; i < TARGET; ++i) {
            const float st = i * ratio, ed = (i + 1) * ratio;
            if (floorf(st) == floorf(ed)) {
                eq[(int) floorf(st)] += (ed - st) * q[i];
            } else {
                eq[(int) floorf(st)] += (ceilf(st) - st) * q[i];
                for (int j = (int) ceilf(st); j < (int) floorf(ed); ++j) eq[j] += 1.0f * q[i];
                const int tail = (int) floorf(ed) >= bins ? bins - 1 : (int) floorf(ed);
                eq[tail] += (ed - floorf(ed)) / 1.0f * q[i];
            }
        }
        float kl = 0.0f;
        for (int i = 0; i < bins; ++i) kl += accp[i] * logf(accp[i] / eq[i]);
        kl_out[bins - MIN_BINS] = kl;
    }
}

/* model_quant.hpp:420-431: the first candidate with the least divergence (below the starting value 32768.6);
 * threshold = (best + 0.5) * max / 2048 */
float oracle_calib_threshold_kl(const float *hist, int64_t elem_count, float max_abs) {
    static float kl[ORACLE_CALIB_BINS];
    oracle_calib_kl_curve(hist, elem_count, kl);
    float best_kl = 32768.6f;
    int best_bins = 0;
    for (int bins = 128; bins < ORACLE_CALIB_BINS; ++bins)
        if (kl[bins - 128] < best_kl) {
            best_kl = kl[bins - 128];
            best_bins = bins;
        }
    return (best_bins + 0.5f) * max_abs / ORACLE_CALIB_BINS;
}

/* model_quant.hpp:585-610, one value per candidate clipping range: the mean squared distance (in bins) of every
 * bin centre from its level on a 128-level grid over the range, values beyond it clipped to the top level */
void oracle_calib_mse_curve(const float *hist, int64_t elem_count, float *loss_out) {
    enum { TARGET = 128, MIN_BINS = 128 };
    const int32_t elem_size = (int32_t) elem_count;      /* the reference keeps the count in an int32 */
    for (int bins = MIN_BINS; bins < ORACLE_CALIB_BINS; ++bins) {
        float loss = 0.0f;
        const float step = (float) bins / (TARGET - 1);
        for (int idx = 0; idx < ORACLE_CALIB_BINS; ++idx) {
            float iq = roundf(((float) idx + 0.5f) / step);
            iq = iq > 127.0f ? 127.0f : iq;
            iq *= step;
            const float err = (float) ((float) idx + 0.5 - iq);      /* "+ 0.5" in double, stored to float */
            loss += (hist[idx] * err * err) / elem_size;
        }
        loss_out[bins - MIN_BINS] = loss;
    }
}

/* model_quant.hpp:611-618: the first candidate with the least loss (below the starting value 32768) */
float oracle_calib_threshold_mse(const float *hist, int64_t elem_count, float max_abs) {
    static float loss[ORACLE_CALIB_BINS];
    oracle_calib_mse_curve(hist, elem_count, loss);
    int best_bins = 0;
    float loss_min = 32768.0f;
    for (int bins = 128; bins < ORACLE_CALIB_BINS; ++bins)
        if (loss[bins - 128] < loss_min) {
            loss_min = loss[bins - 128];
            best_bins = bins;
        }
    return (best_bins + 0.5f) * max_abs / ORACLE_CALIB_BINS;
}

static int cmp_abs_desc(const void *a, const void *b) {
    const float x = fabsf(*(const float *) a), y = fabsf(*(const float *) b);
    return x > y ? -1 : x < y ? 1 : 0;
}

/* model_quant.hpp:99-183: every image keeps its (1 - 0.99998) * 10 * elems largest magnitudes; the threshold is
 * the element of rank (1 - 0.99998) * images * elems among all kept ones.  x holds `images` tensors of `elems`
 * values.  Returns the magnitude (the reference returns the signed element). */
float oracle_calib_threshold_percent(const float *x, int images, int32_t elems) {
    const float percent = 99.998 / 100;
    const int32_t keep = (int32_t) (elems * (1 - percent) * 10);
    const int32_t total = (int32_t) (images * elems * (1 - percent) * 10);
    float *large = (float *) calloc(total > 0 ? total : 1, sizeof(float));
    float *tmp = (float *) malloc((size_t) elems * sizeof(float));
    for (int i = 0; i < images; ++i) {
        memcpy(tmp, x + (size_t) i * elems, (size_t) elems * sizeof(float));
        qsort(tmp, elems, sizeof(float), cmp_abs_desc);
        if ((int64_t) i * keep + keep <= total) memcpy(large + (size_t) i * keep, tmp, (size_t) keep * sizeof(float));
    }
    qsort(large, total, sizeof(float), cmp_abs_desc);
    const int32_t idx = (int32_t) ((1 - percent) * images * elems);
    const float thr = (total > 0 && idx < total) ? fabsf(large[idx]) : 0.0f;
    free(tmp);
    free(large);
    return thr;
}

/* ---------------------------------------------------------------------------------------------
 * MatMul (device/x86/MatMul/mat_mul.c:10-102) and Gemm (device/x86/Gemm/gemm.c:9-79)
 * ------------------------------------------------------------------------------------------- */
int oracle_matmul_f32(int batch, int M, int K, int N, int b_shared, const float *A, const float *B, float *C) {
    if (batch < 1 || M < 1 || K < 1 || N < 1) return -1;
    /* threading policy of mat_mul.c:35-98: many batches -> one thread per batch */
    if (batch % 8 == 0 || batch > 64) {
#pragma omp parallel for num_threads(g_threads) schedule(dynamic, 1)
        for (int b = 0; b < batch; ++b)
            sgemm_rows(C + (size_t) b * M * N, A + (size_t) b * M * K, b_shared ? B : B + (size_t) b * K * N, N, K, 0, M);
    } else {
        for (int b = 0; b < batch; ++b)
            sgemm_mt(C + (size_t) b * M * N, A + (size_t) b * M * K, b_shared ? B : B + (size_t) b * K * N, M, N, K);
    }
    return 0;
}

int oracle_gemm_f32(int M, int K, int N, const float *A, const float *W, const float *bias, float *C) {
    if (M < 1 || K < 1 || N < 1) return -1;
    /* gemm.c:35-76: ascending-k scalar dot product against row n of W, bias added last */
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int m = 0; m < M; ++m) {
        const float *a = A + (size_t) m * K;
        for (int n0 = 0; n0 < N; n0 += 8) {
            const int nn = imin(8, N - n0);
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int k = 0; k < K; ++k)
                for (int t = 0; t < nn; ++t) acc[t] = acc[t] + a[k] * W[(size_t) (n0 + t) * K + k];
            for (int t = 0; t < nn; ++t) C[(size_t) m * N + n0 + t] = acc[t] + bias[n0 + t];
        }
    }
    return 0;
}

/* MatMul -> Add(bias over the last dim) -> table GELU, the chain the reference runs for a
 * transformer MLP (tools/optimize/op_fusion.hpp:195-222 keeps Gelu a node of its own).  The bias
 * Add is one rounded fp32 addition per element (device/x86/Add/add.c). */
int oracle_matmul_bias_gelu_f32(int batch, int M, int K, int N, int b_shared, const float *A, const float *B,
                                const float *bias, const float *gelu_lut, float *C) {
    int rc = oracle_matmul_f32(batch, M, K, N, b_shared, A, B, C);
    if (rc) return rc;
    const int64_t rows = (int64_t) batch * M;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        float *c = C + r * N;
        for (int n = 0; n < N; ++n) {
            float v = c[n];
            if (bias) v = v + bias[n];
            if (gelu_lut) v = lut_apply(v, gelu_lut);
            c[n] = v;
        }
    }
    return 0;
}

/* round-to-nearest-even narrowing used to model the bf16 / fp16 MFMA input modes */
void oracle_round_bf16(const float *x, float *y, int64_t count) {
    for (int64_t i = 0; i < count; ++i) {
        uint32_t u;
        memcpy(&u, &x[i], 4);
        if ((u & 0x7f800000u) != 0x7f800000u) u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
        memcpy(&y[i], &u, 4);
    }
}

void oracle_round_f16(const float *x, float *y, int64_t count) {
    /* F16C conversion, round to nearest even */
    for (int64_t i = 0; i < count; ++i) y[i] = _cvtsh_ss(_cvtss_sh(x[i], _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
}


/* ---------------------------------------------------------------------------------------------
 * The operators around the convolutions: Add, Relu, MaxPool, GlobalAveragePool
 * ------------------------------------------------------------------------------------------- */

/* device/x86/Add/add.c:18-80 and fun_0 / fun_1 / fun_2_dim3..6: out has the shape of the operand with
 * more elements (`large`); `small` is aligned to the same rank and broadcast where its extent is 1 */
int oracle_add_f32(int ndim, const int32_t *large_shape, const int32_t *small_shape, const float *large,
                   const float *small, float *out) {
    if (ndim < 1 || ndim > 6) return -1;
    int64_t n = 1;
    int32_t sstride[6], ext[6];
    int64_t acc = 1;
    for (int k = ndim - 1; k >= 0; --k) {
        if (small_shape[k] != large_shape[k] && small_shape[k] != 1) return -1;
        ext[k] = large_shape[k];
        sstride[k] = small_shape[k] == 1 ? 0 : (int32_t) acc;      /* add.c:165-167: stride 0 on broadcast dims */
        acc *= small_shape[k];
        n *= large_shape[k];
    }
    for (int64_t i = 0; i < n; ++i) {
        int64_t rest = i, j = 0;
        for (int k = ndim - 1; k >= 0; --k) {
            j += (rest % ext[k]) * sstride[k];
            rest /= ext[k];
        }
        out[i] = large[i] + small[j];
    }
    return 0;
}

/* device/x86/Relu/relu.c:21-52: 32 elements at a time through _mm256_max_ps(0, x) = (0 > x ? 0 : x), the
 * remaining n % 32 through (x > 0 ? x : 0) */
void oracle_relu_f32(const float *x, float *y, int64_t n) {
    const int64_t body = n / 32 * 32;
    for (int64_t i = 0; i < body; ++i) y[i] = 0.0f > x[i] ? 0.0f : x[i];
    for (int64_t i = body; i < n; ++i) y[i] = x[i] > 0.0f ? x[i] : 0.0f;
}

/* device/x86/MaxPool/maxpool.c:40-88 with pad_maxpool.h: pad value -32768000, running maximum from -3276800;
 * strides[0] steps along w and strides[1] along h */
int oracle_maxpool_f32(int n, int c, int h, int w, int kh, int kw, int stride_w, int stride_h, int pad, int oh, int ow,
                       const float *x, float *y) {
    if ((oh - 1) * stride_h + kh > h + 2 * pad || (ow - 1) * stride_w + kw > w + 2 * pad) return -1;
    const int ph = h + 2 * pad, pw = w + 2 * pad;
    float *padded = (float *) malloc((size_t) ph * pw * sizeof(float));
    for (int p = 0; p < n * c; ++p) {
        for (int i = 0; i < ph * pw; ++i) padded[i] = -32768000.0f;
        for (int i = 0; i < h; ++i) memcpy(padded + (size_t) (i + pad) * pw + pad, x + ((size_t) p * h + i) * w, (size_t) w * 4);
        for (int i = 0; i < oh; ++i)
            for (int j = 0; j < ow; ++j) {
                const float *win = padded + (size_t) i * stride_h * pw + j * stride_w;
                float m = -3276800.0f;
                for (int a = 0; a < kh; ++a)
                    for (int b = 0; b < kw; ++b) m = win[a * pw + b] > m ? win[a * pw + b] : m;
                y[((size_t) p * oh + i) * ow + j] = m;
            }
    }
    free(padded);
    return 0;
}

/* device/x86/GlobalAveragePool/global_avgpool.c:27-42 */
void oracle_global_avgpool_f32(int n, int c, int h, int w, const float *x, float *y) {
    const float coeff = 1.0f / (h * w);
    for (int p = 0; p < n * c; ++p) {
        float psum = 0;
        for (int i = 0; i < h * w; ++i) psum += x[(size_t) p * h * w + i];
        y[p] = psum * coeff;
    }
}


/* ---------------------------------------------------------------------------------------------
 * The operators around the MatMuls of a transformer block: LayerNormalization, Softmax, Transpose
 * (table GELU is oracle_lut_act_f32)
 * ------------------------------------------------------------------------------------------- */

/* device/x86/LayerNormalization/layer_normalization.c:28-97.  strided == 0: rows contiguous; strided != 0:
 * element i of row r at i * rows + r (the "axes[0] == 1" form).  EPSILON is the double 1e-20 (nn_common.h:19). */
void oracle_layernorm_f32(int rows, int reduce, int strided, const float *x, const float *w, const float *b, float *y) {
    const float inv_n = 1.0f / reduce;
    const int64_t step = strided ? rows : 1;
    for (int r = 0; r < rows; ++r) {
        const float *src = x + (strided ? (int64_t) r : (int64_t) r * reduce);
        float *dst = y + (strided ? (int64_t) r : (int64_t) r * reduce);
        float psum = 0, psq = 0;
        for (int i = 0; i < reduce; ++i) {
            psum += src[i * step];
            psq += src[i * step] * src[i * step];
        }
        const float mean = psum * inv_n;
        float var = inv_n * psq - mean * mean;
        var += 1e-20;
        const float inv_std = 1.0f / sqrtf(var);
        for (int i = 0; i < reduce; ++i) {
            const float t = (src[i * step] - mean) * inv_std;
            dst[i * step] = t * w[i] + b[i];
        }
    }
}

/* device/x86/Softmax/softmax.c:26-59 (last axis) and :62-118 (axis 1 of a batch-1 tensor, strided) */
void oracle_softmax_f32(int rows, int reduce, int strided, const float *x, float *y) {
    const int64_t step = strided ? rows : 1;
    for (int r = 0; r < rows; ++r) {
        const float *src = x + (strided ? (int64_t) r : (int64_t) r * reduce);
        float *dst = y + (strided ? (int64_t) r : (int64_t) r * reduce);
        float mx = -32768.0f;
        for (int i = 0; i < reduce; ++i) mx = src[i * step] > mx ? src[i * step] : mx;
        float total = 0;
        for (int i = 0; i < reduce; ++i) {
            dst[i * step] = expf(src[i * step] - mx);
            total += dst[i * step];
        }
        const float inv = 1.0f / total;
        for (int i = 0; i < reduce; ++i) dst[i * step] = dst[i * step] * inv;
    }
}

/* device/x86/Transpose/transpose.c:24-140: output dimension k comes from input dimension perm[k] */
int oracle_transpose_f32(int ndim, const int32_t *in_shape, const int32_t *perm, const float *x, float *y) {
    if (ndim < 1 || ndim > 6) return -1;
    int64_t in_stride[6], n = 1;
    for (int i = ndim - 1; i >= 0; --i) {
        in_stride[i] = n;
        n *= in_shape[i];
    }
    int32_t out_shape[6];
    int64_t cstride[6];
    for (int k = 0; k < ndim; ++k) {
        out_shape[k] = in_shape[perm[k]];
        cstride[k] = in_stride[perm[k]];
    }
    for (int64_t o = 0; o < n; ++o) {
        int64_t rest = o, src = 0;
        for (int k = ndim - 1; k >= 0; --k) {
            src += (rest % out_shape[k]) * cstride[k];
            rest /= out_shape[k];
        }
        y[o] = x[src];
    }
    return 0;
}
