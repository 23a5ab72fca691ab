// The operators either side of the convolutions of a ResNet-style graph, so that a chain can stay in
// HBM: broadcasting Add (optionally with the ReLU that follows a residual add fused in), ReLU, MaxPool
// and GlobalAveragePool.  All four are bound by memory bandwidth; results are bit-identical to
// device/x86/Add/add.c, Relu/relu.c, MaxPool/maxpool.c and GlobalAveragePool/global_avgpool.c.
#include <string.h>

#include "onhip_internal.hpp"

namespace onhip {

__device__ __forceinline__ unsigned ew_div(unsigned x, const Div31 &d) {
    return (__umulhi(x, d.magic) >> d.shift) + (x & d.pass);
}

// ---- Add -------------------------------------------------------------------------------------------
// out[i] = large[i] + small[j(i)] (add.c: the operand with fewer elements is broadcast onto the other).
// MODE 0: same number of elements, 1: small is one value, 2: per-dimension broadcast (strides 0),
// 3: small covers the trailing dimensions of large (a bias vector): its index is i mod its size; both sizes are
// multiples of 4 and everything is 16-byte aligned, four elements per thread.
struct AddParams {
    long long n;              // output elements
    int ndim;
    Div31 div[6];             // by the extents of the large operand, innermost first
    int extent[6];
    int small_stride[6];      // innermost first; 0 where the small operand is broadcast
    int relu;                 // 1: "r > 0 ? r : 0" on every element; 2: relu.c's two rules by element index (relu_body below
                              // n_body = n - n % 32, relu_tail from there on)
    long long n_body;
    Div31 div_small;          // MODE 3: by the number of float4 groups of the small operand
    int small4;
};

__device__ __forceinline__ float add_then_relu(float r, int relu, long long i, long long n_body) {
    if (relu == 2) return i < n_body ? relu_body(r) : relu_tail(r);
    return (relu && !(r > 0)) ? 0.0f : r;
}

template <int MODE>
__global__ __launch_bounds__(256) void add_kernel(AddParams p, const float *__restrict__ large,
                                                  const float *__restrict__ small, float *__restrict__ out) {
    if constexpr (MODE == 0) {
        // four elements per thread when everything is 16-byte aligned (checked by the launcher)
        const long long i4 = (long long) blockIdx.x * 256 + threadIdx.x;
        if (i4 * 4 + 3 < p.n) {
            const float4 a = reinterpret_cast<const float4 *>(large)[i4], b = reinterpret_cast<const float4 *>(small)[i4];
            // operand order of add.c:96: small + large
            float4 r = make_float4(__fadd_rn(b.x, a.x), __fadd_rn(b.y, a.y), __fadd_rn(b.z, a.z), __fadd_rn(b.w, a.w));
            if (p.relu == 2 && i4 * 4 < p.n_body) {   // n_body is a multiple of 32: the four share a rule
                r.x = relu_body(r.x); r.y = relu_body(r.y); r.z = relu_body(r.z); r.w = relu_body(r.w);
            } else if (p.relu) { r.x = r.x > 0 ? r.x : 0; r.y = r.y > 0 ? r.y : 0; r.z = r.z > 0 ? r.z : 0; r.w = r.w > 0 ? r.w : 0; }
            reinterpret_cast<float4 *>(out)[i4] = r;
        } else if (i4 * 4 < p.n) {
            for (long long i = i4 * 4; i < p.n; ++i) out[i] = add_then_relu(__fadd_rn(small[i], large[i]), p.relu, i, p.n_body);
        }
    } else if constexpr (MODE == 3) {
        const long long i4 = (long long) blockIdx.x * 256 + threadIdx.x;
        if (i4 * 4 >= p.n) return;
        const unsigned q = ew_div((unsigned) i4, p.div_small);
        const unsigned j4 = (unsigned) i4 - q * (unsigned) p.small4;
        const float4 a = reinterpret_cast<const float4 *>(large)[i4], b = reinterpret_cast<const float4 *>(small)[j4];
        float4 r = make_float4(__fadd_rn(a.x, b.x), __fadd_rn(a.y, b.y), __fadd_rn(a.z, b.z), __fadd_rn(a.w, b.w));
        if (p.relu == 2 && i4 * 4 < p.n_body) {
            r.x = relu_body(r.x); r.y = relu_body(r.y); r.z = relu_body(r.z); r.w = relu_body(r.w);
        } else if (p.relu) { r.x = r.x > 0 ? r.x : 0; r.y = r.y > 0 ? r.y : 0; r.z = r.z > 0 ? r.z : 0; r.w = r.w > 0 ? r.w : 0; }
        reinterpret_cast<float4 *>(out)[i4] = r;
    } else {
        const long long i = (long long) blockIdx.x * 256 + threadIdx.x;
        if (i >= p.n) return;
        long long j = 0;
        if constexpr (MODE == 2) {
            unsigned rest = (unsigned) i;
#pragma unroll
            for (int k = 0; k < 6; ++k) {
                if (k < p.ndim) {
                    const unsigned q = ew_div(rest, p.div[k]);
                    j += (long long) (rest - q * (unsigned) p.extent[k]) * p.small_stride[k];
                    rest = q;
                }
            }
        }
        out[i] = add_then_relu(__fadd_rn(large[i], small[j]), p.relu, i, p.n_body);
    }
}

// ---- ReLU ------------------------------------------------------------------------------------------
// relu.c:27-52: vector body and scalar tail differ on NaN and negative zero (relu_body / relu_tail); both rules
// are kept.

__global__ __launch_bounds__(256) void relu_kernel(const float *__restrict__ x, float *__restrict__ y, long long n,
                                                   long long n_body) {
    const long long i4 = (long long) blockIdx.x * 256 + threadIdx.x;
    if (i4 * 4 + 3 < n_body) {
        float4 v = reinterpret_cast<const float4 *>(x)[i4];
        v.x = relu_body(v.x); v.y = relu_body(v.y); v.z = relu_body(v.z); v.w = relu_body(v.w);
        reinterpret_cast<float4 *>(y)[i4] = v;
    } else if (i4 * 4 < n) {
        for (long long i = i4 * 4; i < min(n, i4 * 4 + 4); ++i) y[i] = i < n_body ? relu_body(x[i]) : relu_tail(x[i]);
    }
}

// ---- MaxPool -----------------------------------------------------------------------------------------
// maxpool.c:62-86: the running maximum starts at -3276800 (smaller inputs are clamped to it) and the
// padding value -32768000 never wins, so padded cells are simply skipped.  One thread per output, lanes
// along ow.
struct PoolParams {
    int planes, H, W, OH, OW, kh, kw, sw, sh, pad;
    Div31 div_ow, div_oh;
};

__global__ __launch_bounds__(256) void maxpool_kernel(PoolParams p, const float *__restrict__ x, float *__restrict__ y,
                                                      long long total) {
    const long long o = (long long) blockIdx.x * 256 + threadIdx.x;
    if (o >= total) return;
    const unsigned t = ew_div((unsigned) o, p.div_ow);
    const int ow = (int) ((unsigned) o - t * (unsigned) p.OW);
    const unsigned plane = ew_div(t, p.div_oh);
    const int oh = (int) (t - plane * (unsigned) p.OH);
    const float *src = x + (long long) plane * p.H * p.W;
    const int ih0 = oh * p.sh - p.pad, iw0 = ow * p.sw - p.pad;
    float m = -3276800.0f;
    for (int i = 0; i < p.kh; ++i) {
        const int ih = ih0 + i;
        if ((unsigned) ih >= (unsigned) p.H) continue;
        for (int j = 0; j < p.kw; ++j) {
            const int iw = iw0 + j;
            if ((unsigned) iw >= (unsigned) p.W) continue;
            const float v = src[ih * p.W + iw];
            m = v > m ? v : m;
        }
    }
    y[o] = m;
}

// Max pooling on int8 NHWC activations (channels padded to 16): a thread takes 16 channels of one output pixel, one
// 16-byte load per tap.  The quantiser of conv.c:961-973 never decreases with its argument, so the maximum of the quantised
// values is the quantised maximum: what an int8 convolution reading the fp32 result of maxpool.c would make of it (the
// -3276800 the reference starts from quantises to -128, below which no int8 lies).  cg: 16-byte groups per pixel.
__device__ __forceinline__ unsigned max_s8x4(unsigned a, unsigned b) {
    unsigned r = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int x = (int) (a << (24 - 8 * k)) >> 24, y = (int) (b << (24 - 8 * k)) >> 24;
        r |= ((unsigned) (x > y ? x : y) & 0xffu) << (8 * k);
    }
    return r;
}

__global__ __launch_bounds__(256) void maxpool_nhwc_s8_kernel(PoolParams p, const uint4 *__restrict__ x, uint4 *__restrict__ y,
                                                              long long total, int cg, Div31 div_cg) {
    const long long o = (long long) blockIdx.x * 256 + threadIdx.x;
    if (o >= total) return;
    const unsigned pix = ew_div((unsigned) o, div_cg);
    const int g = (int) ((unsigned) o - pix * (unsigned) cg);
    const unsigned t = ew_div(pix, p.div_ow);
    const int ow = (int) (pix - t * (unsigned) p.OW);
    const unsigned img = ew_div(t, p.div_oh);        // planes = images here
    const int oh = (int) (t - img * (unsigned) p.OH);
    const int ih0 = oh * p.sh - p.pad, iw0 = ow * p.sw - p.pad;
    uint4 m = make_uint4(0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u);   // -128 in every byte
    for (int i = 0; i < p.kh; ++i) {
        const int ih = ih0 + i;
        if ((unsigned) ih >= (unsigned) p.H) continue;
        for (int j = 0; j < p.kw; ++j) {
            const int iw = iw0 + j;
            if ((unsigned) iw >= (unsigned) p.W) continue;
            const uint4 v = x[((long long) (img * (unsigned) p.H + (unsigned) ih) * p.W + iw) * cg + g];
            m.x = max_s8x4(m.x, v.x); m.y = max_s8x4(m.y, v.y); m.z = max_s8x4(m.z, v.z); m.w = max_s8x4(m.w, v.w);
        }
    }
    y[o] = m;
}

// The pooling of a ResNet stem, 3x3 stride 2 padding 1 on rows of a multiple of four floats: a thread produces two
// neighbouring outputs from one 16-byte load and one single float per input row (columns 4p-1 .. 4p+3 cover both
// windows), instead of nine single loads per output.  The maximum does not depend on the order of its operands, and a
// NaN never wins in either kernel, so the results are those of maxpool_kernel bit for bit.
__global__ __launch_bounds__(256) void maxpool_3x3s2_kernel(PoolParams p, const float *__restrict__ x, float *__restrict__ y,
                                                            long long pairs, Div31 div_owp) {
    const long long o = (long long) blockIdx.x * 256 + threadIdx.x;
    if (o >= pairs) return;
    const unsigned t = ew_div((unsigned) o, div_owp);
    const int owp = (int) ((unsigned) o - t * (unsigned) (p.OW / 2));
    const unsigned plane = ew_div(t, p.div_oh);
    const int oh = (int) (t - plane * (unsigned) p.OH);
    const float *src = x + (long long) plane * p.H * p.W + 4 * owp;
    float m0 = -3276800.0f, m1 = -3276800.0f;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const int ih = 2 * oh - 1 + i;
        if ((unsigned) ih >= (unsigned) p.H) continue;
        const float *row = src + (long long) ih * p.W;
        const float4 v = *reinterpret_cast<const float4 *>(row);
        if (owp > 0) {
            const float l = row[-1];
            m0 = l > m0 ? l : m0;
        }
        m0 = v.x > m0 ? v.x : m0;
        m0 = v.y > m0 ? v.y : m0;
        m1 = v.y > m1 ? v.y : m1;
        m1 = v.z > m1 ? v.z : m1;
        m1 = v.w > m1 ? v.w : m1;
    }
    *reinterpret_cast<float2 *>(y + ((long long) plane * p.OH + oh) * p.OW + 2 * owp) = make_float2(m0, m1);
}

// ---- GlobalAveragePool -------------------------------------------------------------------------------
// global_avgpool.c:27-42: the elements of a plane are added one after the other in memory order, then the
// sum is multiplied by 1.0f / (H*W).  A workgroup copies a run of whole planes into LDS (coalesced), then
// one thread per plane adds its elements in that same order.
constexpr int GAP_LDS_FLOATS = 8192;

__global__ __launch_bounds__(256) void gap_kernel(const float *__restrict__ x, float *__restrict__ y, int planes, int hw,
                                                  int planes_per_wg, float coeff) {
    __shared__ float tile[GAP_LDS_FLOATS];
    const int plane0 = blockIdx.x * planes_per_wg;
    const int np = min(planes_per_wg, planes - plane0);
    if (planes_per_wg >= 1 && hw * planes_per_wg <= GAP_LDS_FLOATS) {
        const float *src = x + (long long) plane0 * hw;
        for (int i = threadIdx.x; i < np * hw; i += 256) tile[i] = src[i];
        __syncthreads();
        if ((int) threadIdx.x < np) {
            float s = 0.0f;
            const float *t = tile + threadIdx.x * hw;
            for (int i = 0; i < hw; ++i) s = __fadd_rn(s, t[i]);
            y[plane0 + threadIdx.x] = __fmul_rn(s, coeff);
        }
    } else {
        // planes too large for LDS: one thread per plane straight from memory (rare: pooling large maps)
        const int plane = blockIdx.x * 256 + threadIdx.x;
        if (plane >= planes) return;
        const float *t = x + (long long) plane * hw;
        float s = 0.0f;
        for (int i = 0; i < hw; ++i) s = __fadd_rn(s, t[i]);
        y[plane] = __fmul_rn(s, coeff);
    }
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace onhip

using namespace onhip;

extern "C" {

int onhip_add_f32(const onhip_add_desc_t *d, const float *large, const float *small, float *out, void *stream) {
    if (!d || !large || !small || !out) return set_error(ONHIP_ERR_ARG, "add: null pointer");
    if (d->ndim < 1 || d->ndim > 6) return set_error(ONHIP_ERR_ARG, "add: rank %d (1..6 supported)", d->ndim);
    AddParams p;
    memset(&p, 0, sizeof(p));
    long long n = 1, ns = 1;
    for (int i = 0; i < d->ndim; ++i) {
        if (d->large_shape[i] < 1 || d->small_shape[i] < 1) return set_error(ONHIP_ERR_ARG, "add: empty dimension");
        if (d->small_shape[i] != d->large_shape[i] && d->small_shape[i] != 1)
            return set_error(ONHIP_ERR_ARG, "add: shapes do not broadcast (dim %d: %d onto %d)", i, d->small_shape[i],
                             d->large_shape[i]);
        n *= d->large_shape[i];
        ns *= d->small_shape[i];
    }
    if (n >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "add: tensors of 2^31 elements or more are not supported");
    p.n = n;
    p.ndim = d->ndim;
    p.relu = d->relu == 2 ? 2 : d->relu ? 1 : 0;
    p.n_body = n - n % 32;
    int stride = 1;
    for (int k = 0; k < d->ndim; ++k) {        // innermost first
        const int dim = d->ndim - 1 - k;
        p.extent[k] = d->large_shape[dim];
        p.div[k] = make_div31((unsigned) d->large_shape[dim]);
        p.small_stride[k] = d->small_shape[dim] == 1 ? 0 : stride;
        stride *= d->small_shape[dim];
    }
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // a bias-like operand: leading extents 1, then exactly the trailing extents of the large operand
    bool trailing = ns > 1 && ns < n;
    {
        int k = 0;
        while (k < d->ndim && d->small_shape[k] == 1) ++k;
        for (; k < d->ndim; ++k) trailing = trailing && d->small_shape[k] == d->large_shape[k];
    }
    if (ns == n) {
        if (aligned16(large) && aligned16(small) && aligned16(out)) {
            hipLaunchKernelGGL(add_kernel<0>, dim3((unsigned) ((n / 4 + 1 + 255) / 256)), dim3(256), 0, st, p, large, small, out);
        } else {
            // unaligned operands: the broadcast kernel with unit strides is the same sum
            hipLaunchKernelGGL(add_kernel<2>, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, st, p, large, small, out);
        }
    } else if (trailing && ns % 4 == 0 && n % 4 == 0 && aligned16(large) && aligned16(small) && aligned16(out)) {
        p.small4 = (int) (ns / 4);
        p.div_small = make_div31((unsigned) p.small4);
        hipLaunchKernelGGL(add_kernel<3>, dim3((unsigned) ((n / 4 + 255) / 256)), dim3(256), 0, st, p, large, small, out);
    } else if (ns == 1) {
        hipLaunchKernelGGL(add_kernel<1>, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, st, p, large, small, out);
    } else {
        hipLaunchKernelGGL(add_kernel<2>, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, st, p, large, small, out);
    }
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int onhip_relu_f32(const float *x, float *y, long long n, void *stream) {
    if (!x || !y || n < 1) return set_error(ONHIP_ERR_ARG, "relu: bad argument");
    if (!aligned16(x) || !aligned16(y)) return set_error(ONHIP_ERR_ARG, "relu: tensors must be 16-byte aligned");
    hipLaunchKernelGGL(relu_kernel, dim3((unsigned) ((n / 4 + 1 + 255) / 256)), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), x, y, n, n / 32 * 32);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int onhip_maxpool_out_shape(const onhip_pool_desc_t *d, int32_t *oh, int32_t *ow) {
    if (!d || !oh || !ow) return set_error(ONHIP_ERR_ARG, "maxpool: null pointer");
    if (d->n < 1 || d->c < 1 || d->h < 1 || d->w < 1 || d->kh < 1 || d->kw < 1 || d->stride_h < 1 || d->stride_w < 1 ||
        d->pad < 0)
        return set_error(ONHIP_ERR_ARG, "maxpool: bad shape");
    if (d->h + 2 * d->pad < d->kh || d->w + 2 * d->pad < d->kw) return set_error(ONHIP_ERR_ARG, "maxpool: window larger than input");
    *oh = (d->h + 2 * d->pad - d->kh) / d->stride_h + 1;   // host/ops/max_pool.h: floor mode
    *ow = (d->w + 2 * d->pad - d->kw) / d->stride_w + 1;
    return ONHIP_OK;
}

int onhip_maxpool_f32(const onhip_pool_desc_t *d, int32_t oh, int32_t ow, const float *x, float *y, void *stream) {
    int32_t moh, mow;
    int rc = onhip_maxpool_out_shape(d, &moh, &mow);
    if (rc) return rc;
    if (!x || !y) return set_error(ONHIP_ERR_ARG, "maxpool: null pointer");
    // the output extent comes from the caller's operand descriptor, as in maxpool.c:35-38; every window must
    // lie inside the padded input
    if (oh < 1 || ow < 1 || oh > moh || ow > mow)
        return set_error(ONHIP_ERR_ARG, "maxpool: output %dx%d does not fit (at most %dx%d)", oh, ow, moh, mow);
    PoolParams p;
    p.planes = d->n * d->c; p.H = d->h; p.W = d->w; p.OH = oh; p.OW = ow;
    p.kh = d->kh; p.kw = d->kw; p.sw = d->stride_w; p.sh = d->stride_h; p.pad = d->pad;
    p.div_ow = make_div31((unsigned) ow);
    p.div_oh = make_div31((unsigned) oh);
    const long long total = (long long) p.planes * oh * ow;
    if (total >= (1LL << 31) || (long long) p.planes * d->h * d->w >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "maxpool: tensors of 2^31 elements or more are not supported");
    if (d->kh == 3 && d->kw == 3 && d->stride_h == 2 && d->stride_w == 2 && d->pad == 1 && d->w % 4 == 0 && ow == d->w / 2 &&
        aligned16(x) && (reinterpret_cast<uintptr_t>(y) & 7) == 0) {
        const long long pairs = total / 2;   // ow is even here
        hipLaunchKernelGGL(maxpool_3x3s2_kernel, dim3((unsigned) ((pairs + 255) / 256)), dim3(256), 0,
                           reinterpret_cast<hipStream_t>(stream), p, x, y, pairs, make_div31((unsigned) (ow / 2)));
    } else {
        hipLaunchKernelGGL(maxpool_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0,
                           reinterpret_cast<hipStream_t>(stream), p, x, y, total);
    }
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int onhip_maxpool_s8_nhwc(const onhip_pool_desc_t *d, int32_t oh, int32_t ow, const int8_t *x, int8_t *y, void *stream) {
    int32_t moh, mow;
    int rc = onhip_maxpool_out_shape(d, &moh, &mow);
    if (rc) return rc;
    if (!x || !y) return set_error(ONHIP_ERR_ARG, "maxpool: null pointer");
    if (oh < 1 || ow < 1 || oh > moh || ow > mow)
        return set_error(ONHIP_ERR_ARG, "maxpool: output %dx%d does not fit (at most %dx%d)", oh, ow, moh, mow);
    if (!aligned16(x) || !aligned16(y)) return set_error(ONHIP_ERR_ARG, "maxpool: int8 tensors must be 16-byte aligned");
    const int cg = (d->c + 15) / 16;
    PoolParams p;
    p.planes = d->n; p.H = d->h; p.W = d->w; p.OH = oh; p.OW = ow;
    p.kh = d->kh; p.kw = d->kw; p.sw = d->stride_w; p.sh = d->stride_h; p.pad = d->pad;
    p.div_ow = make_div31((unsigned) ow);
    p.div_oh = make_div31((unsigned) oh);
    const long long total = (long long) d->n * oh * ow * cg;
    if (total >= (1LL << 31) || (long long) d->n * d->h * d->w * cg >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "maxpool: tensors of 2^31 groups or more are not supported");
    hipLaunchKernelGGL(maxpool_nhwc_s8_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       p, reinterpret_cast<const uint4 *>(x), reinterpret_cast<uint4 *>(y), total, cg, make_div31((unsigned) cg));
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int onhip_global_avgpool_f32(int32_t n, int32_t c, int32_t h, int32_t w, const float *x, float *y, void *stream) {
    if (!x || !y || n < 1 || c < 1 || h < 1 || w < 1) return set_error(ONHIP_ERR_ARG, "global avgpool: bad argument");
    const long long planes = (long long) n * c, hw = (long long) h * w;
    if (planes * hw >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "global avgpool: tensor too large");
    const float coeff = 1.0f / (h * w);
    int ppw = (int) (GAP_LDS_FLOATS / hw);
    if (ppw > 256) ppw = 256;
    unsigned grid;
    if (ppw >= 1) {
        // keep at least a few workgroups per CU busy when there are few planes
        const long long want = (planes + 1023) / 1024;
        if (ppw > want) ppw = (int) (want < 1 ? 1 : want);
        grid = (unsigned) ((planes + ppw - 1) / ppw);
    } else {
        ppw = 0;
        grid = (unsigned) ((planes + 255) / 256);
    }
    hipLaunchKernelGGL(gap_kernel, dim3(grid), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), x, y, (int) planes,
                       (int) hw, ppw, coeff);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // extern "C"
