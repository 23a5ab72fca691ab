// The operators either side of the MatMuls of a transformer block: table GELU, LayerNormalization,
// Softmax and Transpose.  All are bound by memory bandwidth.  GELU, LayerNormalization and Transpose
// reproduce device/x86/Gelu/gelu.c, LayerNormalization/layer_normalization.c and
// Transpose/transpose.c bit for bit; Softmax (device/x86/Softmax/softmax.c) differs from the
// reference by the last bits of expf and is held to the fp32 tolerance.
#include <string.h>

#include "onhip_internal.hpp"

namespace onhip {

__device__ __forceinline__ unsigned vg_div(unsigned x, const Div31 &d) {
    return (__umulhi(x, d.magic) >> d.shift) + (x & d.pass);
}

// ---- table GELU (gelu.c:22-38) ------------------------------------------------------------------------
__device__ __forceinline__ float gelu_lut_one(float v, const float *__restrict__ lut) {
    if (v < -8.0f) return 0.0f;
    if (v >= 8.0f) return v;
    int idx = (int) __fmul_rn(__fadd_rn(v, 8.0f), 512.0f);
    idx = idx > 8191 ? 8191 : idx;         // v just below 8: v + 8 rounds to 16 and the reference reads one past the table
    return lut[idx];                       // a NaN fails both comparisons and indexes the table with (int) NaN
}

// four elements per thread where the tensors allow 128-bit accesses (VEC), else one
template <bool VEC>
__global__ __launch_bounds__(256) void gelu_lut_kernel(const float *__restrict__ x, const float *__restrict__ lut,
                                                       float *__restrict__ y, long long n) {
    const long long i = (long long) blockIdx.x * 256 + threadIdx.x;
    if constexpr (VEC) {
        if (i * 4 + 3 < n) {
            float4 v = reinterpret_cast<const float4 *>(x)[i];
            v.x = gelu_lut_one(v.x, lut); v.y = gelu_lut_one(v.y, lut); v.z = gelu_lut_one(v.z, lut); v.w = gelu_lut_one(v.w, lut);
            reinterpret_cast<float4 *>(y)[i] = v;
        } else {
            for (long long k = i * 4; k < n; ++k) y[k] = gelu_lut_one(x[k], lut);
        }
    } else {
        if (i < n) y[i] = gelu_lut_one(x[i], lut);
    }
}

// ---- LayerNormalization ---------------------------------------------------------------------------------
// layer_normalization.c:62-97: per row, psum and psum of squares added up element by element in float, then
// mean = psum / n (as a product with 1/n), var = (1/n) * psq - mean * mean, + 1e-20 (a double constant),
// 1 / sqrtf(var), and out = (x - mean) * inv_std * weight + bias with every operation rounded.
__device__ __forceinline__ void ln_stats(float psum, float psq, float inv_n, float *mean, float *inv_std) {
    const float m = __fmul_rn(psum, inv_n);
    float var = __fsub_rn(__fmul_rn(inv_n, psq), __fmul_rn(m, m));
    var = (float) ((double) var + 1e-20);
    *mean = m;
    // sqrtf, then 1 / std, each correctly rounded as on the CPU.  The single-precision square root of this
    // toolchain is the bare v_sqrt_f32 (a last bit off on some inputs); the double-precision one rounded to float
    // is exact (53 >= 2 * 24 + 2 bits).  The two steps are kept apart so that they cannot merge into v_rsq_f32.
    float sd = (float) sqrt((double) var);
    asm volatile("" : "+v"(sd));
    *inv_std = __fdiv_rn(1.0f, sd);
}

constexpr int LN_LDS_FLOATS = 8192;

// rows contiguous in memory: a workgroup stages `rpw` rows in LDS (pitch reduce + 1, so the threads that
// each add up one row hit different banks), one thread per row does the sums in memory order, then all
// threads normalise and store
__global__ __launch_bounds__(256) void layernorm_rows_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                             const float *__restrict__ b, float *__restrict__ y, int rows,
                                                             int reduce, int rpw, float inv_n) {
    __shared__ float tile[LN_LDS_FLOATS];
    __shared__ float s_mean[64], s_inv[64];
    const int row0 = blockIdx.x * rpw;
    const int nr = min(rpw, rows - row0);
    const int pitch = reduce + 1;
    const float *src = x + (long long) row0 * reduce;
    const int total = nr * reduce;
    for (int i = threadIdx.x; i < total; i += 256) {
        const int r = i / reduce;
        tile[r * pitch + (i - r * reduce)] = src[i];
    }
    __syncthreads();
    if ((int) threadIdx.x < nr) {
        const float *t = tile + threadIdx.x * pitch;
        float psum = 0.0f, psq = 0.0f;
        for (int i = 0; i < reduce; ++i) {
            psum = __fadd_rn(psum, t[i]);
            psq = __fadd_rn(psq, __fmul_rn(t[i], t[i]));
        }
        ln_stats(psum, psq, inv_n, &s_mean[threadIdx.x], &s_inv[threadIdx.x]);
    }
    __syncthreads();
    float *dst = y + (long long) row0 * reduce;
    for (int i = threadIdx.x; i < total; i += 256) {
        const int r = i / reduce, e = i - r * reduce;
        const float t = __fmul_rn(__fsub_rn(tile[r * pitch + e], s_mean[r]), s_inv[r]);
        dst[i] = __fadd_rn(__fmul_rn(t, w[e]), b[e]);
    }
}

// The same for rows of a multiple of four floats, 16-byte aligned: a thread's share of the workgroup's rows (up to
// LN_VEC 16-byte pieces) is requested in one go and held in registers, so the staging costs one memory round trip instead of
// one per loop iteration; sums in memory order by one thread per row as above; the normalised rows leave as 16-byte stores.
constexpr int LN_VEC = 8;

__global__ __launch_bounds__(256) void layernorm_rows4_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                              const float *__restrict__ b, float *__restrict__ y, int rows,
                                                              int reduce, int rpw, float inv_n) {
    __shared__ float tile[LN_LDS_FLOATS];
    __shared__ float s_mean[64], s_inv[64];
    const int row0 = blockIdx.x * rpw;
    const int nr = min(rpw, rows - row0);
    const int pitch = reduce + 1, groups = reduce / 4;
    const int total = nr * groups;
    const float4 *src = reinterpret_cast<const float4 *>(x + (long long) row0 * reduce);
    float4 v[LN_VEC];
    int at[LN_VEC], col[LN_VEC];
#pragma unroll
    for (int i = 0; i < LN_VEC; ++i) {
        const int f = threadIdx.x + i * 256;
        const bool live = f < total;
        const int ff = live ? f : 0;
        const int r = ff / groups;
        col[i] = (ff - r * groups) * 4;
        at[i] = live ? r * pitch + col[i] : -1;
        v[i] = live ? src[ff] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
#pragma unroll
    for (int i = 0; i < LN_VEC; ++i)
        if (at[i] >= 0) {
            tile[at[i]] = v[i].x; tile[at[i] + 1] = v[i].y; tile[at[i] + 2] = v[i].z; tile[at[i] + 3] = v[i].w;
        }
    __syncthreads();
    if ((int) threadIdx.x < nr) {
        const float *t = tile + threadIdx.x * pitch;
        float psum = 0.0f, psq = 0.0f;
        for (int i = 0; i < reduce; ++i) {
            psum = __fadd_rn(psum, t[i]);
            psq = __fadd_rn(psq, __fmul_rn(t[i], t[i]));
        }
        ln_stats(psum, psq, inv_n, &s_mean[threadIdx.x], &s_inv[threadIdx.x]);
    }
    __syncthreads();
    float4 *dst = reinterpret_cast<float4 *>(y + (long long) row0 * reduce);
    float4 wv[LN_VEC], bv[LN_VEC];
#pragma unroll
    for (int i = 0; i < LN_VEC; ++i) {
        wv[i] = *reinterpret_cast<const float4 *>(w + col[i]);
        bv[i] = *reinterpret_cast<const float4 *>(b + col[i]);
    }
#pragma unroll
    for (int i = 0; i < LN_VEC; ++i) {
        if (at[i] < 0) continue;
        const int r = at[i] / pitch;
        const float m = s_mean[r], s = s_inv[r];
        float4 o;
        o.x = __fadd_rn(__fmul_rn(__fmul_rn(__fsub_rn(v[i].x, m), s), wv[i].x), bv[i].x);
        o.y = __fadd_rn(__fmul_rn(__fmul_rn(__fsub_rn(v[i].y, m), s), wv[i].y), bv[i].y);
        o.z = __fadd_rn(__fmul_rn(__fmul_rn(__fsub_rn(v[i].z, m), s), wv[i].z), bv[i].z);
        o.w = __fadd_rn(__fmul_rn(__fmul_rn(__fsub_rn(v[i].w, m), s), wv[i].w), bv[i].w);
        dst[threadIdx.x + i * 256] = o;
    }
}

// one thread per row straight from memory: rows too long for LDS (stride 1), or the "axis 1" form of
// layer_normalization.c:28-60 where the elements of a row lie `stride` apart and neighbouring threads read
// neighbouring addresses
__global__ __launch_bounds__(256) void layernorm_thread_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                               const float *__restrict__ b, float *__restrict__ y,
                                                               int rows, int reduce, long long row_step, long long stride,
                                                               float inv_n) {
    const int r = blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    const float *src = x + r * row_step;
    float *dst = y + r * row_step;
    float psum = 0.0f, psq = 0.0f;
    for (int i = 0; i < reduce; ++i) {
        const float v = src[i * stride];
        psum = __fadd_rn(psum, v);
        psq = __fadd_rn(psq, __fmul_rn(v, v));
    }
    float mean, inv_std;
    ln_stats(psum, psq, inv_n, &mean, &inv_std);
    for (int i = 0; i < reduce; ++i) {
        const float t = __fmul_rn(__fsub_rn(src[i * stride], mean), inv_std);
        dst[i * stride] = __fadd_rn(__fmul_rn(t, w[i]), b[i]);
    }
}

// ---- Softmax ----------------------------------------------------------------------------------------
// softmax.c:40-58: max from -32768, exp(x - max), sum, times 1 / sum.  Last axis: one wavefront per row.
__global__ __launch_bounds__(256) void softmax_rows_kernel(const float *__restrict__ x, float *__restrict__ y, int rows,
                                                           int reduce) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= rows) return;
    const float *src = x + (long long) row * reduce;
    float *dst = y + (long long) row * reduce;
    float m = -32768.0f;
    for (int i = lane; i < reduce; i += 64) m = src[i] > m ? src[i] : m;
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const float o = __shfl_xor(m, s, 64);
        m = o > m ? o : m;
    }
    float sum = 0.0f;
    for (int i = lane; i < reduce; i += 64) {
        const float e = expf(__fsub_rn(src[i], m));
        dst[i] = e;
        sum += e;
    }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) sum += __shfl_xor(sum, s, 64);
    const float inv = __fdiv_rn(1.0f, sum);
    for (int i = lane; i < reduce; i += 64) dst[i] = __fmul_rn(dst[i], inv);   // each lane re-reads its own stores
}

// axis 1 of a batch-1 tensor (softmax.c:85-117): element i of column c at i * cols + c; one thread per column
__global__ __launch_bounds__(256) void softmax_cols_kernel(const float *__restrict__ x, float *__restrict__ y, int cols,
                                                           int reduce) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    float m = -32768.0f;
    for (int i = 0; i < reduce; ++i) {
        const float v = x[(long long) i * cols + c];
        m = v > m ? v : m;
    }
    float sum = 0.0f;
    for (int i = 0; i < reduce; ++i) {
        const float e = expf(__fsub_rn(x[(long long) i * cols + c], m));
        y[(long long) i * cols + c] = e;
        sum = __fadd_rn(sum, e);
    }
    const float inv = __fdiv_rn(1.0f, sum);
    for (int i = 0; i < reduce; ++i) y[(long long) i * cols + c] = __fmul_rn(y[(long long) i * cols + c], inv);
}

// ---- Transpose ----------------------------------------------------------------------------------------
// out[o0..o5] = in[...] with out dim k taken from in dim perm[k] (transpose.c:52-76, :118-137): one thread per
// output element, the input offset is the dot product of the output coordinates with the permuted strides
struct TransposeParams {
    long long n;
    int ndim;
    Div31 div[6];          // by the output extents, innermost first
    int extent[6];
    int in_stride[6];      // input stride of the dimension each output dimension comes from, innermost first
};

__global__ __launch_bounds__(256) void transpose_kernel(TransposeParams p, const float *__restrict__ x, float *__restrict__ y) {
    const long long o = (long long) blockIdx.x * 256 + threadIdx.x;
    if (o >= p.n) return;
    unsigned rest = (unsigned) o;
    long long src = 0;
#pragma unroll
    for (int k = 0; k < 6; ++k) {
        if (k < p.ndim) {
            const unsigned q = vg_div(rest, p.div[k]);
            src += (long long) (rest - q * (unsigned) p.extent[k]) * p.in_stride[k];
            rest = q;
        }
    }
    y[o] = x[src];
}

// A batch of plain matrix transposes, x [batch][rows][cols] -> y [batch][cols][rows], through a 32 x 33 LDS tile: both
// the reads and the writes are runs of 32 consecutive floats (the element-wise kernel above reads one float per 32-byte
// sector there: 8 x the bytes).  Grid (column tiles, row tiles, batch).
__global__ __launch_bounds__(256) void transpose_tiled_kernel(const float *__restrict__ x, float *__restrict__ y, int rows, int cols) {
    __shared__ float tile[32][33];
    const long long base = (long long) blockIdx.z * rows * cols;
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
    for (int i = ty; i < 32; i += 8) {
        const int r = r0 + i, c = c0 + tx;
        if (r < rows && c < cols) tile[i][tx] = x[base + (long long) r * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = ty; i < 32; i += 8) {
        const int c = c0 + i, r = r0 + tx;
        if (c < cols && r < rows) y[base + (long long) c * rows + r] = tile[tx][i];
    }
}

}  // namespace onhip

using namespace onhip;

extern "C" {

int onhip_gelu_lut_f32(const float *x, const float *gelu_lut, float *y, long long n, void *stream) {
    if (!x || !gelu_lut || !y || n < 1) return set_error(ONHIP_ERR_ARG, "gelu: bad argument");
    if ((n + 255) / 256 > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "gelu: tensor too large");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0)
        hipLaunchKernelGGL(gelu_lut_kernel<true>, dim3((unsigned) ((n / 4 + 1 + 255) / 256)), dim3(256), 0, st, x, gelu_lut, y, n);
    else
        hipLaunchKernelGGL(gelu_lut_kernel<false>, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, st, x, gelu_lut, y, n);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int onhip_layernorm_f32(int32_t rows, int32_t reduce, int32_t strided, const float *x, const float *weight,
                        const float *bias, float *y, void *stream) {
    if (!x || !weight || !bias || !y || rows < 1 || reduce < 1) return set_error(ONHIP_ERR_ARG, "layernorm: bad argument");
    if ((long long) rows * reduce >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "layernorm: tensor too large");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const float inv_n = 1.0f / reduce;
    if (strided) {
        hipLaunchKernelGGL(layernorm_thread_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, x, weight, bias, y, rows,
                           reduce, 1LL, (long long) rows, inv_n);
    } else if (reduce % 4 == 0 && reduce >= 32 && reduce + 1 <= LN_LDS_FLOATS / 4 &&
               ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(bias)) & 15) == 0) {
        // as many rows per workgroup as a thread's LN_VEC registers of 16 bytes cover, at most 64, and few enough that
        // every compute unit gets a workgroup
        int rpw = LN_VEC * 256 / (reduce / 4);
        rpw = rpw > 64 ? 64 : rpw;
        if (rpw > LN_LDS_FLOATS / (reduce + 1)) rpw = LN_LDS_FLOATS / (reduce + 1);
        const int spread = (rows + 511) / 512;
        if (rpw > spread) rpw = spread < 1 ? 1 : spread;
        hipLaunchKernelGGL(layernorm_rows4_kernel, dim3((rows + rpw - 1) / rpw), dim3(256), 0, st, x, weight, bias, y, rows,
                           reduce, rpw, inv_n);
    } else if (reduce + 1 <= LN_LDS_FLOATS / 4) {
        int rpw = LN_LDS_FLOATS / (reduce + 1);
        if (rpw > 64) rpw = 64;
        hipLaunchKernelGGL(layernorm_rows_kernel, dim3((rows + rpw - 1) / rpw), dim3(256), 0, st, x, weight, bias, y, rows,
                           reduce, rpw, inv_n);
    } else {
        hipLaunchKernelGGL(layernorm_thread_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, x, weight, bias, y, rows,
                           reduce, (long long) reduce, 1LL, inv_n);
    }
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int onhip_softmax_f32(int32_t rows, int32_t reduce, int32_t strided, const float *x, float *y, void *stream) {
    if (!x || !y || rows < 1 || reduce < 1) return set_error(ONHIP_ERR_ARG, "softmax: bad argument");
    if ((long long) rows * reduce >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "softmax: tensor too large");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (strided) hipLaunchKernelGGL(softmax_cols_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, x, y, rows, reduce);
    else hipLaunchKernelGGL(softmax_rows_kernel, dim3((rows + 3) / 4), dim3(256), 0, st, x, y, rows, reduce);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int onhip_transpose_f32(const onhip_transpose_desc_t *d, const float *x, float *y, void *stream) {
    if (!d || !x || !y) return set_error(ONHIP_ERR_ARG, "transpose: null pointer");
    if (d->ndim < 1 || d->ndim > 6) return set_error(ONHIP_ERR_ARG, "transpose: rank %d (1..6 supported)", d->ndim);
    int in_stride[6], seen = 0;
    long long n = 1;
    for (int i = d->ndim - 1; i >= 0; --i) {
        if (d->in_shape[i] < 1) return set_error(ONHIP_ERR_ARG, "transpose: empty dimension");
        in_stride[i] = (int) n;
        n *= d->in_shape[i];
        if (n >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "transpose: tensor too large");
    }
    TransposeParams p;
    memset(&p, 0, sizeof(p));
    p.n = n;
    p.ndim = d->ndim;
    for (int k = 0; k < d->ndim; ++k) {        // innermost output dimension first
        const int od = d->ndim - 1 - k;
        const int id = d->perm[od];
        if (id < 0 || id >= d->ndim || (seen & (1 << id))) return set_error(ONHIP_ERR_ARG, "transpose: perm is not a permutation");
        seen |= 1 << id;
        p.extent[k] = d->in_shape[id];
        p.div[k] = make_div31((unsigned) d->in_shape[id]);
        p.in_stride[k] = in_stride[id];
    }
    // Extents of one dropped and output dimensions that are neighbours in the input as well merged, what is left may be a
    // batch of plain matrix transposes (ViT: [batch, channels, tokens, 1] <-> [batch, tokens, channels, 1]; k^T of the
    // attention): those go through the LDS tile.
    {
        long long ext[6], str[6];
        int m = 0;
        for (int k = 0; k < d->ndim; ++k) {
            if (p.extent[k] == 1) continue;
            if (m > 0 && (long long) p.in_stride[k] == str[m - 1] * ext[m - 1]) ext[m - 1] *= p.extent[k];
            else { ext[m] = p.extent[k]; str[m] = p.in_stride[k]; ++m; }
        }
        const bool matrix = (m == 2 || m == 3) && str[1] == 1 && str[0] == ext[1] && (m == 2 || str[2] == ext[0] * ext[1]);
        const long long batch = m == 3 ? ext[2] : 1;
        if (matrix && ext[0] >= 8 && ext[1] >= 8 && batch <= 65535 && (ext[0] + 31) / 32 <= 65535 && ext[0] < (1LL << 31) && ext[1] < (1LL << 31)) {
            // x [batch][rows = ext[0]][cols = ext[1]] (cols contiguous) -> y [batch][cols][rows]
            const dim3 grid((unsigned) ((ext[1] + 31) / 32), (unsigned) ((ext[0] + 31) / 32), (unsigned) batch);
            hipLaunchKernelGGL(transpose_tiled_kernel, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream), x, y, (int) ext[0], (int) ext[1]);
            ONHIP_CHECK_HIP(hipGetLastError());
            return ONHIP_OK;
        }
    }
    hipLaunchKernelGGL(transpose_kernel, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       p, x, y);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // extern "C"
