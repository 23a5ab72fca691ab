// Offline quantisation support: what turns an fp32 model into the operands the W8A32 kernels take.
//   * per-output-channel weight / bias quantiser (tools/optimize/model_quant.hpp:6-29), host arrays;
//   * activation-scale calibration (model_quant.hpp:83-185 percentile, :197-435 KL, :437-623 MSE): the
//     passes over the activations (running max |x|, 2048-bin histogram, digit histograms of a radix selection)
//     run on the GPU over device-resident tensors in a workspace the caller brings (nothing is allocated here),
//     the search over 1920 candidate clipping bins and the walk over the digit histograms run on the host.
// input_scale = threshold / 127 (model_quant.hpp:668).
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "onhip_internal.hpp"

namespace onhip {

// ---- running maximum of |x| -----------------------------------------------------------------------------
// |x| as an integer keeps the order of non-negative floats, so one atomicMax per workgroup does it.
__global__ __launch_bounds__(256) void abs_max_kernel(const float *x, long long n, unsigned *out_bits) {
    unsigned m = 0;
    for (long long i = (long long) blockIdx.x * 256 + threadIdx.x; i < n; i += (long long) gridDim.x * 256) {
        const unsigned b = __float_as_uint(x[i]) & 0x7fffffffu;
        // NaN compares false in the reference's "max > |x| ? max : |x|" only when max is the NaN; skip NaN here
        m = (b > m && b <= 0x7f800000u) ? b : m;
    }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const unsigned o = (unsigned) __shfl_xor((int) m, s, 64);
        m = o > m ? o : m;
    }
    if ((threadIdx.x & 63) == 0) atomicMax(out_bits, m);
}

// ---- 2048-bin histogram of |x| over [0, max_abs], zeros skipped (model_quant.hpp:325-332) ------------------
__global__ __launch_bounds__(256) void abs_histogram_kernel(const float *x, long long n, float max_abs,
                                                            unsigned long long *hist) {
    __shared__ unsigned local[ONHIP_CALIB_BINS];
    for (int i = threadIdx.x; i < ONHIP_CALIB_BINS; i += 256) local[i] = 0;
    __syncthreads();
    for (long long i = (long long) blockIdx.x * 256 + threadIdx.x; i < n; i += (long long) gridDim.x * 256) {
        const float v = x[i];
        if (v == 0.0f) continue;
        // fabs(x) * 2048 * 1.0f / max: left to right, each step rounded to float
        int idx = (int) __fdiv_rn(__fmul_rn(__fmul_rn(fabsf(v), (float) ONHIP_CALIB_BINS), 1.0f), max_abs);
        idx = idx < ONHIP_CALIB_BINS - 1 ? idx : ONHIP_CALIB_BINS - 1;
        idx = idx < 0 ? 0 : idx;
        atomicAdd(&local[idx], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < ONHIP_CALIB_BINS; i += 256)
        if (local[i]) atomicAdd(&hist[i], (unsigned long long) local[i]);
}

// ---- radix selection on the bit patterns of |x| (which order like the values) -----------------------------------
// One pass: the 256-bin histogram of the digit at `shift` over the keys of image blockIdx.y whose digits above it equal
// prefix[image] (union == 0) or the single prefix[0] (union != 0: one histogram for all images, and a key takes part
// only if it lies above its image's threshold thr[image]; images with skip[image] != 0 take no part).
__global__ __launch_bounds__(256) void select_hist_kernel(const float *x, int elems, int shift, unsigned mask,
                                                          const unsigned *prefix, const unsigned *thr, const unsigned *skip,
                                                          int united, unsigned long long *hist) {
    __shared__ unsigned local[256];
    local[threadIdx.x] = 0;
    __syncthreads();
    const int img = blockIdx.y;
    if (!united || !skip[img]) {
        const unsigned want = prefix[united ? 0 : img];
        const unsigned floor_key = united ? thr[img] : 0u;
        const float *xi = x + (size_t) img * elems;
        for (int i = blockIdx.x * 256 + threadIdx.x; i < elems; i += gridDim.x * 256) {
            const unsigned key = __float_as_uint(xi[i]) & 0x7fffffffu;
            if ((key & mask) == want && (!united || key > floor_key)) atomicAdd(&local[(key >> shift) & 255u], 1u);
        }
    }
    __syncthreads();
    if (local[threadIdx.x]) atomicAdd(&hist[(size_t) (united ? 0 : img) * 256 + threadIdx.x], (unsigned long long) local[threadIdx.x]);
}

__global__ __launch_bounds__(256) void fill_u64_kernel(unsigned long long *p, long long n) {
    const long long i = (long long) blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

static int grid_for(long long n) {
    long long g = (n + 255) / 256;
    return (int) (g < 1 ? 1 : g > 4096 ? 4096 : g);
}

}  // namespace onhip

using namespace onhip;

extern "C" {

size_t onhip_calib_workspace_bytes(int images) {
    if (images < 1) images = 1;
    // the 2048-bin histogram; or per image a 256-bin digit histogram, its prefix, its threshold and its skip flag
    const size_t hist = ONHIP_CALIB_BINS * sizeof(unsigned long long);
    const size_t sel = (size_t) images * (256 * sizeof(unsigned long long) + 3 * sizeof(unsigned));
    return ((hist > sel ? hist : sel) + 255) / 256 * 256;
}

static int check_workspace(const char *what, void *workspace, size_t bytes, size_t need) {
    if (!workspace || bytes < need)
        return set_error(ONHIP_ERR_WORKSPACE, "%s: workspace of %zu bytes needed (onhip_calib_workspace_bytes), %zu given", what, need,
                         workspace ? bytes : (size_t) 0);
    if (reinterpret_cast<uintptr_t>(workspace) % 8) return set_error(ONHIP_ERR_WORKSPACE, "%s: workspace must be 8-byte aligned", what);
    return ONHIP_OK;
}

int onhip_calib_abs_max(const float *x, long long n, float *max_abs, void *workspace, size_t workspace_bytes, void *stream) {
    if (!x || !max_abs || n < 1) return set_error(ONHIP_ERR_ARG, "calib abs max: bad argument");
    int rc = check_workspace("calib abs max", workspace, workspace_bytes, sizeof(unsigned));
    if (rc) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    unsigned *bits = static_cast<unsigned *>(workspace);
    unsigned start;
    const float cur = *max_abs > 0.0f ? *max_abs : 0.0f;
    memcpy(&start, &cur, sizeof(start));
    hipError_t e = hipMemcpyAsync(bits, &start, sizeof(start), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(abs_max_kernel, dim3(grid_for(n)), dim3(256), 0, st, x, n, bits);
        e = hipGetLastError();
    }
    unsigned result = start;
    if (e == hipSuccess) e = hipMemcpyAsync(&result, bits, sizeof(result), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return set_error(ONHIP_ERR_RUNTIME, "calib abs max: %s", hipGetErrorString(e));
    memcpy(max_abs, &result, sizeof(result));
    return ONHIP_OK;
}

int onhip_calib_histogram(const float *x, long long n, float max_abs, float *hist, void *workspace, size_t workspace_bytes,
                          void *stream) {
    if (!x || !hist || n < 1 || !(max_abs > 0.0f)) return set_error(ONHIP_ERR_ARG, "calib histogram: bad argument");
    const size_t bytes = ONHIP_CALIB_BINS * sizeof(unsigned long long);
    int rc = check_workspace("calib histogram", workspace, workspace_bytes, bytes);
    if (rc) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    unsigned long long *dev = static_cast<unsigned long long *>(workspace);
    std::vector<unsigned long long> counts(ONHIP_CALIB_BINS, 0);
    hipLaunchKernelGGL(fill_u64_kernel, dim3(ONHIP_CALIB_BINS / 256), dim3(256), 0, st, dev, (long long) ONHIP_CALIB_BINS);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) {
        hipLaunchKernelGGL(abs_histogram_kernel, dim3(grid_for(n)), dim3(256), 0, st, x, n, max_abs, dev);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(counts.data(), dev, bytes, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return set_error(ONHIP_ERR_RUNTIME, "calib histogram: %s", hipGetErrorString(e));
    // the reference keeps float counters and adds 1.0f per element: past 2^24 a float counter stops growing
    for (int i = 0; i < ONHIP_CALIB_BINS; ++i) {
        const double sum = (double) hist[i] + (double) counts[i];
        hist[i] = (hist[i] >= 16777216.0f) ? hist[i] : (sum > 16777216.0 ? 16777216.0f : (float) sum);
    }
    return ONHIP_OK;
}

// KL search (model_quant.hpp:345-431)
static float threshold_kl(const float *hist, long long elem_count, float max_abs) {
    const int target = 128, bins_total = ONHIP_CALIB_BINS;
    const float eps = 1e-7f;
    float best_kl = 32768.6f;
    int best = 0;
    std::vector<float> p(bins_total), clipped(bins_total), q(target), expanded(bins_total);
    for (int bins = 128; bins < bins_total; ++bins) {
        for (int i = 0; i < bins; ++i) {
            p[i] = eps + hist[i];
            clipped[i] = p[i];
        }
        for (int i = bins; i < bins_total; ++i) clipped[bins - 1] += hist[i];
        for (int i = 0; i < bins; ++i) {
            clipped[i] = (float) (clipped[i] / (double) elem_count);
            p[i] = (float) (p[i] / (double) elem_count);
        }
        const float ratio = (float) bins * 1.0f / target;
        for (int i = 0; i < target; ++i) {
            const float lo = i * ratio, hi = (i + 1) * ratio;
            const float flo = floorf(lo), fhi = floorf(hi);
            float v = 0.0f;
            if (flo == fhi) {
                v += (hi - lo) * p[(int) flo];
            } else {
                v += (ceilf(lo) - lo) * p[(int) flo];
                for (int j = (int) ceilf(lo); j < (int) fhi; ++j) v += p[j];
                if (hi - fhi != 0.0f) v += (hi - fhi) * p[(int) fhi];   // weight 0 at the last level: nothing to read
            }
            q[i] = v / (hi - lo);
        }
        for (int i = 0; i < bins; ++i) expanded[i] = eps;
        for (int i = 0; i < target; ++i) {
            const float lo = i * ratio, hi = (i + 1) * ratio;
            const float flo = floorf(lo), fhi = floorf(hi);
            if (flo == fhi) {
                expanded[(int) flo] += (hi - lo) * q[i];
            } else {
                expanded[(int) flo] += (ceilf(lo) - lo) * q[i];
                for (int j = (int) ceilf(lo); j < (int) fhi; ++j) expanded[j] += 1.0f * q[i];
                const int tail = (int) fhi >= bins ? bins - 1 : (int) fhi;
                expanded[tail] += (hi - fhi) / 1.0f * q[i];
            }
        }
        float kl = 0.0f;
        for (int i = 0; i < bins; ++i) kl += clipped[i] * logf(clipped[i] / expanded[i]);
        if (kl < best_kl) {
            best_kl = kl;
            best = bins;
        }
    }
    return (best + 0.5f) * max_abs / bins_total;
}

// MSE search (model_quant.hpp:585-618)
static float threshold_mse(const float *hist, long long elem_count, float max_abs) {
    const int bins_total = ONHIP_CALIB_BINS;
    const int32_t count = (int32_t) elem_count;
    float loss_min = 32768.0f;
    int best = 0;
    for (int bins = 128; bins < bins_total; ++bins) {
        const float step = (float) bins / 127;
        float loss = 0.0f;
        for (int idx = 0; idx < bins_total; ++idx) {
            float level = roundf(((float) idx + 0.5f) / step);
            level = level > 127.0f ? 127.0f : level;
            level *= step;
            const float err = (float) ((float) idx + 0.5 - level);
            loss += (hist[idx] * err * err) / count;
        }
        if (loss < loss_min) {
            loss_min = loss;
            best = bins;
        }
    }
    return (best + 0.5f) * max_abs / bins_total;
}

int onhip_calib_threshold(int method, const float *hist, long long elem_count, float max_abs, float *threshold) {
    if (!hist || !threshold || elem_count < 1 || !(max_abs > 0.0f))
        return set_error(ONHIP_ERR_ARG, "calib threshold: bad argument");
    if (method == ONHIP_CALIB_KL) *threshold = threshold_kl(hist, elem_count, max_abs);
    else if (method == ONHIP_CALIB_MSE) *threshold = threshold_mse(hist, elem_count, max_abs);
    else return set_error(ONHIP_ERR_ARG, "calib threshold: unknown method %d", method);
    return ONHIP_OK;
}

// Percentile (model_quant.hpp:99-183): per image the (1 - 0.99998) * 10 * elems largest magnitudes are kept; the
// threshold is the magnitude of rank (1 - 0.99998) * images * elems among all kept ones.  Nothing is sorted: a radix
// selection, most significant byte first, finds per image the smallest kept magnitude T_i and how many copies of it are
// kept, and then the wanted rank among everything kept (the keys above their image's T_i, counted on the device, plus
// the kept copies of each T_i and the zeros the reference's list starts from, added on the host).  Eight passes over
// the data, each a 256-bin histogram per image in the caller's workspace.
int onhip_calib_percentile(const float *x, int images, int elems, float *threshold, void *workspace, size_t workspace_bytes,
                           void *stream) {
    if (!x || !threshold || images < 1 || elems < 1) return set_error(ONHIP_ERR_ARG, "calib percentile: bad argument");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const float percent = 99.998 / 100;
    const int keep = (int) (elems * (1 - percent) * 10);
    const int total = (int) (images * elems * (1 - percent) * 10);
    const int rank = (int) ((1 - percent) * images * elems);
    *threshold = 0.0f;
    if (total < 1 || rank >= total || keep < 1) return ONHIP_OK;
    int rc = check_workspace("calib percentile", workspace, workspace_bytes, onhip_calib_workspace_bytes(images));
    if (rc) return rc;
    unsigned long long *hist = static_cast<unsigned long long *>(workspace);
    unsigned *d_prefix = reinterpret_cast<unsigned *>(hist + (size_t) images * 256);
    unsigned *d_thr = d_prefix + images, *d_skip = d_thr + images;
    std::vector<unsigned long long> h((size_t) images * 256);
    std::vector<unsigned> prefix(images, 0), skip(images, 0);
    std::vector<long long> left(images, keep - 1);   // how many larger keys of the current prefix group still precede the wanted one
    const int blocks = elems / 2048 + 1 > 1024 ? 1024 : elems / 2048 + 1;
    auto pass = [&](int shift, unsigned mask, int united) -> int {
        const long long bins = (long long) (united ? 1 : images) * 256;
        hipLaunchKernelGGL(fill_u64_kernel, dim3((unsigned) ((bins + 255) / 256)), dim3(256), 0, st, hist, bins);
        ONHIP_CHECK_HIP(hipGetLastError());
        ONHIP_CHECK_HIP(hipMemcpyAsync(d_prefix, prefix.data(), (size_t) images * 4, hipMemcpyHostToDevice, st));
        hipLaunchKernelGGL(select_hist_kernel, dim3(blocks, images), dim3(256), 0, st, x, elems, shift, mask, d_prefix, d_thr, d_skip,
                           united, hist);
        ONHIP_CHECK_HIP(hipGetLastError());
        ONHIP_CHECK_HIP(hipMemcpyAsync(h.data(), hist, (size_t) bins * 8, hipMemcpyDeviceToHost, st));
        ONHIP_CHECK_HIP(hipStreamSynchronize(st));
        return ONHIP_OK;
    };
    // per image: the keep-th largest key
    for (int shift = 24; shift >= 0; shift -= 8) {
        const unsigned mask = shift == 24 ? 0u : 0xffffffffu << (shift + 8);
        rc = pass(shift, mask, 0);
        if (rc) return rc;
        for (int i = 0; i < images; ++i) {
            long long before = 0;
            int b = 255;
            for (; b > 0; --b) {
                const long long c = (long long) h[(size_t) i * 256 + b];
                if (before + c > left[i]) break;
                before += c;
            }
            left[i] -= before;
            prefix[i] |= (unsigned) b << shift;
        }
    }
    // image i keeps every key above T_i = prefix[i] and left[i] + 1 copies of T_i; an image whose slice would run past the
    // list is not copied (model_quant.hpp:150-160 as restated by the oracle) and the list's untouched tail stays zero
    std::vector<unsigned> thr = prefix;
    long long zeros = total;
    for (int i = 0; i < images; ++i) {
        skip[i] = ((long long) i * keep + keep <= total) ? 0u : 1u;
        if (!skip[i]) zeros -= keep;
    }
    ONHIP_CHECK_HIP(hipMemcpyAsync(d_thr, thr.data(), (size_t) images * 4, hipMemcpyHostToDevice, st));
    ONHIP_CHECK_HIP(hipMemcpyAsync(d_skip, skip.data(), (size_t) images * 4, hipMemcpyHostToDevice, st));
    std::fill(prefix.begin(), prefix.end(), 0u);
    long long want = rank;
    for (int shift = 24; shift >= 0; shift -= 8) {
        const unsigned mask = shift == 24 ? 0u : 0xffffffffu << (shift + 8);
        rc = pass(shift, mask, 1);
        if (rc) return rc;
        for (int i = 0; i < images; ++i)
            if (!skip[i] && (thr[i] & mask) == prefix[0]) h[(thr[i] >> shift) & 255u] += (unsigned long long) (left[i] + 1);
        if (prefix[0] == 0u) h[0] += (unsigned long long) zeros;
        long long before = 0;
        int b = 255;
        for (; b > 0; --b) {
            const long long c = (long long) h[b];
            if (before + c > want) break;
            before += c;
        }
        want -= before;
        prefix[0] |= (unsigned) b << shift;
    }
    memcpy(threshold, &prefix[0], 4);
    return ONHIP_OK;
}

// Per output channel: aux = max|w|; w8 = (int8) (w * 127 / aux), truncating; bias32 = (int32) (b * 127 / aux)
// (model_quant.hpp:6-29).  Host arrays: this runs once, offline, on a few megabytes.
int onhip_quant_weight_bias(const float *w, const float *bias, int32_t cout, int32_t per_channel, int8_t *w8,
                            int32_t *bias32, float *weight_aux) {
    if (!w || !w8 || !weight_aux || cout < 1 || per_channel < 1 || (bias && !bias32))
        return set_error(ONHIP_ERR_ARG, "quant weight: bad argument");
    for (int32_t oc = 0; oc < cout; ++oc) {
        const float *row = w + (size_t) oc * per_channel;
        float aux = 0.0f;
        for (int32_t i = 0; i < per_channel; ++i) aux = fabsf(row[i]) > aux ? fabsf(row[i]) : aux;
        for (int32_t i = 0; i < per_channel; ++i) w8[(size_t) oc * per_channel + i] = (int8_t) (row[i] * 127 / aux);
        if (bias) bias32[oc] = (int32_t) (bias[oc] * 127 / aux);
        weight_aux[oc] = aux;
    }
    return ONHIP_OK;
}

}  // extern "C"
