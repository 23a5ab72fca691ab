// Offline quantisation support: what turns an fp32 model into the operands the W8A32 kernels take.
//   * per-output-channel weight / bias quantiser (tools/optimize/model_quant.hpp:6-29), host arrays;
//   * activation-scale calibration (model_quant.hpp:83-185 percentile, :197-435 KL, :437-623 MSE): the
//     passes over the activations (running max |x|, 2048-bin histogram, largest magnitudes) run on the GPU
//     over device-resident tensors, the search over 1920 candidate clipping bins runs on the host.
// input_scale = threshold / 127 (model_quant.hpp:668).
#include <hipcub/hipcub.hpp>

#include <math.h>
#include <stdlib.h>
#include <string.h>

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

__global__ __launch_bounds__(256) void abs_bits_kernel(const float *x, long long n, unsigned *keys) {
    const long long i = (long long) blockIdx.x * 256 + threadIdx.x;
    if (i < n) keys[i] = __float_as_uint(x[i]) & 0x7fffffffu;
}

static int grid_for(long long n) {
    long long g = (n + 255) / 256;
    return (int) (g < 1 ? 1 : g > 4096 ? 4096 : g);
}

}  // namespace onhip

using namespace onhip;

extern "C" {

int onhip_calib_abs_max(const float *x, long long n, float *max_abs, void *stream) {
    if (!x || !max_abs || n < 1) return set_error(ONHIP_ERR_ARG, "calib abs max: bad argument");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    unsigned *bits = nullptr;
    ONHIP_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&bits), sizeof(unsigned)));
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
    (void) hipFree(bits);
    if (e != hipSuccess) return set_error(ONHIP_ERR_RUNTIME, "calib abs max: %s", hipGetErrorString(e));
    memcpy(max_abs, &result, sizeof(result));
    return ONHIP_OK;
}

int onhip_calib_histogram(const float *x, long long n, float max_abs, float *hist, void *stream) {
    if (!x || !hist || n < 1 || !(max_abs > 0.0f)) return set_error(ONHIP_ERR_ARG, "calib histogram: bad argument");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    unsigned long long *dev = nullptr;
    const size_t bytes = ONHIP_CALIB_BINS * sizeof(unsigned long long);
    ONHIP_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&dev), bytes));
    std::vector<unsigned long long> counts(ONHIP_CALIB_BINS, 0);
    hipError_t e = hipMemcpyAsync(dev, counts.data(), bytes, hipMemcpyHostToDevice, st);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(abs_histogram_kernel, dim3(grid_for(n)), dim3(256), 0, st, x, n, max_abs, dev);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(counts.data(), dev, bytes, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    (void) hipFree(dev);
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
// threshold is the magnitude of rank (1 - 0.99998) * images * elems among all kept ones.  Magnitudes are sorted
// as integers (the bit pattern of |x| orders like the value) with a device radix sort.
int onhip_calib_percentile(const float *x, int images, int elems, float *threshold, void *stream) {
    if (!x || !threshold || images < 1 || elems < 1) return set_error(ONHIP_ERR_ARG, "calib percentile: bad argument");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const float percent = 99.998 / 100;
    const int keep = (int) (elems * (1 - percent) * 10);
    const int total = (int) (images * elems * (1 - percent) * 10);
    const int rank = (int) ((1 - percent) * images * elems);
    *threshold = 0.0f;
    if (total < 1 || rank >= total || keep < 1) return ONHIP_OK;
    unsigned *keys = nullptr, *sorted = nullptr, *large = nullptr, *large_sorted = nullptr;
    void *tmp = nullptr;
    size_t tmp_bytes = 0, tmp2 = 0;
    hipError_t e = hipcub::DeviceRadixSort::SortKeysDescending(nullptr, tmp_bytes, keys, sorted, elems, 0, 32, st);
    if (e == hipSuccess) e = hipcub::DeviceRadixSort::SortKeysDescending(nullptr, tmp2, large, large_sorted, total, 0, 32, st);
    if (tmp2 > tmp_bytes) tmp_bytes = tmp2;
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&keys), (size_t) elems * 4);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&sorted), (size_t) elems * 4);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&large), (size_t) total * 4);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&large_sorted), (size_t) total * 4);
    if (e == hipSuccess) e = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 16);
    if (e == hipSuccess) e = hipMemsetAsync(large, 0, (size_t) total * 4, st);
    for (int i = 0; i < images && e == hipSuccess; ++i) {
        hipLaunchKernelGGL(abs_bits_kernel, dim3((elems + 255) / 256), dim3(256), 0, st, x + (size_t) i * elems,
                           (long long) elems, keys);
        e = hipGetLastError();
        size_t tb = tmp_bytes;
        if (e == hipSuccess) e = hipcub::DeviceRadixSort::SortKeysDescending(tmp, tb, keys, sorted, elems, 0, 32, st);
        if (e == hipSuccess && (long long) i * keep + keep <= total)
            e = hipMemcpyAsync(large + (size_t) i * keep, sorted, (size_t) keep * 4, hipMemcpyDeviceToDevice, st);
    }
    size_t tb = tmp_bytes;
    if (e == hipSuccess) e = hipcub::DeviceRadixSort::SortKeysDescending(tmp, tb, large, large_sorted, total, 0, 32, st);
    unsigned bits = 0;
    if (e == hipSuccess) e = hipMemcpyAsync(&bits, large_sorted + rank, 4, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    (void) hipFree(keys); (void) hipFree(sorted); (void) hipFree(large); (void) hipFree(large_sorted); (void) hipFree(tmp);
    if (e != hipSuccess) return set_error(ONHIP_ERR_RUNTIME, "calib percentile: %s", hipGetErrorString(e));
    memcpy(threshold, &bits, 4);
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
