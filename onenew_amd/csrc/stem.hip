// First-layer convolutions: three input channels, k x k filter (7x7 or 3x3), any stride and padding, at most 64 output
// channels, fp32 NCHW.  The implicit-GEMM kernels spend this layer gathering: with three channels there is no run of the
// reduction index that is contiguous in memory, so every operand element is its own load, and the many short tiles pay
// the per-tile set-up over and over.  Here a workgroup takes 128 consecutive output pixels of one output row:
//
//   * the input patch those pixels read (3 channels x k rows x (127 stride + k) columns) is copied into LDS once with
//     coalesced loads, zeros where it hangs over the image's edge;
//   * the weights go to LDS transposed ([reduction index][output channel]);
//   * the B operand of v_mfma_f32_32x32x2_f32 is read straight from the patch: reduction index (tap, channel) is a
//     compile-time position in the patch, the pixel a stride between lanes; the reduction runs over 3 k k (+ 1 zero)
//     indices, none wasted on channel padding;
//   * wavefront w owns pixels 32 w .. 32 w + 31 and both 32-row tiles of output channels.
//
// Same arithmetic as the other fp32 convolutions of this library (fp32 products summed in fp32 by the matrix cores, bias
// after the sum, then the activation): device/x86/Conv/conv.c:1024-1056 (im2col + GEMM) with its epilogue :1216-1304.
#include <string.h>

#include "igemm_kernel.hpp"

namespace onhip {

constexpr int ST_TW = 128;   // output pixels per workgroup

struct StemParams {
    const float *x, *w, *bias;
    float *y;
    int n, h, w_in, oh, ow, cout, stride, pt, pl;
    int packed;        // weights as stem_pack_kernel lays them out (the LDS image) instead of [cout][3][k][k]
    int segs;          // row segments of 128 pixels per output row
    int pw;            // patch columns: 127 * stride + k
    Div31 div_pw;
    Epilogue ep;
};

template <int KS, int EPI, bool TWO>
__global__ __launch_bounds__(256, 2) void stem_f32_kernel(const StemParams p) {
    constexpr int CIN = 3, TAPS = KS * KS, K = TAPS * CIN, KP = (K + 1) / 2 * 2, STEPS = KP / 2;
    constexpr int ROWS = CIN * KS;                       // patch rows: (channel, filter row)
    constexpr int PATCH_MAX = ROWS * (127 * 2 + KS) + 8;   // strides up to 2 fit; larger strides are refused by the host
    __shared__ __attribute__((aligned(16))) float patch[PATCH_MAX];
    // weights in the order the matrix cores read them: [step][row tile][lane half][32 rows] (one conflict-free read per
    // operand: the 64 lanes of a wavefront hit 64 different banks)
    __shared__ __attribute__((aligned(16))) float At[KP * 64];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int pw = p.pw;
    // A workgroup is persistent: it takes a run of consecutive items (an item = 128 pixels of one output row; consecutive
    // items are neighbouring rows, whose patches overlap in all but `stride` rows: L2 hits), loads the weights once, and
    // fetches the next item's patch into registers while the matrix cores work on this one.
    const int items_total = p.n * p.oh * p.segs;
    const int per_wg = (items_total + (int) gridDim.x - 1) / (int) gridDim.x;
    const int item_begin = blockIdx.x * per_wg;
    const int item_end = min(items_total, item_begin + per_wg);
    if (item_begin >= item_end) return;

    // Every load of a phase is issued before the first one is used (fixed trip counts, values held in registers): a loop
    // that loads and stores element by element would pay the memory latency once per element.
    // Weights -> At[k][m], k = tap * 3 + channel; the pad index and rows past cout are zero.  Packed weights
    // (stem_pack_kernel) already are the LDS image: a straight 16-byte copy.
    {
        constexpr int W_PER_T = KP * 64 / 256, W4_PER_T = (KP * 64 / 4 + 255) / 256;
        static_assert(KP * 64 % 256 == 0, "whole passes over the weight tile");
        if (p.packed) {   // uniform
            float4 wq[W4_PER_T];
#pragma unroll
            for (int t = 0; t < W4_PER_T; ++t) {
                const int f = tid + t * 256;
                wq[t] = f < KP * 16 ? reinterpret_cast<const float4 *>(p.w)[f] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int t = 0; t < W4_PER_T; ++t) {
                const int f = tid + t * 256;
                if (f < KP * 16) reinterpret_cast<float4 *>(At)[f] = wq[t];
            }
        } else {
            float wv[W_PER_T];
#pragma unroll
            for (int t = 0; t < W_PER_T; ++t) {
                const int f = tid + t * 256;
                const int m = f / KP, k = f - m * KP;   // consecutive threads: consecutive k of one output channel
                const bool ok = m < p.cout && k < K;
                const int kk = ok ? k : 0, mm = ok ? m : 0;
                const int tap = kk / CIN, c = kk - tap * CIN;
                wv[t] = ok ? p.w[(mm * CIN + c) * TAPS + tap] : 0.0f;
            }
#pragma unroll
            for (int t = 0; t < W_PER_T; ++t) {
                const int f = tid + t * 256;
                const int m = f / KP, k = f - m * KP;
                At[(((k >> 1) * 2 + (m >> 5)) * 2 + (k & 1)) * 32 + (m & 31)] = wv[t];
            }
        }
        if (tid < 8) patch[ROWS * pw + tid] = 0.0f;   // the pad index reads just past the last row
    }

    // input patch of an item: row (c, i) holds input row oh * stride - pt + i of channel c, columns ow0 * stride - pl +
    // [0, pw): a thread takes column tid (and tid + 256 where the row is that long) of every row
    constexpr int PCH = (127 * 2 + KS + 255) / 256;   // column chunks of 256 per row, at most
    float pv[ROWS][PCH];
    auto issue = [&](int item) __attribute__((always_inline)) {
        int b = item;
        const int seg = b % p.segs; b /= p.segs;
        const int oh = b % p.oh, img = b / p.oh;
        const int ih0 = oh * p.stride - p.pt, iw0 = seg * ST_TW * p.stride - p.pl;
        const rsrc_t rx = make_rsrc(p.x + (size_t) img * CIN * p.h * p.w_in, (unsigned) (CIN * p.h * p.w_in * 4));
#pragma unroll
        for (int ch = 0; ch < PCH; ++ch) {
            const int col = tid + ch * 256, iw = iw0 + col;
            const bool col_in = col < pw && (unsigned) iw < (unsigned) p.w_in;
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const int ih = ih0 + r % KS;                                        // uniform
                const bool in = col_in && (unsigned) ih < (unsigned) p.h;
                pv[r][ch] = buf_load_f32(rx, in ? (unsigned) iw * 4u : OOB, (unsigned) (((r / KS) * p.h + ih) * p.w_in) * 4u);
            }
        }
    };
    const rsrc_t ry = make_rsrc(p.y, RSRC_RANGE);
    const rsrc_t rb = make_rsrc(p.bias, p.bias ? (unsigned) (p.cout * 4) : 0u);
    const bool has_bias = p.bias != nullptr;
    const float *pb = patch + (wave * 32 + li) * p.stride;
    const float *ab = At + lh * 32 + li;

    // the biases of this lane's rows: the same for every item
    float bias_r[TWO ? 2 : 1][16];
#pragma unroll
    for (int a = 0; a < (TWO ? 2 : 1); ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
            bias_r[a][r] = buf_load_f32(rb, m < p.cout ? (unsigned) m * 4u : OOB, 0);
        }

    issue(item_begin);
    for (int item = item_begin; item < item_end; ++item) {
        __syncthreads();   // everybody has read the previous patch (and, the first time, written the weights)
#pragma unroll
        for (int ch = 0; ch < PCH; ++ch) {
            const int col = tid + ch * 256;
            if (col < pw) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) patch[r * pw + col] = pv[r][ch];
            }
        }
        __syncthreads();
        if (item + 1 < item_end) issue(item + 1);   // uniform

        f32x16 acc[2];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][r] = 0.0f;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            // the two reduction indices of this step, one per lane half: positions in the patch known at compile time
            const int k0 = 2 * s, k1 = 2 * s + 1;
            const int t0 = k0 / CIN, c0 = k0 % CIN, t1 = (k1 < K ? k1 : 0) / CIN, c1 = (k1 < K ? k1 : 0) % CIN;
            const int o0 = (c0 * KS + t0 / KS) * pw + t0 % KS, o1 = (c1 * KS + t1 / KS) * pw + t1 % KS;
            const float bv = pb[lh ? o1 : o0];   // index K (the pad) multiplies a zero weight
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(ab[s * 128], bv, acc[0], 0, 0, 0);
            if constexpr (TWO) acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(ab[s * 128 + 64], bv, acc[1], 0, 0, 0);
        }

        // store: lane = pixel, rows 8 (r / 4) + 4 lh + r % 4 of each 32-channel tile
        int b = item;
        const int seg = b % p.segs; b /= p.segs;
        const int oh = b % p.oh, img = b / p.oh;
        const int ow = seg * ST_TW + wave * 32 + li;
        const bool col_ok = ow < p.ow;
#pragma unroll
        for (int a = 0; a < (TWO ? 2 : 1); ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
                const bool ok = col_ok && m < p.cout;
                const unsigned off = ok ? (unsigned) (((img * p.cout + m) * p.oh + oh) * p.ow + ow) * 4u : OOB;
                const float v = acc[a][r];
                // bias after the full sum; without a bias the value is left alone (the sign of a zero sum) and, like the
                // reference (conv.c:18-27), so is the activation: p.ep says NOT_ACT then
                const float vb = __fadd_rn(v, bias_r[a][r]);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(act_fast<EPI>(has_bias ? vb : v, p.ep)), ry, off, 0, 0);
            }
        }
    }
}

// weights [cout][3][k][k] -> [step][row tile][lane half][32 rows] (kp * 64 floats), reduction index 2 * step + lane half =
// tap * 3 + channel, row = 32 * tile + position; zeros in the pad index and past cout
__global__ __launch_bounds__(256) void stem_pack_kernel(const float *w, int cout, int taps, int kp, float *packed) {
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (f >= kp * 64) return;
    const int k = (f >> 7) * 2 + ((f >> 5) & 1), m = ((f >> 6) & 1) * 32 + (f & 31);
    const int tap = k / 3, c = k - tap * 3;
    packed[f] = (m < cout && k < taps * 3) ? w[(m * 3 + c) * taps + tap] : 0.0f;
}

int stem_pack_launch(const onhip_conv_desc_t &d, const float *w, float *packed, hipStream_t stream) {
    const int taps = d.kh * d.kw, kp = (taps * 3 + 1) / 2 * 2;
    hipLaunchKernelGGL(stem_pack_kernel, dim3((unsigned) ((kp * 64 + 255) / 256)), dim3(256), 0, stream, w, d.cout, taps, kp, packed);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// the layer has the shape this kernel is written for (whatever the image size): its packed weights have the kernel's layout
bool stem_f32_shape(const onhip_conv_desc_t &d) {
    if (d.group != 1 || d.cin != 3 || d.cout > 64 || d.kh != d.kw || (d.kh != 7 && d.kh != 3)) return false;
    if (d.stride_h != d.stride_w || d.stride_h < 1 || d.stride_h > 2) return false;
    return d.compute == ONHIP_COMPUTE_F32 && !(d.has_bias && d.act_type == SILU);
}

bool stem_f32_ok(const onhip_conv_desc_t &d, int OH, int OW) {
    if (!stem_f32_shape(d)) return false;
    const long long wgs = (long long) d.n * OH * ((OW + ST_TW - 1) / ST_TW);
    if (wgs > 0x7fffffffLL || (long long) d.n * 3 * d.h * d.w >= (1LL << 29) || (long long) d.n * d.cout * OH * OW >= (1LL << 29)) return false;
    return true;
}

template <int KS>
static int stem_launch_ks(const StemParams &p, unsigned grid, hipStream_t stream) {
    const bool two = p.cout > 32;
#define ONHIP_STEM_LAUNCH(EPI)                                                                                              \
    do {                                                                                                                    \
        if (two) hipLaunchKernelGGL((stem_f32_kernel<KS, EPI, true>), dim3(grid), dim3(256), 0, stream, p);                 \
        else hipLaunchKernelGGL((stem_f32_kernel<KS, EPI, false>), dim3(grid), dim3(256), 0, stream, p);                    \
    } while (0)
    switch (epi_of_act(p.ep.act)) {
        case EPI_NONE: ONHIP_STEM_LAUNCH(EPI_NONE); break;
        case EPI_RELU: ONHIP_STEM_LAUNCH(EPI_RELU); break;
        case EPI_CLIP: ONHIP_STEM_LAUNCH(EPI_CLIP); break;
        default: ONHIP_STEM_LAUNCH(EPI_GENERIC); break;
    }
#undef ONHIP_STEM_LAUNCH
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int stem_f32_launch(const onhip_conv_desc_t &d, int OH, int OW, const float *x, const float *w, int packed, const float *bias,
                    const Epilogue &ep, float *y, hipStream_t stream) {
    StemParams p;
    memset(&p, 0, sizeof(p));
    p.x = x; p.w = w; p.bias = d.has_bias ? bias : nullptr; p.y = y;
    p.n = d.n; p.h = d.h; p.w_in = d.w; p.oh = OH; p.ow = OW; p.cout = d.cout; p.stride = d.stride_h; p.pt = d.pad_t; p.pl = d.pad_l;
    p.packed = packed;
    p.segs = (OW + ST_TW - 1) / ST_TW;
    p.pw = (ST_TW - 1) * d.stride_h + d.kh;
    p.div_pw = make_div31((unsigned) p.pw);
    p.ep = ep;
    // 7x7: persistent workgroups, two per compute unit (what its LDS allows), each a run of consecutive row segments
    // (measured on 64 x 3 x 7 x 7 stride 2 at 32 x 224 x 224: 123 us against 136 us with one segment per workgroup).
    // 3x3: one segment per workgroup; eight fit a compute unit and hide each other's loads (32 x 3 x 3 x 3 stride 2 at
    // 64 x 224 x 224: 42 us against 50 us with 2048 persistent workgroups).
    const long long items = (long long) d.n * OH * p.segs;
    const long long resident = d.kh == 7 ? 512 : items;
    const unsigned grid = (unsigned) (items < resident ? items : resident);
    return d.kh == 7 ? stem_launch_ks<7>(p, grid, stream) : stem_launch_ks<3>(p, grid, stream);
}

}  // namespace onhip
