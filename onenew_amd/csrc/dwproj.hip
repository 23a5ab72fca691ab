// Depthwise 3x3 convolution (+ bias + activation) followed by a 1x1 convolution (+ bias + activation [+ residual Add]) in
// one launch: the second half of an inverted-residual block (MobileNetV2: depthwise + CLIP -> linear projection).  The
// depthwise result, the widest tensor of the block, never reaches memory: it is produced 16 channels at a time for the
// workgroup's band of output rows, lands in LDS as the B operand of the projection's MFMAs, and is gone.
//
// Replaces two evaluations of device/x86/Conv/conv.c: the depthwise path (:757-899; taps added in ascending (i, j)
// order to a zero sum, multiply and add rounded separately, bias last, then the activation: the same operations in the
// same order here, so the values the projection multiplies are bit-identical to the separate depthwise operator's) and
// the 1x1 convolution (im2col + GEMM :1024-1056, fp32 sums in MFMA order like the library's other fp32 convolutions).
//
//   * a workgroup owns a band of whole output rows of one image (up to 128 pixels) and all output channels, and walks
//     the depthwise channels in chunks of 16;
//   * the input rows a chunk needs (16 channels x the band's rows + halo) are fetched with 16-byte loads into registers a
//     whole chunk ahead, then laid into an LDS patch whose rows have a zero column on either side and zeros where the
//     band hangs over the top or bottom of the image: the depthwise arithmetic reads the patch without predicates;
//   * a wavefront computes four channels of the chunk (the channel is uniform in a wavefront: filter taps and bias are
//     scalar loads), a lane two pixels of the band;
//   * the projection weights come k-major ([ce][co padded to 32], packed once), a chunk is one contiguous run;
//   * v_mfma_f32_32x32x2_f32 operands: A = weights[k][m = lane % 32], B = depthwise[k][pixel = lane % 32], k = 2 s +
//     lane / 32: both conflict-free LDS reads.  Wavefront w owns the 32 pixels w of the band and every row tile.
// Per chunk: depthwise arithmetic of the chunk -> barrier -> next chunk's registers into the patch, the loads of the
// chunk after it issued -> MFMAs of the chunk -> barrier.
#include <string.h>

#include "igemm_kernel.hpp"

namespace onhip {

constexpr int DP_BN = 128;      // pixels of a band, at most
constexpr int DP_KC = 16;       // depthwise channels per chunk
constexpr int DP_SLOTS = 10;    // load slots per thread and chunk, at most
constexpr int DP_PATCH = 9472;  // floats of the input patch, at most (37 KiB)

struct DwProjParams {
    const float *x;        // [n][ce][h][w]
    const float *dw_w;     // [ce][9]
    const float *dw_b;     // [ce]
    const float *pw_t;     // [ce][cop]: the 1x1 weights k-major, output channels padded to cop with zeros
    const float *pw_b;     // [co] or nullptr
    const float *res;      // [n][co][oh][ow] or nullptr
    float *y;              // [n][co][oh][ow]
    int n, ce, h, w, oh, ow, stride, co, cop;
    int band_rows;         // output rows per workgroup
    int bands;             // bands per image
    int in_rows;           // input rows of a band: (band_rows - 1) * stride + 3
    int groups;            // load groups per input row: w / V
    int slots;             // load slots per thread: ceil(16 * in_rows * groups / 256)
    unsigned x_bytes;      // extent of x
    Div31 div_ow, div_groups, div_rowgroups;   // by ow, by groups, by in_rows * groups
    Epilogue dw_ep, pw_ep;
};

template <int DW_EPI, int MT, int V>
__global__ __launch_bounds__(256, 2) void dwproj_f32_kernel(const DwProjParams p) {
    __shared__ __attribute__((aligned(16))) float patch[DP_PATCH];
    __shared__ __attribute__((aligned(16))) float Bt[DP_KC][DP_BN];
    __shared__ __attribute__((aligned(16))) float At[2][DP_KC * MT * 32];   // [k][cop]

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int pitch = p.w + 2, plane = p.in_rows * pitch;   // patch: [channel][input row][1 + w + 1]
    const int HW = p.h * p.w, OHW = p.oh * p.ow;
    const int img = blockIdx.x / p.bands, band = blockIdx.x - img * p.bands;
    const int oh0 = band * p.band_rows;
    const int ih_first = oh0 * p.stride - 1;                // input row of patch row 0 (may be -1)
    const int chunks = p.ce / DP_KC;

    // load slots: (channel of the chunk, input row, group of V columns), the same for every chunk
    unsigned g_off[DP_SLOTS];   // byte offset inside channel 0 of the chunk; rows outside the image: out of range (zero)
    int l_off[DP_SLOTS];        // float offset in the patch, -1 = no slot
    const int total_slots = DP_KC * p.in_rows * p.groups;
#pragma unroll
    for (int i = 0; i < DP_SLOTS; ++i) {
        const int f = tid + i * 256;
        const bool live = f < total_slots;
        const int ff = live ? f : 0;
        const int k = (int) div31((unsigned) ff, p.div_rowgroups);
        const int rem = ff - k * p.in_rows * p.groups;
        const int ir = (int) div31((unsigned) rem, p.div_groups), g = rem - ir * p.groups;
        const int ih = ih_first + ir;
        const bool in = live && (unsigned) ih < (unsigned) p.h;
        g_off[i] = in ? (unsigned) ((((img * p.ce + k) * p.h + ih) * p.w + g * V)) * 4u : OOB;
        l_off[i] = live ? k * plane + ir * pitch + 1 + g * V : -1;
    }
    // this lane's two pixels of a band: patch offset of the window's top-left corner (padding column included)
    int win[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int q = lane + 64 * j;
        const bool in = q < p.band_rows * p.ow;
        const int qq = in ? q : 0;
        const int r = (int) div31((unsigned) qq, p.div_ow), c = qq - r * p.ow;
        win[j] = in ? r * p.stride * pitch + c * p.stride : -1;
    }
    // the zero columns left and right of every patch row, once
    for (int f = tid; f < DP_KC * p.in_rows; f += 256) {
        patch[f * pitch] = 0.0f;
        patch[f * pitch + p.w + 1] = 0.0f;
    }

    const rsrc_t rx = make_rsrc(p.x, p.x_bytes);
    const int a_vec = DP_KC * p.cop / 4;   // 16-byte pieces of a weight chunk
    constexpr int A_PER_T = (DP_KC * MT * 32 / 4 + 255) / 256;

    float xr[DP_SLOTS][V];
    float4 areg[A_PER_T];
    auto issue = [&](int i_chunk) __attribute__((always_inline)) {
        const unsigned soff = (unsigned) (i_chunk * DP_KC * HW) * 4u;
#pragma unroll
        for (int i = 0; i < DP_SLOTS; ++i) {
            if (i >= p.slots) break;   // uniform
            if constexpr (V == 4) {
                const uint4 q = buf_load_b128(rx, g_off[i], soff);
                xr[i][0] = __uint_as_float(q.x); xr[i][1] = __uint_as_float(q.y); xr[i][2] = __uint_as_float(q.z); xr[i][3] = __uint_as_float(q.w);
            } else {
                xr[i][0] = buf_load_f32(rx, g_off[i], soff);
            }
        }
        const float4 *src = reinterpret_cast<const float4 *>(p.pw_t + (size_t) i_chunk * DP_KC * p.cop);
#pragma unroll
        for (int i = 0; i < A_PER_T; ++i) {
            const int f = tid + i * 256;
            areg[i] = f < a_vec ? src[f] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto stage = [&](int chunk) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < DP_SLOTS; ++i) {
            if (i >= p.slots) break;
            if (l_off[i] >= 0) {
#pragma unroll
                for (int e = 0; e < V; ++e) patch[l_off[i] + e] = xr[i][e];
            }
        }
        float4 *dst = reinterpret_cast<float4 *>(At[chunk & 1]);
#pragma unroll
        for (int i = 0; i < A_PER_T; ++i) {
            const int f = tid + i * 256;
            if (f < a_vec) dst[f] = areg[i];
        }
    };
    auto depthwise = [&](int chunk) __attribute__((always_inline)) {
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            const int k = wave * 4 + cc;
            const int c = chunk * DP_KC + k;   // uniform: scalar loads
            const float *wc = p.dw_w + c * 9;
            const float bias = p.dw_b[c];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (win[j] < 0) { Bt[k][lane + 64 * j] = 0.0f; continue; }
                const float *tp = patch + k * plane + win[j];
                float acc = 0.0f;
#pragma unroll
                for (int i = 0; i < 3; ++i)
#pragma unroll
                    for (int t = 0; t < 3; ++t) acc = __fadd_rn(acc, __fmul_rn(wc[i * 3 + t], tp[i * pitch + t]));
                Bt[k][lane + 64 * j] = act_fast<DW_EPI>(__fadd_rn(acc, bias), p.dw_ep);
            }
        }
    };

    f32x16 acc[MT];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][r] = 0.0f;
    const rsrc_t ry = make_rsrc(p.y, RSRC_RANGE);
    const rsrc_t rr = make_rsrc(p.res, p.res ? RSRC_RANGE : 0u);
    const rsrc_t rb = make_rsrc(p.pw_b, p.pw_b ? (unsigned) (p.co * 4) : 0u);
    const bool has_bias = p.pw_b != nullptr, has_res = p.res != nullptr;
    const int q = wave * 32 + li;   // this lane's pixel of a band in the accumulators

    issue(0);
    __syncthreads();   // the zero columns are in place
    stage(0);
    if (chunks > 1) issue(1);
    __syncthreads();
    for (int chunk = 0; chunk < chunks; ++chunk) {
        depthwise(chunk);
        __syncthreads();
        if (chunk + 1 < chunks) stage(chunk + 1);   // uniform
        if (chunk + 2 < chunks) issue(chunk + 2);
        const float *ab = At[chunk & 1];
#pragma unroll
        for (int s = 0; s < DP_KC / 2; ++s) {
            const float b = Bt[2 * s + lh][wave * 32 + li];
#pragma unroll
            for (int a = 0; a < MT; ++a)
                acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(ab[(2 * s + lh) * p.cop + a * 32 + li], b, acc[a], 0, 0, 0);
        }
        __syncthreads();
    }

    // store: lane = pixel of the band (rows of a band are contiguous in NCHW), rows 8 (r / 4) + 4 lh + r % 4 of each tile
    const bool col_ok = q < min(p.band_rows, p.oh - oh0) * p.ow;
    const bool plain = !has_bias || p.pw_ep.act == NOT_ACT;   // conv.c:18-27: without a bias the activation is skipped too
    // every bias and residual value is requested before the first one is used: one memory round trip for the store
    float bias[MT][16], resv[MT][16];
    unsigned off[MT][16];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
            const bool ok = col_ok && m < p.co;
            off[a][r] = ok ? (unsigned) ((img * p.co + m) * OHW + oh0 * p.ow + q) * 4u : OOB;
            bias[a][r] = buf_load_f32(rb, (unsigned) m * 4u, 0);   // past the last channel, or no bias: zero
            resv[a][r] = buf_load_f32(rr, off[a][r], 0);          // no residual: an empty buffer, zeros
        }
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float v = acc[a][r];
            const float vb = __fadd_rn(v, bias[a][r]);
            v = has_bias ? vb : v;
            if (!plain) v = apply_act(v, p.pw_ep);
            const float vr = __fadd_rn(v, resv[a][r]);
            v = has_res ? vr : v;
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), ry, off[a][r], 0, 0);
        }
}

__global__ __launch_bounds__(256) void dwproj_pack_kernel(const float *w, int ce, int co, int cop, float *packed) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= ce * cop) return;
    const int k = idx / cop, m = idx - k * cop;
    packed[idx] = m < co ? w[(size_t) m * ce + k] : 0.0f;
}

int dwproj_pack_launch(const float *w, int ce, int co, float *packed, hipStream_t stream) {
    const int cop = (co + 31) / 32 * 32;
    hipLaunchKernelGGL(dwproj_pack_kernel, dim3((unsigned) ((ce * cop + 255) / 256)), dim3(256), 0, stream, w, ce, co, cop, packed);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// the band of output rows one workgroup takes, or 0 when the kernel does not fit the shape
int dwproj_band_rows(const onhip_conv_desc_t &dw, int OH, int OW, int co) {
    if (OW > DP_BN || co > 128) return 0;
    int rows = DP_BN / OW;
    rows = rows > OH ? OH : rows;
    const int v = dw.w % 4 == 0 ? 4 : 1;
    for (; rows >= 1; --rows) {
        const int in_rows = (rows - 1) * dw.stride_h + 3;
        const long long slots = ((long long) DP_KC * in_rows * (dw.w / v) + 255) / 256;
        if ((long long) DP_KC * in_rows * (dw.w + 2) <= DP_PATCH && slots <= DP_SLOTS) return rows;
    }
    return 0;
}

template <int DW_EPI, int V>
static int dwproj_launch_epi(const DwProjParams &p, hipStream_t stream) {
    const dim3 grid((unsigned) (p.n * p.bands));
    switch (p.cop / 32) {
        case 1: hipLaunchKernelGGL((dwproj_f32_kernel<DW_EPI, 1, V>), grid, dim3(256), 0, stream, p); break;
        case 2: hipLaunchKernelGGL((dwproj_f32_kernel<DW_EPI, 2, V>), grid, dim3(256), 0, stream, p); break;
        case 3: hipLaunchKernelGGL((dwproj_f32_kernel<DW_EPI, 3, V>), grid, dim3(256), 0, stream, p); break;
        default: hipLaunchKernelGGL((dwproj_f32_kernel<DW_EPI, 4, V>), grid, dim3(256), 0, stream, p); break;
    }
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// dw: the depthwise convolution (3x3, pads 1, stride 1 or 2, channels a multiple of 16), pw: the 1x1 convolution on its
// result; shapes are checked by the caller (onhip_dw_project_f32, dwproj_band_rows != 0 included)
int dwproj_f32_launch(const onhip_conv_desc_t &dw, const onhip_conv_desc_t &pw, int OH, int OW, const float *x, const float *dw_w,
                      const float *dw_b, const float *pw_t, const float *pw_b, const float *res, const Epilogue &dw_ep,
                      const Epilogue &pw_ep, float *y, hipStream_t stream) {
    DwProjParams p;
    memset(&p, 0, sizeof(p));
    p.x = x; p.dw_w = dw_w; p.dw_b = dw_b; p.pw_t = pw_t; p.pw_b = pw_b; p.res = res; p.y = y;
    p.n = dw.n; p.ce = dw.cin; p.h = dw.h; p.w = dw.w; p.oh = OH; p.ow = OW; p.stride = dw.stride_h;
    p.co = pw.cout; p.cop = (pw.cout + 31) / 32 * 32;
    p.band_rows = dwproj_band_rows(dw, OH, OW, pw.cout);
    if (p.band_rows < 1) return set_error(ONHIP_ERR_ARG, "dw + project: no band of rows fits the kernel");
    p.bands = (OH + p.band_rows - 1) / p.band_rows;
    p.in_rows = (p.band_rows - 1) * p.stride + 3;
    const int v = dw.w % 4 == 0 ? 4 : 1;
    p.groups = dw.w / v;
    p.slots = (DP_KC * p.in_rows * p.groups + 255) / 256;
    p.x_bytes = (unsigned) ((size_t) dw.n * dw.cin * dw.h * dw.w * 4);
    p.div_ow = make_div31((unsigned) OW);
    p.div_groups = make_div31((unsigned) p.groups);
    p.div_rowgroups = make_div31((unsigned) (p.in_rows * p.groups));
    p.dw_ep = dw_ep;
    p.pw_ep = pw_ep;
    if (dw_ep.act == CLIP) return v == 4 ? dwproj_launch_epi<EPI_CLIP, 4>(p, stream) : dwproj_launch_epi<EPI_CLIP, 1>(p, stream);
    return v == 4 ? dwproj_launch_epi<EPI_GENERIC, 4>(p, stream) : dwproj_launch_epi<EPI_GENERIC, 1>(p, stream);
}

}  // namespace onhip
