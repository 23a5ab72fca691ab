// A whole inverted-residual block in one launch: 1x1 expansion (+ bias + activation) -> depthwise 3x3 (pads 1, stride 1
// or 2, + bias + activation) -> 1x1 projection (+ bias + activation) [-> Add of a residual tensor].  The two wide tensors
// of the block (MobileNetV2: six times the block's input) never reach memory.  Replaces three (four) evaluations of the
// reference's operators: device/x86/Conv/conv.c 1x1 path (:1024-1056) twice, the depthwise path (:757-899) and
// device/x86/Add/add.c.
//
//   * a workgroup owns a band of whole output rows of one image (up to 128 pixels) and all output channels; the block's
//     input for those rows plus the halo rows (every input channel) is loaded once into LDS, Xs[channel][row][column];
//   * the expanded channels are walked in chunks of 16.  The chunk's expansion is an MFMA product
//     W_exp[16 x cin] . Xs[cin x patch pixels] (v_mfma_f32_16x16x4_f32: A = weights[m = lane % 16][k = lane / 16], packed
//     once so that a lane's values are consecutive words; B = Xs[k = lane / 16][pixel = lane % 16]; D = [m = 4 (lane / 16)
//     + r][pixel = lane % 16]) whose result goes, with bias and activation, into the LDS patch the depthwise stage reads:
//     [channel / 4][input row][1 + w + 1][channel % 4], a zero column on either side, rows above / below the image left
//     zero; a lane's four values are one 16-byte store, and the depthwise stage reads a tap of four channels at once.  Halo rows
//     are expanded by both neighbouring bands: (rows + 2) / rows (stride 1) of the expansion's arithmetic, none of its
//     memory traffic;
//   * depthwise and projection as in dwproj.hip: taps added in ascending (i, j) order to a zero sum, multiply and add
//     rounded separately, bias last (conv.c:757-899), so the depthwise stage is bit-identical to the operator on the same
//     input; the projection accumulates in v_mfma_f32_32x32x2_f32 with its weights k-major in registers;
//   * per chunk: [projection of the previous chunk, expansion of this one] -> barrier -> depthwise -> barrier.  Two
//     workgroups share a compute unit, one in its MFMA phase while the other does depthwise arithmetic.
// The expansion sums in another order than the library's separate 1x1 kernel (k in steps of 4 instead of 2), so the block
// equals the chain of three operators within fp32 summation error, not bit for bit.
#include <stdlib.h>
#include <string.h>

#include <atomic>

#include "igemm_kernel.hpp"

namespace onhip {

constexpr int IR_BN = 128;        // output pixels of a band, at most
constexpr int IR_KC = 16;         // expanded channels per chunk
constexpr int IR_XSLOTS = 12;
constexpr int IR_TPW = 9;         // pixel tiles of the expansion per wavefront, at most     // 16-byte input loads per thread, at most
constexpr int IR_LDS_HALF = 80 * 1024;   // bytes of LDS a workgroup may take: two workgroups per compute unit

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x32 __attribute__((ext_vector_type(32)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

struct IrParams {
    const float *x;        // [n][cin][h][w]
    const float *exp_w;    // [ce / 16][cin / 4][64]: A fragments of the expansion
    const float *exp_b;    // [ce]
    const float *dw_w;     // [ce][9]
    const float *dw_b;     // [ce]
    const float *pw_t;     // [ce][cop]: projection weights k-major, output channels padded to cop with zeros
    const float *pw_b;     // [co] or nullptr
    const float *res;      // [n][co][oh][ow] or nullptr
    float *y;              // [n][co][oh][ow]
    int n, cin, ce, h, w, oh, ow, stride, co, cop;
    int band_rows, bands, in_rows;
    int P;                 // in_rows * w: pixels of a band's input
    int xs_pitch;          // floats between the channels of Xs (P rounded up so that four rows fall into four bank groups)
    int tiles;             // ceil(P / 16)
    int vec;               // floats per load of the block input: 4 (rows a multiple of 4 floats) or 2
    int groups;            // loads per channel: P / vec
    int slots;             // loads per thread: ceil(cin * groups / 256)
    unsigned x_bytes;
    int xs_floats, patch_floats;   // LDS: Xs, then one or two patches
    Div31 div_ow, div_w, div_groups;
    Epilogue exp_ep, dw_ep, pw_ep;
};

// the CLIP of act_fast (v > lo ? v : lo, then t < hi ? t : hi; a NaN becomes lo) as one instruction: v_med3_f32 returns
// the smallest operand when one of them is a NaN, and orders -0 below +0 like the comparisons do
template <int EPI>
__device__ __forceinline__ float ir_act(float v, const Epilogue &e) {
    if constexpr (EPI == EPI_CLIP) return __builtin_amdgcn_fmed3f(v, e.clip_min, e.clip_max);
    else return apply_act(v, e);
}

extern __shared__ __attribute__((aligned(16))) float ir_lds[];

// NBUF = 2: two patches, the next chunk's expansion overlaps this chunk's depthwise stage (one barrier per chunk)
template <int EPI, int KS, int MT, int NBUF>
__global__ __launch_bounds__(256, 2) void irblock_f32_kernel(const IrParams p) {
    float *const Xs = ir_lds;
    float *const patch0 = ir_lds + p.xs_floats;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int l16 = lane & 15, lq = lane >> 4;
    const int pxh = wave & 1, kh = wave >> 1;   // which 64 pixels of the band, which 8 channels of a chunk
    const int pitch = p.w + 2, plane = p.in_rows * pitch;
    const int OHW = p.oh * p.ow;
    const int img = blockIdx.x / p.bands, band = blockIdx.x - img * p.bands;
    const int oh0 = band * p.band_rows;
    const int ih_first = oh0 * p.stride - 1;   // input row of patch row 0 (may be -1)
    const int chunks = p.ce / IR_KC;

    // the whole patch to zero once: padding columns and the rows outside the image stay that way
    for (int f = tid; f < NBUF * p.patch_floats / 4; f += 256) reinterpret_cast<float4 *>(patch0)[f] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);

    // block input: channel c, floats [0, P) of the rows ih_first .. (contiguous in memory), rows outside the image zero
    {
        const rsrc_t rx = make_rsrc(p.x, p.x_bytes);
        uint4 xr[IR_XSLOTS];
        int l_off[IR_XSLOTS];
#pragma unroll
        for (int i = 0; i < IR_XSLOTS; ++i) {
            xr[i] = make_uint4(0u, 0u, 0u, 0u);
            l_off[i] = -1;
            if (i >= p.slots) continue;   // uniform
            const int f = tid + i * 256;
            const bool live = f < p.cin * p.groups;
            const int ff = live ? f : 0;
            const int c = (int) div31((unsigned) ff, p.div_groups), g = ff - c * p.groups;
            const int ir = (int) div31((unsigned) (p.vec * g), p.div_w);   // a load lies inside one row: w is a multiple of vec
            const int ih = ih_first + ir;
            const bool in = live && (unsigned) ih < (unsigned) p.h;
            // vec * g = ir * w + column: the float offset from the start of row ih_first
            const unsigned off = in ? (unsigned) (((img * p.cin + c) * p.h + ih_first) * p.w + p.vec * g) * 4u : OOB;
            if (p.vec == 4) {   // uniform
                xr[i] = buf_load_b128(rx, off, 0);
            } else {
                const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(rx, off, 0, 0);
                xr[i] = make_uint4(t.x, t.y, 0u, 0u);
            }
            l_off[i] = live ? c * p.xs_pitch + p.vec * g : -1;
        }
#pragma unroll
        for (int i = 0; i < IR_XSLOTS; ++i)
            if (l_off[i] >= 0) {
                if (p.vec == 4) *reinterpret_cast<uint4 *>(Xs + l_off[i]) = xr[i];
                else *reinterpret_cast<uint2 *>(Xs + l_off[i]) = make_uint2(xr[i].x, xr[i].y);
            }
    }

    // this lane's pixel of the band in the depthwise stage: patch offset of the window's top-left corner (a lane past the
    // band computes on the first window and contributes a zero: no branch in the stage)
    const int q = pxh * 64 + lane;
    const bool q_ok = q < p.band_rows * p.ow;
    int win;
    {
        const int qq = q_ok ? q : 0;
        const int r = (int) div31((unsigned) qq, p.div_ow), c = qq - r * p.ow;
        win = r * p.stride * pitch + c * p.stride;
    }

    const rsrc_t rew = make_rsrc(p.exp_w, (unsigned) (p.ce * p.cin * 4));
    const rsrc_t reb = make_rsrc(p.exp_b, (unsigned) (p.ce * 4));
    const rsrc_t rpw = make_rsrc(p.pw_t, (unsigned) (p.ce * p.cop * 4));
    float aexp[KS];       // expansion weights of the chunk about to be expanded
    float eb[4];          // and its biases for this lane's four rows
    float pa[8][MT];      // projection weights of this wavefront's 8 channels of the chunk about to be projected
    auto load_exp = [&](int chunk) __attribute__((always_inline)) {
        const unsigned soff = (unsigned) (chunk * KS * 64) * 4u;
#pragma unroll
        for (int s = 0; s < KS; ++s) aexp[s] = buf_load_f32(rew, (unsigned) lane * 4u + (unsigned) s * 256u, soff);
#pragma unroll
        for (int r = 0; r < 4; ++r) eb[r] = buf_load_f32(reb, (unsigned) (4 * lq + r) * 4u, (unsigned) (chunk * IR_KC) * 4u);
    };
    auto load_proj = [&](int chunk) __attribute__((always_inline)) {
        const unsigned soff = (unsigned) ((chunk * IR_KC + kh * 8) * p.cop) * 4u;
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int a = 0; a < MT; ++a) pa[c][a] = buf_load_f32(rpw, (unsigned) (c * p.cop + a * 32 + li) * 4u, soff);
    };
    // chunk's expansion into the patch: wavefront w takes the pixel tiles w, w + 4, ..., two at a time (two independent
    // chains of MFMAs).  Where a lane's four values of tile j (one pixel, the four channels 4 (lane / 16) .. + 3, which are
    // one channel group of the patch) go is the same for every chunk: eo[j], in floats, or -1 for a pixel past the band's
    // input or in a row outside the image.
    int eo[IR_TPW];
#pragma unroll
    for (int j = 0; j < IR_TPW; ++j) {
        const int px = 16 * (wave + 4 * j) + l16;
        const int ir = (int) div31((unsigned) px, p.div_w), col = px - ir * p.w;
        const bool ok = px < p.P && (unsigned) (ih_first + ir) < (unsigned) p.h;
        eo[j] = ok ? ((lq * p.in_rows + ir) * pitch + 1 + col) * 4 : -1;
    }
    auto expand_tiles = [&](float *patch, auto j0, auto nt) __attribute__((always_inline)) {
        constexpr int NT = decltype(nt)::value, J0 = decltype(j0)::value;
        f32x4 e[NT];
        float xv[NT][KS];
#pragma unroll
        for (int u = 0; u < NT; ++u) {
            e[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            const float *xb = Xs + lq * p.xs_pitch + 16 * (wave + 4 * (J0 + u)) + l16;
#pragma unroll
            for (int s = 0; s < KS; ++s) xv[u][s] = xb[4 * s * p.xs_pitch];
        }
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int u = 0; u < NT; ++u) e[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(aexp[s], xv[u][s], e[u], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < NT; ++u) {
            if (eo[J0 + u] >= 0) {
                float4 o;
                o.x = ir_act<EPI>(__fadd_rn(e[u][0], eb[0]), p.exp_ep);
                o.y = ir_act<EPI>(__fadd_rn(e[u][1], eb[1]), p.exp_ep);
                o.z = ir_act<EPI>(__fadd_rn(e[u][2], eb[2]), p.exp_ep);
                o.w = ir_act<EPI>(__fadd_rn(e[u][3], eb[3]), p.exp_ep);
                *reinterpret_cast<float4 *>(patch + eo[J0 + u]) = o;
            }
        }
    };
    auto expand_from = [&](float *patch, auto j0) __attribute__((always_inline)) {
        constexpr int J0 = decltype(j0)::value;
        if (wave + 4 * J0 < p.tiles) {   // uniform
            if (J0 + 1 < IR_TPW && wave + 4 * (J0 + 1) < p.tiles) expand_tiles(patch, j0, std::integral_constant<int, (J0 + 1 < IR_TPW ? 2 : 1)>());
            else expand_tiles(patch, j0, std::integral_constant<int, 1>());
        }
    };
    auto expand = [&](float *patch) __attribute__((always_inline)) {
        expand_from(patch, std::integral_constant<int, 0>());
        expand_from(patch, std::integral_constant<int, 2>());
        expand_from(patch, std::integral_constant<int, 4>());
        expand_from(patch, std::integral_constant<int, 6>());
        expand_from(patch, std::integral_constant<int, 8>());
    };

    // v_mfma_f32_32x32x1_2b_f32: two 32x32 blocks (pixels 0..31 and 32..63 of the wavefront's 64), one reduction index per
    // instruction, so the depthwise channel is uniform in the wavefront (taps and bias are scalar loads) and a lane's
    // depthwise value is the B operand as it stands: A = weights[k][m = lane % 32] for both blocks, B = depthwise[k][pixel =
    // lane], D register r: block r / 16, row 8 ((r % 16) / 4) + 4 (lane / 32) + r % 4, column lane % 32.
    f32x32 acc[MT];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int r = 0; r < 32; ++r) acc[a][r] = 0.0f;
    // depthwise values of this wavefront's 8 channels for the lane's pixel, each straight into the projection's MFMAs
    auto depthwise_project = [&](int chunk, const float *patch) __attribute__((always_inline)) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            // one channel group (four channels side by side in the patch): nine 16-byte reads give the lane its window in
            // all four
            float wd[4][9], bd[4];
            float4 tv[9];
            const int g = kh * 2 + half;
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                const int c = chunk * IR_KC + g * 4 + cc;   // uniform: scalar loads
#pragma unroll
                for (int i = 0; i < 9; ++i) wd[cc][i] = p.dw_w[c * 9 + i];
                bd[cc] = p.dw_b[c];
            }
            const float4 *tp = reinterpret_cast<const float4 *>(patch) + g * plane + win;
#pragma unroll
            for (int i = 0; i < 3; ++i)
#pragma unroll
                for (int t = 0; t < 3; ++t) tv[i * 3 + t] = tp[i * pitch + t];
            __builtin_amdgcn_sched_barrier(0);   // every window is requested before the arithmetic starts
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 9; ++i) {
                    const float tap = cc == 0 ? tv[i].x : cc == 1 ? tv[i].y : cc == 2 ? tv[i].z : tv[i].w;
                    sum = __fadd_rn(sum, __fmul_rn(wd[cc][i], tap));
                }
                float v = ir_act<EPI>(__fadd_rn(sum, bd[cc]), p.dw_ep);
                v = q_ok ? v : 0.0f;
#pragma unroll
                for (int a = 0; a < MT; ++a) acc[a] = __builtin_amdgcn_mfma_f32_32x32x1f32(pa[half * 4 + cc][a], v, acc[a], 0, 0, 0);
            }
        }
    };

    load_exp(0);
    __syncthreads();   // Xs and the zeroed patches are in place
    expand(patch0);
    if (chunks > 1) load_exp(1);
    load_proj(0);
    __syncthreads();
    for (int chunk = 0; chunk < chunks; ++chunk) {
        if constexpr (NBUF == 2) {
            float *cur = patch0 + (chunk & 1) * p.patch_floats, *nxt = patch0 + ((chunk + 1) & 1) * p.patch_floats;
            if (chunk + 1 < chunks) {   // uniform
                expand(nxt);
                if (chunk + 2 < chunks) load_exp(chunk + 2);
            }
            depthwise_project(chunk, cur);
            if (chunk + 1 < chunks) load_proj(chunk + 1);
            __syncthreads();
        } else {
            depthwise_project(chunk, patch0);
            __syncthreads();   // the patch is free
            if (chunk + 1 < chunks) {   // uniform
                load_proj(chunk + 1);
                expand(patch0);
                if (chunk + 2 < chunks) load_exp(chunk + 2);
            }
            __syncthreads();
        }
    }

    // the two halves of every chunk were summed by different wavefronts: those of the upper half hand their sums over
    // through LDS (Xs and the patches are free now), the others add them and store
    float *xchg = ir_lds + (size_t) (pxh * 64 + lane) * (32 * MT + 1);   // odd pitch: no two lanes of a wavefront in one bank
    if (kh == 1) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int r = 0; r < 32; ++r) xchg[a * 32 + r] = acc[a][r];
    }
    __syncthreads();
    if (kh == 1) return;

    // store: D register r of lane l is pixel 32 (r / 16) + l % 32 of the wavefront's 64 (rows of a band are contiguous in
    // NCHW) and output channel 8 ((r % 16) / 4) + 4 (l / 32) + r % 4 of row tile a
    const rsrc_t ry = make_rsrc(p.y, RSRC_RANGE);
    const rsrc_t rr = make_rsrc(p.res, p.res ? RSRC_RANGE : 0u);
    const rsrc_t rb = make_rsrc(p.pw_b, p.pw_b ? (unsigned) (p.co * 4) : 0u);
    const bool has_bias = p.pw_b != nullptr, has_res = p.res != nullptr;
    const int band_px = min(p.band_rows, p.oh - oh0) * p.ow;
    const bool plain = !has_bias || p.pw_ep.act == NOT_ACT;   // conv.c:18-27: without a bias the activation is skipped too
    // every bias and residual value is requested before the first one is used: one memory round trip for the store
    float bias[MT][16], resv[MT][32];
    unsigned off[MT][32];
#pragma unroll
    for (int a = 0; a < MT; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) bias[a][r] = buf_load_f32(rb, (unsigned) (a * 32 + 8 * (r / 4) + 4 * lh + (r % 4)) * 4u, 0);
#pragma unroll
        for (int r = 0; r < 32; ++r) {
            const int m = a * 32 + 8 * ((r % 16) / 4) + 4 * lh + (r % 4);
            const int px = pxh * 64 + 32 * (r / 16) + li;
            const bool ok = px < band_px && m < p.co;
            off[a][r] = ok ? (unsigned) ((img * p.co + m) * OHW + oh0 * p.ow + px) * 4u : OOB;
            resv[a][r] = buf_load_f32(rr, off[a][r], 0);   // no residual: an empty buffer, zeros
        }
    }
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int r = 0; r < 32; ++r) {
            float v = __fadd_rn(acc[a][r], xchg[a * 32 + r]);
            const float vb = __fadd_rn(v, bias[a][r % 16]);
            v = has_bias ? vb : v;
            if (!plain) v = apply_act(v, p.pw_ep);
            const float vr = __fadd_rn(v, resv[a][r]);
            v = has_res ? vr : v;
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), ry, off[a][r], 0, 0);
        }
}

// expansion weights [ce][cin] -> [ce / 16][cin / 4][64] (lane l of step s: row 16 chunk + l % 16, column 4 s + l / 16),
// then the projection weights [co][ce] -> [ce][cop] k-major, zeros in the padding columns
__global__ __launch_bounds__(256) void irblock_pack_kernel(const float *w_exp, const float *w_proj, int cin, int ce, int co, int cop,
                                                           float *packed) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int n_exp = ce * cin;
    if (idx < n_exp) {
        const int l = idx & 63, s = (idx >> 6) % (cin / 4), chunk = (idx >> 6) / (cin / 4);
        packed[idx] = w_exp[(size_t) (chunk * 16 + (l & 15)) * cin + 4 * s + (l >> 4)];
    } else if (idx < n_exp + ce * cop) {
        const int j = idx - n_exp;
        const int k = j / cop, m = j - k * cop;
        packed[idx] = m < co ? w_proj[(size_t) m * ce + k] : 0.0f;
    }
}

int irblock_pack_launch(const float *w_exp, const float *w_proj, int cin, int ce, int co, float *packed, hipStream_t stream) {
    const int cop = (co + 31) / 32 * 32;
    const int total = ce * cin + ce * cop;
    hipLaunchKernelGGL(irblock_pack_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, stream, w_exp, w_proj, cin, ce, co, cop, packed);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

static int ir_xs_pitch(int P) {
    int pp = (P + 15) / 16 * 16;
    if (pp % 32 == 0) pp += 16;   // rows k, k + 1, k + 2, k + 3 of an MFMA's B operand in four different groups of 16 banks
    return pp;
}

// the band of output rows one workgroup takes, or 0 when the kernel does not fit the shape
int irblock_band_rows(const onhip_conv_desc_t &dw, int OH, int OW, int cin) {
    if (OW > IR_BN || dw.w % 2) return 0;
    const int vec = dw.w % 4 ? 2 : 4;
    int rows = IR_BN / OW;
    rows = rows > OH ? OH : rows;
    if (const char *env = getenv("ONHIP_IR_ROWS")) {   // tuning hook: at most this many output rows per band
        const int r = atoi(env);
        if (r >= 1 && r < rows) rows = r;
    }
    // the tallest band that fits and still leaves one workgroup per compute unit; failing that, the tallest that fits
    int tallest = 0;
    for (; rows >= 1; --rows) {
        const int in_rows = (rows - 1) * dw.stride_h + 3;
        const int P = in_rows * dw.w;
        const long long slots = ((long long) cin * (P / vec) + 255) / 256;
        const long long lds = ((long long) cin * ir_xs_pitch(P) + 4 + (long long) IR_KC * in_rows * (dw.w + 2) + 4) * 4;
        if (lds > IR_LDS_HALF || slots > IR_XSLOTS || (P + 15) / 16 > 4 * IR_TPW) continue;
        if (!tallest) tallest = rows;
        if ((long long) dw.n * ((OH + rows - 1) / rows) >= 256) return rows;
    }
    return tallest;
}

template <int EPI, int KS, int MT, int NBUF>
static int irblock_launch_one(const IrParams &p, size_t lds_bytes, hipStream_t stream) {
    // more than 64 KiB of dynamic LDS has to be asked for once per kernel
    static std::atomic<size_t> allowed{64 * 1024};
    if (lds_bytes > allowed.load()) {
        ONHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(irblock_f32_kernel<EPI, KS, MT, NBUF>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, IR_LDS_HALF));
        allowed.store(IR_LDS_HALF);
    }
    hipLaunchKernelGGL((irblock_f32_kernel<EPI, KS, MT, NBUF>), dim3((unsigned) (p.n * p.bands)), dim3(256), lds_bytes, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

template <int EPI, int KS>
static int irblock_launch_ks(const IrParams &p, hipStream_t stream) {
    const int mt = p.cop / 32;
    if (mt > 2) return set_error(ONHIP_ERR_ARG, "inverted-residual block: more than 64 output channels");
    // LDS: Xs, the patch(es), and at least room for the exchange of partial sums at the end of a band
    const size_t xchg = (size_t) 128 * (32 * mt + 1);
    const size_t two = (size_t) p.xs_floats + 2 * (size_t) p.patch_floats, one = (size_t) p.xs_floats + p.patch_floats;
    const bool dbl = two * 4 <= (size_t) IR_LDS_HALF;
    size_t floats = dbl ? two : one;
    floats = floats < xchg ? xchg : floats;
    if (floats * 4 > (size_t) IR_LDS_HALF) return set_error(ONHIP_ERR_ARG, "inverted-residual block: %zu bytes of LDS", floats * 4);
    if (mt == 1) return dbl ? irblock_launch_one<EPI, KS, 1, 2>(p, floats * 4, stream) : irblock_launch_one<EPI, KS, 1, 1>(p, floats * 4, stream);
    return dbl ? irblock_launch_one<EPI, KS, 2, 2>(p, floats * 4, stream) : irblock_launch_one<EPI, KS, 2, 1>(p, floats * 4, stream);
}

template <int EPI>
static int irblock_launch_epi(const IrParams &p, hipStream_t stream) {
    switch (p.cin / 4) {
        case 4: return irblock_launch_ks<EPI, 4>(p, stream);
        case 6: return irblock_launch_ks<EPI, 6>(p, stream);
        case 8: return irblock_launch_ks<EPI, 8>(p, stream);
        case 16: return irblock_launch_ks<EPI, 16>(p, stream);
        default: return set_error(ONHIP_ERR_ARG, "inverted-residual block: %d input channels (16, 24, 32 and 64 are built)", p.cin);
    }
}

bool irblock_cin_ok(int cin) { return cin == 16 || cin == 24 || cin == 32 || cin == 64; }

// ex: the 1x1 expansion, dw: the depthwise 3x3 on its result, pw: the 1x1 projection; shapes are checked by the caller
// (irblock_band_rows != 0 and irblock_cin_ok included).  The activations of ex and dw go through one template
// parameter: CLIP when both are CLIP, the general form otherwise.
int irblock_f32_launch(const onhip_conv_desc_t &ex, const onhip_conv_desc_t &dw, const onhip_conv_desc_t &pw, int OH, int OW, const float *x,
                       const float *packed, const float *exp_b, const float *dw_w, const float *dw_b, const float *pw_b, const float *res,
                       const Epilogue &exp_ep, const Epilogue &dw_ep, const Epilogue &pw_ep, float *y, hipStream_t stream) {
    IrParams p;
    memset(&p, 0, sizeof(p));
    p.cop = (pw.cout + 31) / 32 * 32;
    p.x = x; p.exp_w = packed; p.exp_b = exp_b; p.dw_w = dw_w; p.dw_b = dw_b; p.pw_t = packed + (size_t) ex.cout * ex.cin;
    p.pw_b = pw_b; p.res = res; p.y = y;
    p.n = dw.n; p.cin = ex.cin; p.ce = dw.cin; p.h = dw.h; p.w = dw.w; p.oh = OH; p.ow = OW; p.stride = dw.stride_h;
    p.co = pw.cout;
    p.band_rows = irblock_band_rows(dw, OH, OW, ex.cin);
    if (p.band_rows < 1) return set_error(ONHIP_ERR_ARG, "inverted-residual block: no band of rows fits the kernel");
    p.bands = (OH + p.band_rows - 1) / p.band_rows;
    p.in_rows = (p.band_rows - 1) * p.stride + 3;
    p.P = p.in_rows * p.w;
    p.xs_pitch = ir_xs_pitch(p.P);
    p.tiles = (p.P + 15) / 16;
    p.vec = p.w % 4 ? 2 : 4;
    p.groups = p.P / p.vec;
    p.slots = (p.cin * p.groups + 255) / 256;
    p.x_bytes = (unsigned) ((size_t) ex.n * ex.cin * ex.h * ex.w * 4);
    p.div_ow = make_div31((unsigned) OW);
    p.div_w = make_div31((unsigned) p.w);
    p.div_groups = make_div31((unsigned) p.groups);
    p.xs_floats = (p.cin * p.xs_pitch + 3) / 4 * 4;
    p.patch_floats = (IR_KC * p.in_rows * (p.w + 2) + 3) / 4 * 4;
    p.exp_ep = exp_ep;
    p.dw_ep = dw_ep;
    p.pw_ep = pw_ep;
    if (exp_ep.act == CLIP && dw_ep.act == CLIP)
        return irblock_launch_epi<EPI_CLIP>(p, stream);
    return irblock_launch_epi<EPI_GENERIC>(p, stream);
}

}  // namespace onhip
