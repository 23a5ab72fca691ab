// Two kernels for the convolutions of an int8 NHWC chain (int8 in and out) that have few channels: i8patch_kernel, 3x3
// with stride 1 and pads 1, 32 or 64 bytes per input pixel, at most 64 output channels, described here; and
// i8direct_kernel further down (3x3 of any stride with 16 or 32 bytes per pixel, 1x1 with 64 to 128).  The implicit-GEMM
// kernels read every input pixel nine times, once per filter tap, through L2 into LDS, and pay a tile's whole set-up and
// store for two or three K stages; with so few channels that, not the matrix cores, sets their time.  Here
//
//   * a persistent workgroup walks bands of whole output rows of the batch; the band's input rows plus halo,
//     (rows + 2) x (w + 2) pixels with zeros outside the image, are loaded ONCE into an LDS patch (NHWC rows are
//     contiguous: plain 16-byte loads), the next band's into registers while this one is multiplied and stored, a block
//     of 128 or 256 pixels per pass (rows and block chosen so that the last block of a band is as full as possible);
//   * the weights of a wavefront's 32-row tile (at most 32 x 9 x 64 bytes) sit in its registers for the life of the
//     workgroup: lane (row lane % 32, half lane / 32) holds bytes 32 s + 16 half .. + 15 of every (tap, step s);
//   * v_mfma_i32_32x32x32_i8: B = 16 bytes of the pixel under tap (i, j), read from the patch at a per-lane base (computed
//     once per workgroup) plus a compile-time offset, no address arithmetic in the loop; the four wavefronts stand side
//     by side over the band's pixels (WM = 1) or two by two over row tiles and pixels (WM = 2, up to 64 channels);
//   * the store is the int8 NHWC store of the implicit-GEMM kernels (write_tile_nhwc_s8: de-quantisation, bias, activation
//     or quantised table, re-quantisation, transposition through LDS, 16-byte stores), so the results are the same bytes.
// Arithmetic: device/x86/Conv/conv.c:961-973 (the input quantiser, here the producer's), :1024-1056 (int32 sums, then
// the three separately rounded fp32 operations) as everywhere in the int8 path; the int32 sums do not depend on the order.
#include <string.h>

#include <atomic>

#include "igemm_kernel.hpp"

namespace onhip {

constexpr int P8_SLOTS = 8;   // 16-byte patch loads per thread, at most

struct PatchGeom {
    int passes;          // blocks of BN pixels a band is multiplied and stored in
    int rows;            // output rows of a band
    int bands;           // bands per image
    int total;           // bands of the batch
    int prow_px;         // pixels of a patch row: w + 2
    int patch_vecs;      // 16-byte pieces of a patch: (rows + 2) * prow_px * CB / 16
    int slots;           // ceil(patch_vecs / 256)
    Div31 div_ow, div_rowvecs, div_parts;
};

// Which items of 0 .. total - 1 a persistent workgroup takes: workgroups are dealt to the 8 XCDs in turn, each with an L2 of
// its own, so XCD x gets the x-th contiguous eighth of the items and its workgroups walk that eighth together; items next
// to each other (bands and blocks of neighbouring image rows, which share input rows) then meet in one L2 at about the
// same time.  With a grid that is not a multiple of 8: plain striding.
struct ItemWalk { int first, end, step; };
__device__ __forceinline__ ItemWalk xcd_walk(int total) {
    const int g = (int) gridDim.x;
    if (g % 8 != 0) return {(int) blockIdx.x, total, g};
    const int xcd = (int) blockIdx.x & 7, chunk = (total + 7) >> 3;
    const int lo = xcd * chunk, hi = min(total, lo + chunk);
    return {lo + ((int) blockIdx.x >> 3), hi, g >> 3};
}

// WM = 1: the four wavefronts side by side over the pixels (up to 32 output channels); WM = 2: two rows of two (up to 64),
// so a wavefront holds the weights of one 32-row tile only.  TN: 32-pixel tiles per wavefront.
template <int CB, int WM, int TN>
__global__ __launch_bounds__(256, (CB == 32 && TN == 1 ? 3 : 2)) void i8patch_kernel(const IgemmParams p, const PatchGeom g) {
    constexpr int S = CB / 32, PARTS = CB / 16, WN = 4 / WM, BM = 32 * WM, BN = 32 * TN * WN;
    constexpr int STAGE = BN * (BM + 16);
    extern __shared__ __attribute__((aligned(16))) unsigned char p8_lds[];
    unsigned char *const stage = p8_lds;                                   // the store's staging area, then the quantised table
    float *const rows = reinterpret_cast<float *>(p8_lds + STAGE + 8192);   // per-row constants of the store
    unsigned char *const patch = p8_lds + STAGE + 8192 + 2 * BM * 4;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    const int W = p.W, H = p.H;
    const int band_px = g.rows * W;

    // the weights of this wavefront's row tile: [m][tap][CB] bytes, the lane's 16 of every (tap, step)
    i32x4 areg[9][S];
    {
        const rsrc_t ra = make_rsrc(p.A, (unsigned) p.a_slice_bytes);
        const int m = 32 * wm + li;
#pragma unroll
        for (int t = 0; t < 9; ++t)
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const uint4 q = buf_load_b128(ra, m < p.M ? (unsigned) (m * p.lda + t * CB + 32 * s + 16 * lh) : OOB, 0);
                areg[t][s] = i32x4{(int) q.x, (int) q.y, (int) q.z, (int) q.w};
            }
    }
    // the store's per-row constants: weight_aux / 127 (conv.c:1049-1056) and the int32 bias as a float; and, once for the
    // life of the workgroup, the quantised activation table where the store looks for it
    if (tid < BM) {
        const rsrc_t raux = make_rsrc(p.weight_aux, (unsigned) (p.M * 4));
        const rsrc_t rb32 = make_rsrc(p.bias32, p.bias32 ? (unsigned) (p.M * 4) : 0u);
        rows[tid] = __fdiv_rn(buf_load_f32(raux, (unsigned) tid * 4u, 0), 127.0f);
        rows[BM + tid] = (float) (int) __builtin_amdgcn_raw_buffer_load_b32(rb32, (unsigned) tid * 4u, 0, 0);
    }
    const bool table = (p.ep.act == SILU || p.ep.act == ONHIP_ACT_GELU_LUT) && p.ep.qlut != nullptr;
    if (table) {
        const uint4 *src = reinterpret_cast<const uint4 *>(p.ep.qlut);
#pragma unroll
        for (int i = 0; i < 8192 / 16 / 256; ++i) reinterpret_cast<uint4 *>(stage + STAGE)[tid + i * 256] = src[tid + i * 256];
        if (tid == 0) stage[STAGE - 1] = 0;   // the store's "below the table" entry, in padding that nothing else touches
    }

    // patch loads: piece f = (patch row, pixel, part) in that order; where it comes from relative to the band's first
    // input row, where it goes, and whether its column lies inside the image are the same for every band
    int l_off[P8_SLOTS], g_off[P8_SLOTS], prow[P8_SLOTS];
#pragma unroll
    for (int i = 0; i < P8_SLOTS; ++i) {
        const int f = tid + i * 256;
        const bool live = i < g.slots && f < g.patch_vecs;
        const int ff = live ? f : 0;
        const int r = (int) div31((unsigned) ff, g.div_rowvecs), rem = ff - r * g.prow_px * PARTS;
        const int pc = (int) div31((unsigned) rem, g.div_parts), part = rem - pc * PARTS;
        const bool col_ok = pc >= 1 && pc <= W;
        prow[i] = live && col_ok ? r : -1000000;                  // a row index no band makes valid
        g_off[i] = (r * W + pc - 1) * CB + part * 16;              // bytes from the start of the input row above the band
        l_off[i] = live ? ff * 16 : -1;
    }
    const int row_bytes = g.prow_px * CB;

    const rsrc_t rx = make_rsrc(p.B, (unsigned) p.b_slice_bytes);
    uint4 xr[P8_SLOTS];
    auto issue = [&](int band) __attribute__((always_inline)) {
        const int img = band / g.bands, oy0 = (band - img * g.bands) * g.rows;
        const int base = (img * H + oy0 - 1) * W * CB;             // input row oy0 - 1, column 0 (may lie before the tensor)
#pragma unroll
        for (int i = 0; i < P8_SLOTS; ++i) {
            const int iy = oy0 - 1 + prow[i];
            const bool ok = (unsigned) iy < (unsigned) H;          // false for every piece outside the image
            xr[i] = buf_load_b128(rx, ok ? (unsigned) (base + g_off[i]) : OOB, 0);
        }
    };

    IgemmParams ps = p;   // the store's view of the problem: the band's pixels only
    const ItemWalk walk = xcd_walk(g.total);
    int band = walk.first;
    if (band < walk.end) issue(band);
    for (; band < walk.end; band += walk.step) {
        __syncthreads();   // everybody is done with the previous band's patch and staging area
#pragma unroll
        for (int i = 0; i < P8_SLOTS; ++i)
            if (l_off[i] >= 0) *reinterpret_cast<uint4 *>(patch + l_off[i]) = xr[i];
        __syncthreads();
        if (band + walk.step < walk.end) issue(band + walk.step);   // uniform

        const int img = band / g.bands, oy0 = (band - img * g.bands) * g.rows;
        const int n_band = (img * H + oy0) * W;
        ps.N = n_band + min(g.rows, H - oy0) * W;
        for (int pass = 0; pass < g.passes; ++pass) {
            if (n_band + pass * BN >= ps.N) break;   // uniform: a ragged last band ends early
            if (pass > 0) __syncthreads();           // the previous pass's store has left the staging area
            // this lane's pixels in the MFMAs: byte offset in the patch of the window's top-left pixel, per pixel tile
            int boff[TN];
            bool tile_on[TN];
#pragma unroll
            for (int b = 0; b < TN; ++b) {
                const int q0 = pass * BN + 32 * (TN * wn + b);
                tile_on[b] = q0 < band_px;                                // uniform
                const int q = q0 + li < band_px ? q0 + li : 0;
                const int r = (int) div31((unsigned) q, g.div_ow), c = q - r * W;
                boff[b] = (r * g.prow_px + c) * CB + 16 * lh;
            }
            i32x16 acc[1][TN];
#pragma unroll
            for (int b = 0; b < TN; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[0][b][r] = 0;
#pragma unroll
            for (int b = 0; b < TN; ++b) {
                if (!tile_on[b]) continue;
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    const unsigned char *prow_base = patch + boff[b] + i * row_bytes;
                    i32x4 bv[3][S];
#pragma unroll
                    for (int j = 0; j < 3; ++j)
#pragma unroll
                        for (int s = 0; s < S; ++s) bv[j][s] = *reinterpret_cast<const i32x4 *>(prow_base + j * CB + 32 * s);
#pragma unroll
                    for (int j = 0; j < 3; ++j)
#pragma unroll
                        for (int s = 0; s < S; ++s)
                            acc[0][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[3 * i + j][s], bv[j][s], acc[0][b], 0, 0, 0);
                }
            }
            const int n0 = n_band + pass * BN;
            const int m_wave = 32 * wm, n_wave = n0 + 32 * TN * wn;
            switch (p.ep.act) {
                case NOT_ACT:
                case RELU6: write_tile_nhwc_s8<EPI_NONE, BM, BN, 1, TN, true>(ps, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
                case RELU: write_tile_nhwc_s8<EPI_RELU, BM, BN, 1, TN, true>(ps, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
                case CLIP: write_tile_nhwc_s8<EPI_CLIP, BM, BN, 1, TN, true>(ps, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
                case SILU:
                case ONHIP_ACT_GELU_LUT: write_tile_nhwc_s8<EPI_LUT, BM, BN, 1, TN, true>(ps, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
                default: write_tile_nhwc_s8<EPI_GENERIC, BM, BN, 1, TN, true>(ps, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
            }
        }
    }
}

// The same convolution, and 1x1 convolutions, without the patch: every lane loads the 16 bytes of its pixel under each filter tap straight from
// global memory (zeros outside the image from the buffer descriptor's range check).  For strides above 1, where windows
// share few pixels, and for 16 bytes per pixel (up to 16 input channels: a network's first layer), where two taps fill
// one MFMA step: K index 32 k + 16 half of step k is tap (32 k + 16 half) / CB, byte (32 k + 16 half) % CB of the pixel,
// and the packed weights ([m][tap][CB]) are read at that same index.  A persistent workgroup walks blocks of BN output
// pixels of the whole batch; the next block's loads are in flight while this one is stored.
template <int CB, int TAPS, int KW, int WM, int TM, int TN, int OCC>
__global__ __launch_bounds__(256, OCC) void i8direct_kernel(const IgemmParams p, const int blocks) {
    constexpr int NK = (TAPS * CB + 31) / 32, WN = 4 / WM, BM = 32 * TM * WM, BN = 32 * TN * WN;
    constexpr int STAGE = BN * (BM + 16);
    __shared__ __attribute__((aligned(16))) unsigned char lds[STAGE + 8192 + 2 * BM * 4];
    unsigned char *const stage = lds;
    float *const rows = reinterpret_cast<float *>(lds + STAGE + 8192);

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    i32x4 areg[TM][NK];
    {
        const rsrc_t ra = make_rsrc(p.A, (unsigned) p.a_slice_bytes);
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const int m = 32 * (TM * wm + a) + li;
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int kk = 32 * k + 16 * lh;
                const uint4 q = buf_load_b128(ra, m < p.M && kk < TAPS * CB ? (unsigned) (m * p.lda + kk) : OOB, 0);
                areg[a][k] = i32x4{(int) q.x, (int) q.y, (int) q.z, (int) q.w};
            }
        }
    }
    if (tid < BM) {
        const rsrc_t raux = make_rsrc(p.weight_aux, (unsigned) (p.M * 4));
        const rsrc_t rb32 = make_rsrc(p.bias32, p.bias32 ? (unsigned) (p.M * 4) : 0u);
        rows[tid] = __fdiv_rn(buf_load_f32(raux, (unsigned) tid * 4u, 0), 127.0f);
        rows[BM + tid] = (float) (int) __builtin_amdgcn_raw_buffer_load_b32(rb32, (unsigned) tid * 4u, 0, 0);
    }
    const bool table = (p.ep.act == SILU || p.ep.act == ONHIP_ACT_GELU_LUT) && p.ep.qlut != nullptr;
    if (table) {
        const uint4 *src = reinterpret_cast<const uint4 *>(p.ep.qlut);
#pragma unroll
        for (int i = 0; i < 8192 / 16 / 256; ++i) reinterpret_cast<uint4 *>(stage + STAGE)[tid + i * 256] = src[tid + i * 256];
        if (tid == 0) stage[STAGE - 1] = 0;   // the store's "below the table" entry, in padding that nothing else touches
    }

    // where step k's bytes lie relative to the window's first pixel: the same for every block.  Filters of many taps
    // (MANY: a 7x7 first layer, 25 steps) work the three numbers out per load instead of holding them, and load a block's
    // pixels when its turn comes rather than a block ahead: the registers go to the weights.
    constexpr bool MANY = NK > 12;
    int tap_i[MANY ? 1 : NK], tap_j[MANY ? 1 : NK], tap_byte[MANY ? 1 : NK];
    auto tap_of = [&](int k, int &ti, int &tj, int &tb) __attribute__((always_inline)) {
        const int kk = 32 * k + 16 * lh, tap = kk / CB;
        const int i = tap / KW;
        ti = tap < TAPS ? i : 1 << 28;              // past the last tap: outside any image
        tj = tap - KW * i;
        tb = kk % CB;
    };
    if constexpr (!MANY) {
#pragma unroll
        for (int k = 0; k < NK; ++k) tap_of(k, tap_i[k], tap_j[k], tap_byte[k]);
    }
    const rsrc_t rx = make_rsrc(p.B, (unsigned) p.b_slice_bytes);
    uint4 bx[TN][NK];
    auto issue = [&](int blk) __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int q = blk * BN + 32 * (TN * wn + b) + li;
            const bool live = q < p.N;
            const int qq = live ? q : 0;
            const int img = (int) div31((unsigned) qq, p.div_ohw), rem = qq - img * p.OHW;
            const int oy = (int) div31((unsigned) rem, p.div_ow), ox = rem - oy * p.OW;
            const int iy0 = live ? oy * p.sh - p.pt : -(1 << 29), ix0 = ox * p.sw - p.pl;
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                int ti, tj, tb;
                if constexpr (MANY) tap_of(k, ti, tj, tb);
                else { ti = tap_i[k]; tj = tap_j[k]; tb = tap_byte[k]; }
                const int iy = iy0 + ti, ix = ix0 + tj;
                const bool ok = (unsigned) iy < (unsigned) p.H && (unsigned) ix < (unsigned) p.W;
                bx[b][k] = buf_load_b128(rx, ok ? (unsigned) (((img * p.H + iy) * p.W + ix) * CB + tb) : OOB, 0);
            }
        }
    };

    const ItemWalk walk = xcd_walk(blocks);
    int blk = walk.first;
    if (!MANY && blk < walk.end) issue(blk);
    for (; blk < walk.end; blk += walk.step) {
        if constexpr (MANY) issue(blk);
        i32x16 acc[TM][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b) {
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;
#pragma unroll
                for (int k = 0; k < NK; ++k) {
                    const i32x4 bv = i32x4{(int) bx[b][k].x, (int) bx[b][k].y, (int) bx[b][k].z, (int) bx[b][k].w};
                    acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[a][k], bv, acc[a][b], 0, 0, 0);
                }
            }
        if (!MANY && blk + walk.step < walk.end) issue(blk + walk.step);   // uniform
        __syncthreads();   // the previous block's store has left the staging area (and, the first time, the table is there)
        const int n0 = blk * BN, m_wave = 32 * TM * wm, n_wave = n0 + 32 * TN * wn;
        switch (p.ep.act) {
            case NOT_ACT:
            case RELU6: write_tile_nhwc_s8<EPI_NONE, BM, BN, TM, TN, true>(p, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
            case RELU: write_tile_nhwc_s8<EPI_RELU, BM, BN, TM, TN, true>(p, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
            case CLIP: write_tile_nhwc_s8<EPI_CLIP, BM, BN, TM, TN, true>(p, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
            case SILU:
            case ONHIP_ACT_GELU_LUT: write_tile_nhwc_s8<EPI_LUT, BM, BN, TM, TN, true>(p, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
            default: write_tile_nhwc_s8<EPI_GENERIC, BM, BN, TM, TN, true>(p, acc, stage, 0, n0, m_wave, n_wave, li, lh, tid, rows, true); break;
        }
    }
}

// the int8 NHWC chain form of a 3x3 convolution of any stride and padding with 16 or 32 bytes per input pixel and at most
// 64 output channels; of a 7x7 convolution with 16 bytes per pixel and at most 64; of a 1x1 convolution with 64, 96 or 128 bytes per pixel and at most 64 output channels (with two
// row tiles per wavefront, up to 128 channels, it was measured level with the implicit-GEMM kernels or behind them)
bool i8direct_ok(const IgemmParams &p) {
    if (!p.out_s8 || p.out_mode != OUT_PLAIN || p.c_stride_m != 1 || p.acc_out) return false;
    if (p.lda != p.khkw * p.pix_stride || p.b_slice_bytes >= (1LL << 31) - 64) return false;
    if (p.kh == 3 && p.kw == 3) return p.M <= 64 && (p.pix_stride == 16 || p.pix_stride == 32);
    if (p.kh == 7 && p.kw == 7) return p.M <= 64 && p.pix_stride == 16;   // a first layer: up to 16 input channels
    if (p.kh == 1 && p.kw == 1) return p.M <= 64 && (p.pix_stride == 64 || p.pix_stride == 96 || p.pix_stride == 128);
    return false;
}

template <int CB, int TAPS, int KW, int WM, int TM, int TN, int OCC>
static int i8direct_launch_one(IgemmParams p, hipStream_t stream) {
    constexpr int BN = 32 * TN * (4 / WM);
    const int blocks = (p.N + BN - 1) / BN;
    p.div_ohw = make_div31((unsigned) p.OHW);
    p.div_ow = make_div31((unsigned) p.OW);
    const int grid = blocks < 256 * OCC ? (blocks + 7) / 8 * 8 : 256 * OCC;   // OCC workgroups per compute unit; a multiple of 8 (xcd_walk)
    hipLaunchKernelGGL((i8direct_kernel<CB, TAPS, KW, WM, TM, TN, OCC>), dim3((unsigned) grid), dim3(256), 0, stream, p, blocks);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int i8direct_launch(const IgemmParams &p, hipStream_t stream) {
    if (p.kh == 7) return p.M <= 32 ? i8direct_launch_one<16, 49, 7, 1, 1, 1, 2>(p, stream) : i8direct_launch_one<16, 49, 7, 2, 1, 1, 2>(p, stream);
    if (p.kh == 1) {   // as many workgroups per compute unit as the registers allow: 64 -> 64 on 160 x 160, 28.0 -> 22.4 us with 4 against 2
        if (p.pix_stride == 64) return i8direct_launch_one<64, 1, 1, 2, 1, 2, 4>(p, stream);
        if (p.pix_stride == 96) return i8direct_launch_one<96, 1, 1, 2, 1, 2, 3>(p, stream);
        return i8direct_launch_one<128, 1, 1, 2, 1, 2, 3>(p, stream);
    }
    // measured on a first layer (3 -> 32 channels, stride 2) and the layer after it (32 -> 64): three workgroups per
    // compute unit help the former, whose time is the store's arithmetic; smaller or larger blocks help neither
    if (p.pix_stride == 16) return p.M <= 32 ? i8direct_launch_one<16, 9, 3, 1, 1, 2, 3>(p, stream) : i8direct_launch_one<16, 9, 3, 2, 1, 2, 2>(p, stream);
    return p.M <= 32 ? i8direct_launch_one<32, 9, 3, 1, 1, 2, 2>(p, stream) : i8direct_launch_one<32, 9, 3, 2, 1, 2, 2>(p, stream);
}

static int i8patch_rows(const IgemmParams &p, int *big);

// the problems this kernel takes: the int8 NHWC chain form of a 3x3 convolution, stride 1, pads 1, 32 or 64 bytes per
// input pixel, at most 64 output channels
bool i8patch_ok(const IgemmParams &p, bool any_shape) {
    if (!p.out_s8 || p.out_mode != OUT_PLAIN || p.c_stride_m != 1 || p.acc_out) return false;
    if (p.kh != 3 || p.kw != 3 || p.sh != 1 || p.sw != 1 || p.pt != 1 || p.pl != 1) return false;
    if (p.pix_stride != 32 && p.pix_stride != 64) return false;
    if (p.M > 64 || p.OW != p.W || p.OHW != p.HW || p.W < 4) return false;
    if (p.lda != 9 * p.pix_stride) return false;
    int big = 0;
    const int rows = i8patch_rows(p, &big);
    if (rows < 1) return false;
    if (any_shape) return true;
    // measured against the implicit-GEMM kernels (batch 16): ahead with 32 bytes per pixel and one row tile (160 x 160:
    // 22.9 against 36.3 us) and with 64 bytes and two (80 x 80: 16.0 against 17.0), the other two combinations not
    // measured; behind wherever the batch has fewer bands than the chip has compute units (40 x 40: 16 against 9 us)
    const bool measured = (p.pix_stride == 32 && p.M <= 32) || (p.pix_stride == 64 && p.M > 32);
    const long long bands = (long long) (p.N / p.OHW) * ((p.H + rows - 1) / rows);
    return measured && bands >= 256;
}

template <int CB, int WM, int TN>
static int i8patch_launch_one(const IgemmParams &p, PatchGeom g, hipStream_t stream) {
    constexpr int BM = 32 * WM, BN = 32 * TN * (4 / WM);
    const size_t lds = (size_t) BN * (BM + 16) + 8192 + 2 * BM * 4 + (size_t) g.patch_vecs * 16;
    if (lds > 80 * 1024) return set_error(ONHIP_ERR_ARG, "int8 patch kernel: %zu bytes of LDS", lds);
    static std::atomic<size_t> allowed{64 * 1024};
    if (lds > allowed.load()) {
        ONHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(i8patch_kernel<CB, WM, TN>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            80 * 1024));
        allowed.store(80 * 1024);
    }
    int grid = CB == 32 && TN == 1 ? 768 : 512;   // three or two workgroups per compute unit; a multiple of 8 (xcd_walk)
    grid = grid > g.total ? (g.total + 7) / 8 * 8 : grid;
    hipLaunchKernelGGL((i8patch_kernel<CB, WM, TN>), dim3((unsigned) grid), dim3(256), lds, stream, p, g);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// whole rows per band and the block (128 or 256 pixels) the band is multiplied and stored in, pass after pass: the pair
// whose last block is fullest (a store costs the same for an empty pixel), the larger block unless it is 7 % emptier
// (measured: three rows of 160 pixels in two blocks of 256 beat four rows in five blocks of 128, 22.9 against 24.3 us,
// with two workgroups per compute unit each) -- except with 32 bytes per pixel and one row tile, where the 128-pixel
// variant fits three workgroups per compute unit and wins (21.7 us) --, more rows per band (fewer halo rows) between
// equals; within the patch loads a thread has registers for and the LDS two workgroups share.  0: no row fits
static int i8patch_rows(const IgemmParams &p, int *big) {
    const int W = p.W, H = p.H, cb = p.pix_stride, bm = p.M > 32 ? 64 : 32;
    int best_rows = 0;
    double best = 0.0;
    for (int bn = 128; bn <= 256; bn += 128) {
        if (bn == 256 && cb == 64 && bm == 64) continue;   // four pixel tiles per wavefront and 72 registers of weights do not fit
        for (int rows = 1; rows <= H && rows <= 32; ++rows) {
            const long long vecs = (long long) (rows + 2) * (W + 2) * cb / 16;
            if (vecs > 256LL * P8_SLOTS || (long long) bn * (bm + 16) + 8192 + 2 * bm * 4 + vecs * 16 > 80 * 1024) break;
            const int passes = (rows * W + bn - 1) / bn;
            const double score = (double) rows * W / ((double) passes * bn) + 0.001 * rows + (bn == 256 && !(cb == 32 && bm == 32) ? 0.07 : 0.0);
            if (score > best) { best = score; best_rows = rows; *big = bn == 256; }
        }
    }
    return best_rows;
}

int i8patch_launch(const IgemmParams &p, hipStream_t stream) {
    const int W = p.W, H = p.H, cb = p.pix_stride, images = p.N / p.OHW;
    PatchGeom g;
    memset(&g, 0, sizeof(g));
    int big = 0;
    g.rows = i8patch_rows(p, &big);
    if (!g.rows) return set_error(ONHIP_ERR_ARG, "int8 patch kernel: rows of %d pixels do not fit", W);
    g.passes = (g.rows * W + (big ? 256 : 128) - 1) / (big ? 256 : 128);
    g.bands = (H + g.rows - 1) / g.rows;
    g.total = images * g.bands;
    g.prow_px = W + 2;
    g.patch_vecs = (g.rows + 2) * g.prow_px * cb / 16;
    g.slots = (g.patch_vecs + 255) / 256;
    g.div_ow = make_div31((unsigned) W);
    g.div_rowvecs = make_div31((unsigned) (g.prow_px * cb / 16));
    g.div_parts = make_div31((unsigned) (cb / 16));
    if (p.M <= 32) {   // four wavefronts side by side: 128 pixels are one tile each, 256 two
        if (cb == 32) return big ? i8patch_launch_one<32, 1, 2>(p, g, stream) : i8patch_launch_one<32, 1, 1>(p, g, stream);
        return big ? i8patch_launch_one<64, 1, 2>(p, g, stream) : i8patch_launch_one<64, 1, 1>(p, g, stream);
    }
    if (cb == 32) return big ? i8patch_launch_one<32, 2, 4>(p, g, stream) : i8patch_launch_one<32, 2, 2>(p, g, stream);
    return i8patch_launch_one<64, 2, 2>(p, g, stream);
}

}  // namespace onhip
