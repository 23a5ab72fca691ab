// Implicit-GEMM kernel family for gfx950 (MI355X): C[M, N] = A[M, K] * B[K, N] on 32x32 MFMA tiles
// with the whole epilogue (bias, activation, W8A32 de-quantisation, re-quantisation) fused in
// registers.
//
// Work decomposition
//   * one workgroup = 256 threads = 4 wavefronts (64 lanes) computes a BM x BN tile of C; each
//     wavefront owns a (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA blocks held in accumulators;
//   * K is walked in tiles of 4 "units"; a unit is 16 bytes of one A row / one B column along K
//     (4 fp32, 8 bf16/fp16 or 16 int8 values), which is exactly what one lane feeds to the MFMA
//     instructions v_mfma_f32_32x32x2_f32 (x4), v_mfma_f32_32x32x16_{bf16,f16},
//     v_mfma_i32_32x32x32_i8;
//   * LDS holds, double-buffered, A as [unit][row][16 B] and B as [unit][column][16 B]: a half
//     wavefront reads 32 consecutive 16-byte slots (conflict-free ds_read_b128), lanes 0-31 take the
//     even unit and lanes 32-63 the odd unit of an MFMA step;
//   * global loads for tile t+1 are issued before the MFMAs of tile t and written to the other LDS
//     buffer afterwards: one barrier per K tile.
//
// B never exists in memory.  BL_GATHER builds it element by element from NCHW activations
// (implicit im2col), BL_TAPC does the same against tap-major packed weights (one filter tap per
// unit), BL_PLAIN reads a 1x1 convolution's input or a row-major [K, N] matrix; in all three lanes
// run along N so every load instruction is a coalesced run of pixels.  BL_KVEC reads 16-byte
// vectors along K from NHWC int8 activations (K ordered tap-major, channel-minor), the units of a
// column on neighbouring lanes.
//
// Every global access is a raw buffer instruction: the per-lane byte offset (the pixel, fixed for
// the whole K loop) goes in the vector offset, the wavefront-uniform part (channel, filter tap,
// K tile) in the scalar offset, so a gathered element costs a handful of scalar operations and a
// compare/select instead of 64-bit address arithmetic.  Padding, ragged tile edges and the K tail
// are handled by pointing the vector offset outside the buffer, which makes the hardware return
// zero: no branches, all loads of a tile in flight together.
//
// Replaces, for the dense cases: device/x86/Conv/conv.c im2col (:168,:260) + opt_gemm.h SGEMM (:17)
// + bias sweep (:405) + do_act (:1216); the int32 GEMM and de-quantisation of conv.c:1024-1056;
// device/x86/MatMul/mat_mul.c:10.
#pragma once
#include "onhip_internal.hpp"
#include <type_traits>
#include <utility>

namespace onhip {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int THREADS = 256;
constexpr unsigned OOB = 0x80000000u;       // vector offset outside every buffer: loads give 0, stores vanish
constexpr unsigned RSRC_RANGE = 0x80000000u; // num_records of the data buffers (all offsets stay below 2 GiB)
constexpr unsigned RSRC_FLAGS = 0x00020000u; // 32-bit data format, raw buffer

typedef __amdgpu_buffer_rsrc_t rsrc_t;

__device__ __forceinline__ rsrc_t make_rsrc(const void *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int) bytes, (int) RSRC_FLAGS);
}
__device__ __forceinline__ float buf_load_f32(rsrc_t r, unsigned voff, unsigned soff) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ uint4 buf_load_b128(rsrc_t r, unsigned voff, unsigned soff) {
    u32x4 q = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
    return make_uint4(q.x, q.y, q.z, q.w);
}

template <int DT> struct Traits;
// mma_part: one MFMA instruction of the PARTS that consume a pair of 16-byte units
template <> struct Traits<DT_F32> {
    static constexpr int KPU = 4;
    static constexpr int RAW = 4;          // fp32 values fetched per unit
    static constexpr int PARTS = 4;        // one v_mfma_f32_32x32x2_f32 per fp32 of the unit
    typedef f32x16 acc_t;
    static __device__ __forceinline__ void mma_part(acc_t &c, const uint4 &a, const uint4 &b, int part) {
        const unsigned av = part == 0 ? a.x : part == 1 ? a.y : part == 2 ? a.z : a.w;
        const unsigned bv = part == 0 ? b.x : part == 1 ? b.y : part == 2 ? b.z : b.w;
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(av), __uint_as_float(bv), c, 0, 0, 0);
    }
};
template <> struct Traits<DT_BF16> {
    static constexpr int KPU = 8;
    static constexpr int RAW = 8;
    static constexpr int PARTS = 1;
    typedef f32x16 acc_t;
    static __device__ __forceinline__ void mma_part(acc_t &c, const uint4 &a, const uint4 &b, int) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                    0, 0, 0);
    }
};
template <> struct Traits<DT_F16> {
    static constexpr int KPU = 8;
    static constexpr int RAW = 8;
    static constexpr int PARTS = 1;
    typedef f32x16 acc_t;
    static __device__ __forceinline__ void mma_part(acc_t &c, const uint4 &a, const uint4 &b, int) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                   0, 0);
    }
};
template <> struct Traits<DT_I8> {
    static constexpr int KPU = 16;
    static constexpr int RAW = 4;          // 4 dwords = 16 int8
    static constexpr int PARTS = 1;
    typedef i32x16 acc_t;
    static __device__ __forceinline__ void mma_part(acc_t &c, const uint4 &a, const uint4 &b, int) {
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a), __builtin_bit_cast(i32x4, b), c, 0, 0,
                                                  0);
    }
};

// what a thread keeps in flight for one unit between the global load and the LDS store
template <int DT> struct RawUnit { float v[Traits<DT>::RAW]; };
template <> struct RawUnit<DT_I8> { uint4 q; };

template <int DT> __device__ __forceinline__ uint4 pack_unit(const RawUnit<DT> &r);
template <> __device__ __forceinline__ uint4 pack_unit<DT_F32>(const RawUnit<DT_F32> &r) {
    return make_uint4(__float_as_uint(r.v[0]), __float_as_uint(r.v[1]), __float_as_uint(r.v[2]),
                      __float_as_uint(r.v[3]));
}
template <> __device__ __forceinline__ uint4 pack_unit<DT_BF16>(const RawUnit<DT_BF16> &r) {
    uint4 o;
    unsigned *w = reinterpret_cast<unsigned *>(&o);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bf16x2 t = {(__bf16) r.v[2 * i], (__bf16) r.v[2 * i + 1]};  // round to nearest even
        w[i] = __builtin_bit_cast(unsigned, t);
    }
    return o;
}
template <> __device__ __forceinline__ uint4 pack_unit<DT_F16>(const RawUnit<DT_F16> &r) {
    uint4 o;
    unsigned *w = reinterpret_cast<unsigned *>(&o);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f16x2 t = {(_Float16) r.v[2 * i], (_Float16) r.v[2 * i + 1]};
        w[i] = __builtin_bit_cast(unsigned, t);
    }
    return o;
}
template <> __device__ __forceinline__ uint4 pack_unit<DT_I8>(const RawUnit<DT_I8> &r) { return r.q; }

// x / d for x * d < 2^32 with magic = floor(2^32 / d) + 1.  d == 1 is encoded as magic == 0 with
// pass == ~0u (the quotient is x itself); otherwise pass == 0.  Branch-free on purpose: a scalar
// branch between two loads would serialise them.
__device__ __forceinline__ unsigned fast_div(unsigned x, unsigned magic, unsigned pass) {
    return __umulhi(x, magic) + (x & pass);
}

// exact floor(x / d) for 0 <= x < 2^31 (see Div31)
__device__ __forceinline__ unsigned div31(unsigned x, const Div31 &d) {
    return (__umulhi(x, d.magic) >> d.shift) + (x & d.pass);
}

// ---- A: one unit of one row ----------------------------------------------------------------------
// voff: byte offset of (row, unit slot) fixed per thread, OOB for rows beyond M;
// soff: byte offset of the K tile (uniform); k0: first reduction index of this unit; klim: end of K
// CHK == false: the tile is known to lie inside K, no per-unit test
template <int DT, bool CHK>
__device__ __forceinline__ void load_a_unit(RawUnit<DT> &r, rsrc_t ra, unsigned voff, unsigned soff, int k0, int klim) {
    constexpr int KPU = Traits<DT>::KPU;
    if constexpr (DT == DT_I8) {
        r.q = buf_load_b128(ra, (!CHK || k0 < klim) ? voff : OOB, soff);
    } else {
        // dwordx4 loads need dword alignment only.  A vector that straddles the end of a row brings
        // in the head of the next row (the end of the buffer reads as zero, dwords are range-checked
        // one by one); those lanes of K are cleared before they reach LDS (clear_a_tail).
#pragma unroll
        for (int q = 0; q < KPU / 4; ++q) {
            const uint4 t = buf_load_b128(ra, (!CHK || k0 + 4 * q < klim) ? voff + 16 * q : OOB, soff);
            r.v[4 * q] = __uint_as_float(t.x); r.v[4 * q + 1] = __uint_as_float(t.y);
            r.v[4 * q + 2] = __uint_as_float(t.z); r.v[4 * q + 3] = __uint_as_float(t.w);
        }
    }
}

// zero the elements of a unit whose reduction index is at or beyond klim (ragged end of K)
template <int DT>
__device__ __forceinline__ void clear_a_tail(RawUnit<DT> &r, int k0, int klim) {
    if constexpr (DT != DT_I8) {
#pragma unroll
        for (int e = 0; e < Traits<DT>::KPU; ++e) r.v[e] = (k0 + e < klim) ? r.v[e] : 0.0f;
    }
}

// ---- B: per-thread column state, fixed for the whole K loop -------------------------------------
struct ColState {
    unsigned pixoff;   // byte offset of the receptive field's origin in the (pad-shifted) buffer, OOB if n >= N
    int ih0, iw0;      // top-left input coordinate of the receptive field
    unsigned mask_lo, mask_hi;  // bit t set: filter tap t (t = i * kw + j, t < 64) falls inside the image
};

template <int BL>
__device__ __forceinline__ ColState make_col(const IgemmParams &p, int n) {
    ColState c;
    const bool valid = n < p.N;
    const int nn = valid ? n : 0;
    const int img = (int) div31((unsigned) nn, p.div_ohw);
    const int pix = nn - img * p.OHW;
    const int oh = (int) div31((unsigned) pix, p.div_ow);
    const int ow = pix - oh * p.OW;
    c.ih0 = oh * p.sh - p.pt;
    c.iw0 = ow * p.sw - p.pl;
    unsigned off;
    if constexpr (BL != BL_KVEC && BL != BL_KVEC_TAP) off = (unsigned) (img * (int) p.b_img_stride + oh * p.sh * p.W + ow * p.sw) * 4u;
    else off = (unsigned) ((img * p.H + oh * p.sh) * p.W + ow * p.sw) * (unsigned) p.pix_stride;
    c.pixoff = valid ? off : OOB;
    c.mask_lo = c.mask_hi = 0;
    if constexpr (BL != BL_PLAIN) {
        if (p.use_tapmask) {
            int i = 0, j = 0;
            for (int t = 0; t < p.khkw; ++t) {
                const bool ok = (unsigned) (c.ih0 + i) < (unsigned) p.H && (unsigned) (c.iw0 + j) < (unsigned) p.W;
                if (ok) { if (t < 32) c.mask_lo |= 1u << t; else c.mask_hi |= 1u << (t - 32); }
                if (++j == p.kw) { j = 0; ++i; }
            }
        }
    }
    return c;
}

// Scalar description of one B load, computed a tile ahead in the shadow of the MFMAs: the
// wavefront-uniform byte offset and the bit that selects the tap in the lane's validity mask
// (0 when the reduction index is past the end of K).
struct BPrep {
    unsigned soff;
    unsigned bit;
    unsigned hi;   // the tap index is 32..63: test mask_hi
};

// item: (unit slot t, element e) for BL_PLAIN / BL_GATHER, unit slot t for BL_TAPC (BL_KVEC works per lane)
template <int DT, int BL>
__device__ __forceinline__ BPrep prep_b(const IgemmParams &p, int u, int e, int klim) {
    constexpr int KPU = Traits<DT>::KPU;
    BPrep r;
    if constexpr (BL == BL_PLAIN) {
        const int k = u * KPU + e;
        r.soff = (unsigned) k * (unsigned) p.HW * 4u;
        r.bit = k < klim ? 1u : 0u;
        r.hi = 0;
    } else if constexpr (BL == BL_GATHER) {
        const unsigned k = (unsigned) (u * KPU + e);
        const unsigned ch = fast_div(k, p.magic_khkw, p.pass_khkw);
        const unsigned rem = k - ch * (unsigned) p.khkw;
        const unsigned i = fast_div(rem, p.magic_kw, p.pass_kw);
        const unsigned j = rem - i * (unsigned) p.kw;
        r.soff = (ch * (unsigned) p.HW + i * (unsigned) p.W + j) * 4u;
        r.bit = (int) k < klim ? (1u << (rem & 31u)) : 0u;
        r.hi = rem >> 5;
    } else {
        // one description per unit: unit -> (tap, channel block), tap -> (i, j)
        const unsigned tap = fast_div((unsigned) u, p.magic_upt, p.pass_upt);
        const unsigned cb = (unsigned) u - tap * (unsigned) p.units_per_tap;
        const unsigned i = fast_div(tap, p.magic_kw, p.pass_kw);
        const unsigned j = tap - i * (unsigned) p.kw;
        r.soff = (cb * (unsigned) KPU * (unsigned) p.HW + i * (unsigned) p.W + j) * 4u;
        r.bit = u * KPU < klim ? (1u << (tap & 31u)) : 0u;
        r.hi = tap >> 5;
    }
    return r;
}

// vector offset of a prepared B load for this lane: the pixel if the tap is inside, else OOB
template <int BL, bool CHK = true>
__device__ __forceinline__ unsigned b_voff(const IgemmParams &p, const ColState &c, const BPrep &q, int u_or_k) {
    if constexpr (BL == BL_PLAIN) {
        return (!CHK || q.bit) ? c.pixoff : OOB;
    } else {
        if (p.use_tapmask) {
            const unsigned word = q.hi ? c.mask_hi : c.mask_lo;
            return (word & q.bit) ? c.pixoff : OOB;
        }
        // more than 64 taps: validity by coordinates (slow path, large filters only)
        unsigned tap;
        if constexpr (BL == BL_GATHER) {
            const unsigned k = (unsigned) u_or_k;
            tap = k - fast_div(k, p.magic_khkw, p.pass_khkw) * (unsigned) p.khkw;
        } else {   // unit index
            tap = fast_div((unsigned) u_or_k, p.magic_upt, p.pass_upt);
        }
        const unsigned i = fast_div(tap, p.magic_kw, p.pass_kw);
        const unsigned j = tap - i * (unsigned) p.kw;
        const bool ok = q.bit != 0 && (unsigned) (c.ih0 + (int) i) < (unsigned) p.H &&
                        (unsigned) (c.iw0 + (int) j) < (unsigned) p.W;
        return ok ? c.pixoff : OOB;
    }
}

// ---- epilogue ----------------------------------------------------------------------------------------
// byte offset of column n inside one batch slice of C (rows are added through the scalar offset)
__device__ __forceinline__ unsigned out_col_offset(const IgemmParams &p, int n, int esz) {
    if (p.out_mode == OUT_CONV) {
        const int img = (int) div31((unsigned) n, p.div_ohw);
        const int pix = n - img * p.OHW;
        return (unsigned) (img * (int) p.c_img_stride + pix) * (unsigned) esz;
    }
    return (unsigned) (n * (int) p.c_stride_n) * (unsigned) esz;
}

// the consumer's activation quantiser (conv.c:961-973) applied to an fp32 result
__device__ __forceinline__ int requant_s8(float y, float inv_scale) {
    float t = __fmul_rn(y, inv_scale);
    t = (t < -128.0f) ? -128.0f : (t > 127.0f) ? 127.0f : t;
    return round_half_away_small(t);
}

// Writes the accumulators of one wavefront.  Lane (li, lh) of a 32x32 block holds column li and rows
// 8*(r/4) + 4*lh + (r%4): the column and the 4*lh part of the row go in the vector offset, the rest
// of the row (uniform) in the scalar offset.  Per-row operands (bias, weight_aux, int32 bias) are all
// requested before the first one is used, through descriptors that are empty when the operand is
// absent, so the epilogue has one memory round trip and no branches.
// RES: the kernel variant for the last convolution of a residual block; the element of p.res at each output's place
// is added after the activation (add_res).  All of a wavefront's addends are requested at once, ahead of the bias:
// one memory round trip, paid for in registers, which is why the variant is a kernel of its own.
// BIAS_LDS: the per-row constants of this wavefront's rows wait in LDS, where the kernel put them when its K loop was
// over, so that the store does not begin with a trip to memory: sbias the per-row bias (-0.0f for a launch without
// one); for int8 operands the de-quantisation factors weight_aux / 127, divided once per row and not by every lane,
// and srow2 the int32 biases as floats.
template <int DT, int EPI, int TM, int TN, bool RES, bool BIAS_LDS = false, class ACC>
__device__ __forceinline__ void write_tile(const IgemmParams &p, ACC (&acc)[TM][TN], int batch, int m_wave, int n_wave,
                                           int li, int lh, const float *sbias = nullptr, const float *srow2 = nullptr) {
    const int esz = (DT == DT_I8 && p.out_s8) ? 1 : 4;
    const rsrc_t rc = make_rsrc(reinterpret_cast<const char *>(p.C) + (size_t) batch * p.c_batch_stride * esz,
                                RSRC_RANGE);
    const bool bias_m_on = p.bias_mode == BIAS_M, bias_n_on = p.bias_mode == BIAS_N;
    const rsrc_t rbias_m = make_rsrc(p.bias, bias_m_on ? (unsigned) (p.M * 4) : 0u);
    const rsrc_t rbias_n = make_rsrc(p.bias, bias_n_on ? (unsigned) (p.N * 4) : 0u);
    const bool m_edge = m_wave + TM * 32 > p.M;   // uniform: only the last row tile checks rows
    const unsigned row_bytes = (unsigned) p.c_stride_m * (unsigned) esz;
    const unsigned lh16 = (unsigned) lh * 16u;    // rows of the upper half wavefront are 4 further down

    unsigned col_voff[TN];
    float bias_n[TN];
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        const int n = n_wave + b * 32 + li;
        const bool ok = n < p.N;
        const int nn = ok ? n : 0;
        col_voff[b] = ok ? out_col_offset(p, nn, esz) + (unsigned) (4 * lh) * row_bytes : OOB;
        bias_n[b] = buf_load_f32(rbias_n, (unsigned) nn * 4u, 0);
    }
    if constexpr (DT == DT_I8) {
        const rsrc_t raux = make_rsrc(p.weight_aux, p.weight_aux ? (unsigned) (p.M * 4) : 0u);
        const rsrc_t rb32 = make_rsrc(p.bias32, p.bias32 ? (unsigned) (p.M * 4) : 0u);
        const rsrc_t racc = make_rsrc(p.acc_out ? p.acc_out + (size_t) batch * p.c_batch_stride : nullptr,
                                      p.acc_out ? RSRC_RANGE : 0u);
        const unsigned row_bytes4 = (unsigned) p.c_stride_m * 4u;
        float aux[TM][16];    // weight_aux / 127 of each of the lane's rows
        float fb32[TM][16];   // and the row's int32 bias as a float
        if constexpr (BIAS_LDS) {
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 c = *reinterpret_cast<const float4 *>(sbias + a * 32 + 8 * q + 4 * lh);
                    const float4 f = *reinterpret_cast<const float4 *>(srow2 + a * 32 + 8 * q + 4 * lh);
                    aux[a][4 * q] = c.x; aux[a][4 * q + 1] = c.y; aux[a][4 * q + 2] = c.z; aux[a][4 * q + 3] = c.w;
                    fb32[a][4 * q] = f.x; fb32[a][4 * q + 1] = f.y; fb32[a][4 * q + 2] = f.z; fb32[a][4 * q + 3] = f.w;
                }
        } else {
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const unsigned soff = (unsigned) (m_wave + a * 32 + 8 * (r / 4) + (r % 4)) * 4u;
                    aux[a][r] = buf_load_f32(raux, lh16, soff);
                    fb32[a][r] = (float) (int) __builtin_amdgcn_raw_buffer_load_b32(rb32, lh16, soff, 0);
                }
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) aux[a][r] = __fdiv_rn(aux[a][r], 127.0f);
        }
        unsigned col_voff4[TN];
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int n = n_wave + b * 32 + li;
            col_voff4[b] = n < p.N ? out_col_offset(p, n, 4) + (unsigned) (4 * lh) * row_bytes4 : OOB;
        }
        // RES: the residual operand of a folded Add (fp32 results): a row tile's addends are requested together
        const rsrc_t rres = make_rsrc(RES ? reinterpret_cast<const char *>(p.res) + (size_t) batch * p.c_batch_stride * 4 : nullptr,
                                      RES ? RSRC_RANGE : 0u);
        const rsrc_t rtwin = make_rsrc(RES ? p.twin : nullptr, RES && p.twin ? RSRC_RANGE : 0u);
        unsigned tq[TN][4];
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int j = 0; j < 4; ++j) tq[b][j] = 0;
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            float rv[RES ? 16 : 1][RES ? TN : 1];
            if constexpr (RES) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m_uni = m_wave + a * 32 + 8 * (r / 4) + (r % 4);
                    const bool row_ok = !m_edge || m_uni + 4 * lh < p.M;
#pragma unroll
                    for (int b = 0; b < TN; ++b) rv[r][b] = buf_load_f32(rres, row_ok ? col_voff[b] : OOB, (unsigned) m_uni * row_bytes);
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m_uni = m_wave + a * 32 + 8 * (r / 4) + (r % 4);
                const bool row_ok = !m_edge || m_uni + 4 * lh < p.M;
                // conv.c:1041-1056: acc * s, + bias, * (aux / 127): three separately rounded operations
                const float coeff = aux[a][r];
                const float fb = fb32[a][r];
#pragma unroll
                for (int b = 0; b < TN; ++b) {
                    const int av = acc[a][b][r];
                    if (p.acc_out)
                        __builtin_amdgcn_raw_buffer_store_b32((unsigned) av, racc, row_ok ? col_voff4[b] : OOB,
                                                              (unsigned) m_uni * row_bytes4, 0);
                    float f = __fmul_rn((float) av, p.in_scale);
                    const float fbias = __fadd_rn(f, fb);
                    f = p.bias32 ? fbias : f;
                    float y = act_fast<EPI>(__fmul_rn(f, coeff), p.ep);
                    if constexpr (RES) {
                        y = add_res(y, rv[r][b], p.res_relu, (col_voff[b] + (unsigned) m_uni * row_bytes) >> 2, p.res_body);
                        // the int8 twin: registers 4 q .. 4 q + 3 are four consecutive channels of the lane's pixel.  The
                        // quantiser's product and clamp as a multiply and a median of three (a NaN comes out as -128 here
                        // and as 0 from the comparisons of requant_s8; no finite operand produces one), the four low
                        // bytes packed with three byte permutes
                        if (p.twin) {   // uniform
                            tq[b][r % 4] = (unsigned) round_half_away_small(
                                __builtin_amdgcn_fmed3f(__fmul_rn(y, p.twin_inv_scale), -128.0f, 127.0f));
                            if (r % 4 == 3) {
                                const int n = n_wave + b * 32 + li, m4 = m_wave + a * 32 + 8 * (r / 4) + 4 * lh;
                                const bool ok = n < p.N && m4 < p.M;
                                const unsigned p01 = __builtin_amdgcn_perm(tq[b][1], tq[b][0], 0x0c0c0400u);
                                const unsigned p23 = __builtin_amdgcn_perm(tq[b][3], tq[b][2], 0x0c0c0400u);
                                __builtin_amdgcn_raw_buffer_store_b32(__builtin_amdgcn_perm(p23, p01, 0x05040100u), rtwin,
                                                                      ok ? (unsigned) (n * p.twin_pitch + m4) : OOB, 0, 0);
                            }
                        }
                    }
                    const unsigned voff = row_ok ? col_voff[b] : OOB;
                    if (p.out_s8)
                        __builtin_amdgcn_raw_buffer_store_b8((unsigned char) requant_s8(y, p.out_inv_scale), rc, voff,
                                                             (unsigned) m_uni * row_bytes, 0);
                    else
                        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(y), rc, voff, (unsigned) m_uni * row_bytes, 0);
                }
            }
        }
    } else {
        float rv[RES ? TM : 1][RES ? 16 : 1][RES ? TN : 1];
        if constexpr (RES) {
            const rsrc_t rres = make_rsrc(reinterpret_cast<const char *>(p.res) + (size_t) batch * p.c_batch_stride * 4, RSRC_RANGE);
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m_uni = m_wave + a * 32 + 8 * (r / 4) + (r % 4);
                    const bool row_ok = !m_edge || m_uni + 4 * lh < p.M;
#pragma unroll
                    for (int b = 0; b < TN; ++b)
                        rv[a][r][b] = buf_load_f32(rres, row_ok ? col_voff[b] : OOB, (unsigned) m_uni * row_bytes);
                }
        }
        float bias_m[TM][16];
        if constexpr (BIAS_LDS) {
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 t = *reinterpret_cast<const float4 *>(sbias + a * 32 + 8 * q + 4 * lh);
                    bias_m[a][4 * q + 0] = t.x; bias_m[a][4 * q + 1] = t.y; bias_m[a][4 * q + 2] = t.z; bias_m[a][4 * q + 3] = t.w;
                }
        } else {
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    bias_m[a][r] = buf_load_f32(rbias_m, lh16, (unsigned) (m_wave + a * 32 + 8 * (r / 4) + (r % 4)) * 4u);
        }
        // One add per value whatever the bias: the addend is the row's or the column's bias, or -0.0f, which leaves every
        // value as it is (the sign of a zero sum included).  Rows are tested against M in the last row tile only.
        float bias_sel[TN];
#pragma unroll
        for (int b = 0; b < TN; ++b) bias_sel[b] = bias_n_on ? bias_n[b] : -0.0f;
        auto store_rows = [&](auto edge) __attribute__((always_inline)) {
            constexpr bool EDGE = decltype(edge)::value;
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m_uni = m_wave + a * 32 + 8 * (r / 4) + (r % 4);   // row of lanes with lh == 0
                    const bool row_ok = !EDGE || m_uni + 4 * lh < p.M;
#pragma unroll
                    for (int b = 0; b < TN; ++b) {
                        // bias after the full sum
                        float v = __fadd_rn(acc[a][b][r], (BIAS_LDS ? !bias_n_on : bias_m_on) ? bias_m[a][r] : bias_sel[b]);
                        v = act_fast<EPI>(v, p.ep);
                        if constexpr (RES)
                            v = add_res(v, rv[a][r][b], p.res_relu, (col_voff[b] + (unsigned) m_uni * row_bytes) >> 2, p.res_body);
                        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rc, row_ok ? col_voff[b] : OOB,
                                                              (unsigned) m_uni * row_bytes, 0);
                    }
                }
        };
        if (m_edge) store_rows(std::true_type{});
        else store_rows(std::false_type{});
    }
}

// int8 NHWC output (element (pixel n, channel m) at n * pitch + m, pitch a multiple of 16): the requantised
// bytes of the workgroup's tile are transposed through LDS so that a thread stores 16 consecutive channels of
// one pixel with a single 128-bit access instead of 16 single bytes to 16 different pixels.  A lane holds four
// consecutive channels of a pixel (accumulator registers 4q .. 4q+3), which go to LDS as one dword.  Channels
// between M and the pitch are written as zero.  stage: BN * (BM + 16) bytes of LDS nobody reads any more.
// rows: when not null, LDS holding the tile's per-row constants, BM de-quantisation factors weight_aux / 127 followed by
// the BM int32 biases as floats (rows m0 .. m0 + BM - 1), which the caller computed once per row; otherwise every lane
// fetches and divides for its own 16 x TM rows.  table_ready: the caller (a persistent workgroup) has already copied the
// quantised activation table to stage + BN * (BM + 16).
template <int EPI, int BM, int BN, int TM, int TN, bool QLUT_IN_LDS, class ACC>
__device__ __forceinline__ void write_tile_nhwc_s8(const IgemmParams &p, ACC (&acc)[TM][TN], unsigned char *stage, int m0,
                                                   int n0, int m_wave, int n_wave, int li, int lh, int tid,
                                                   const float *rows = nullptr, bool table_ready = false) {
    constexpr int PITCH = BM + 16;
    const unsigned lh16 = (unsigned) lh * 16u;
    float aux[TM][16];      // the factor weight_aux / 127 of each of the lane's rows
    float fb32[TM][16];     // and the row's int32 bias as a float
    if (rows) {
        // a lane's rows come in runs of four (8 (r / 4) + 4 lh + r % 4): one 16-byte read per run and constant
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int ml = m_wave - m0 + a * 32 + 8 * q + 4 * lh;
                const float4 c = *reinterpret_cast<const float4 *>(rows + ml);
                const float4 f = *reinterpret_cast<const float4 *>(rows + BM + ml);
                aux[a][4 * q] = c.x; aux[a][4 * q + 1] = c.y; aux[a][4 * q + 2] = c.z; aux[a][4 * q + 3] = c.w;
                fb32[a][4 * q] = f.x; fb32[a][4 * q + 1] = f.y; fb32[a][4 * q + 2] = f.z; fb32[a][4 * q + 3] = f.w;
            }
    } else {
        const rsrc_t raux = make_rsrc(p.weight_aux, p.weight_aux ? (unsigned) (p.M * 4) : 0u);
        const rsrc_t rb32 = make_rsrc(p.bias32, p.bias32 ? (unsigned) (p.M * 4) : 0u);
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const unsigned soff = (unsigned) (m_wave + a * 32 + 8 * (r / 4) + (r % 4)) * 4u;
                aux[a][r] = buf_load_f32(raux, lh16, soff);
                fb32[a][r] = (float) (int) __builtin_amdgcn_raw_buffer_load_b32(rb32, lh16, soff, 0);
            }
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) aux[a][r] = __fdiv_rn(aux[a][r], 127.0f);
    }
    // the quantised activation table (8 KiB) next to the staging area: byte gathers from LDS instead of memory, through
    // a pointer the compiler knows to be LDS (a pointer that may be either makes every gather a flat access)
    typedef const __attribute__((address_space(3))) signed char *lds_s8_t;
    const signed char *qtab = p.ep.qlut;
    lds_s8_t qtab_lds = nullptr;
    if (EPI == EPI_LUT && p.ep.qlut && QLUT_IN_LDS) {
        unsigned char *ql = stage + BN * PITCH;
        if (!table_ready) {   // uniform
            const uint4 *src = reinterpret_cast<const uint4 *>(p.ep.qlut);
#pragma unroll
            for (int i = 0; i < 8192 / 16 / THREADS; ++i) reinterpret_cast<uint4 *>(ql)[tid + i * THREADS] = src[tid + i * THREADS];
            if (tid == 0) ql[-1] = 0;   // the entry "below the table": see the gather
            __syncthreads();
        }
        qtab_lds = (lds_s8_t) ql;
    }
    const bool table = EPI == EPI_LUT && p.ep.qlut != nullptr;   // uniform: the table entries arrive quantised
    float q_lo = -128.0f, q_hi = 127.0f;                         // the merged clamp of the branch without a table
    if constexpr (EPI == EPI_RELU) q_lo = 0.0f;
    if constexpr (EPI == EPI_CLIP) {
        q_lo = fmaxf(__fmul_rn(p.ep.clip_min, p.out_inv_scale), -128.0f);
        q_hi = fminf(__fmul_rn(p.ep.clip_max, p.out_inv_scale), 127.0f);
    }
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int ml = m_wave - m0 + a * 32 + 8 * q + 4 * lh;   // first of the lane's four channels, tile-local
            // the lane's 4 x TN values of this row group in three sweeps (arithmetic, table reads, selection), so that
            // the table reads of a group are all in flight together instead of each being waited for on its own
            float x[TN][4];
            int q8[TN][4];
#pragma unroll
            for (int b = 0; b < TN; ++b)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int r = 4 * q + j;
                    // without a bias fb32 is 0, and adding it changes nothing that reaches an int8 result (the sum of an
                    // integer times a positive scale is never -0)
                    const float f = __fadd_rn(__fmul_rn((float) acc[a][b][r], p.in_scale), fb32[a][r]);
                    x[b][j] = __fmul_rn(f, aux[a][r]);
                }
            if (table && QLUT_IN_LDS) {
                // act_fast<EPI_LUT>'s rules with the table behind the output quantiser and in LDS.  (x + 8) * 512 as one
                // fused multiply-add: the product by 512 is exact, so both round x + 8 once.  Rounded DOWN to an integer
                // and held to -1 .. 8191, the index says "below the table" (x < -8: the result is 0) as -1, and the byte
                // before the table, the last of the staging area's padding that no store or read touches, holds that 0.
                unsigned l[TN][4];
                bool beyond = false;
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        int idx;
                        asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(idx) : "v"(__builtin_fmaf(x[b][j], 512.0f, 4096.0f)));
                        idx = max(-1, min(idx, 8191));
                        l[b][j] = (unsigned char) qtab_lds[idx];
                        beyond |= x[b][j] >= 8.0f;
                    }
                // beyond the table the activation is the identity: rare enough that a wavefront usually skips this whole
                if (__builtin_amdgcn_ballot_w64(beyond) != 0ull) {
#pragma unroll
                    for (int b = 0; b < TN; ++b)
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const unsigned hi = (unsigned) requant_s8(x[b][j], p.out_inv_scale) & 0xffu;
                            l[b][j] = x[b][j] >= 8.0f ? hi : l[b][j];
                        }
                }
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) q8[b][j] = (int) l[b][j];
            } else if (table) {   // the same from the table in global memory
                int l[TN][4];
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        int idx = (int) __fmul_rn(__fadd_rn(x[b][j], 8.0f), 512.0f);
                        idx = idx < 0 ? 0 : idx > 8191 ? 8191 : idx;
                        l[b][j] = qtab[idx];
                    }
                bool beyond = false;
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        q8[b][j] = x[b][j] < -8.0f ? 0 : l[b][j];
                        beyond |= x[b][j] >= 8.0f;
                    }
                if (__builtin_amdgcn_ballot_w64(beyond) != 0ull) {
#pragma unroll
                    for (int b = 0; b < TN; ++b)
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int hi = requant_s8(x[b][j], p.out_inv_scale);
                            q8[b][j] = x[b][j] >= 8.0f ? hi : q8[b][j];
                        }
                }
            } else if constexpr (EPI == EPI_NONE || EPI == EPI_RELU || EPI == EPI_CLIP) {
                // activation, product with 1 / output_scale and the quantiser's clamp as ONE median of three on
                // x / output_scale: the product and its rounding are monotonic, so clamping to [a, b] before it and to
                // [fl(a / s), fl(b / s)] after it give the same float, and two nested clamps are one.  (A NaN comes out as
                // the lower bound here and as 0 from the separate steps; no finite scale or weight produces one.)
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        q8[b][j] = round_half_away_small(__builtin_amdgcn_fmed3f(__fmul_rn(x[b][j], p.out_inv_scale), q_lo, q_hi));
            } else {
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) q8[b][j] = requant_s8(act_fast<EPI>(x[b][j], p.ep), p.out_inv_scale);
            }
            // channels past the last are stored as zero: a mask over the word of four
            const int left = p.M - (m0 + ml);
            const unsigned keep = left >= 4 ? 0xffffffffu : left <= 0 ? 0u : (1u << (8 * left)) - 1u;
#pragma unroll
            for (int b = 0; b < TN; ++b) {
                // the low bytes of four integers into one word: three byte permutes
                const unsigned p01 = __builtin_amdgcn_perm((unsigned) q8[b][1], (unsigned) q8[b][0], 0x0c0c0400u);
                const unsigned p23 = __builtin_amdgcn_perm((unsigned) q8[b][3], (unsigned) q8[b][2], 0x0c0c0400u);
                const unsigned packed = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
                const int nl = n_wave - n0 + b * 32 + li;
                *reinterpret_cast<unsigned *>(stage + nl * PITCH + ml) = packed & keep;
            }
        }
    __syncthreads();
    constexpr int GROUPS = BM / 16;
    const rsrc_t rc = make_rsrc(p.C, RSRC_RANGE);
    const int pitch = (int) p.c_stride_n;
#pragma unroll
    for (int f0 = 0; f0 < BN * GROUPS; f0 += THREADS) {
        const int f = f0 + tid;
        const int nl = f / GROUPS, g = f % GROUPS;
        const uint4 v = *reinterpret_cast<const uint4 *>(stage + nl * PITCH + g * 16);
        const int n = n0 + nl, m = m0 + g * 16;
        const bool ok = ((BN * GROUPS) % THREADS == 0 || f < BN * GROUPS) && n < p.N && m < pitch;
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{v.x, v.y, v.z, v.w}, rc, ok ? (unsigned) (n * pitch + m) : OOB, 0, 0);
    }
}

// two fp32 values rounded to the 16-bit type (nearest even) and packed, low half first; and back
template <int DT> __device__ __forceinline__ unsigned pack_h16(float lo, float hi) {
    if constexpr (DT == DT_BF16) {
        const bf16x2 t = {(__bf16) lo, (__bf16) hi};
        return __builtin_bit_cast(unsigned, t);
    } else {
        const f16x2 t = {(_Float16) lo, (_Float16) hi};
        return __builtin_bit_cast(unsigned, t);
    }
}
template <int DT> __device__ __forceinline__ float unpack_h16(unsigned w, int half) {
    if constexpr (DT == DT_BF16) return __uint_as_float(half ? (w & 0xffff0000u) : (w << 16));
    else {
        const f16x2 t = __builtin_bit_cast(f16x2, w);
        return (float) (half ? t.y : t.x);
    }
}

// 16-bit NHWC output (bf16 or fp16; element (pixel n, channel m) at (n * pitch + m) * 2 bytes, pitch = p.c_stride_n a
// multiple of 8): bias and activation in fp32 on the accumulators, rounding to the 16-bit type, then the tile is
// transposed through LDS so that a thread stores 8 consecutive channels of one pixel with a single 128-bit access.  A
// lane holds four consecutive channels of a pixel (accumulator registers 4q .. 4q+3), which go to LDS as 8 bytes.
// An optional residual operand (p.res16, same layout as the output) is added in fp32 to the rounded value on the way
// out, followed by a ReLU when p.res_relu says so, and the sum is rounded again: what a separate Add (+ Relu) operator
// on the 16-bit tensors would store.  Channels between M and the pitch are written as zero.
// stage: BN * (2 BM + 16) bytes of LDS nobody reads any more.  rows: LDS holding the BM per-row biases of the tile
// (zero where there is none).
template <int DT, int EPI, int BM, int BN, int TM, int TN>
__device__ __forceinline__ void write_tile_nhwc_h16(const IgemmParams &p, f32x16 (&acc)[TM][TN], unsigned char *stage, int m0,
                                                    int n0, int m_wave, int n_wave, int li, int lh, int tid,
                                                    const float *rows) {
    static_assert(DT == DT_BF16 || DT == DT_F16, "16-bit floating-point outputs");
    constexpr int PITCH = 2 * BM + 16;
    // Table activations: the 8192 fp32 entries rounded to the output type, 16 KiB of LDS behind the staging area (the
    // caller leaves them free).  The value stored is round(table[i]) either way; the gathers then hit LDS instead of
    // sending 64 addresses per instruction to memory.
    typedef const __attribute__((address_space(3))) unsigned short *lds_u16_t;
    lds_u16_t tab = nullptr;
    if constexpr (EPI == EPI_LUT) {
        unsigned char *tl = stage + BN * PITCH;
        const float4 *src = reinterpret_cast<const float4 *>(p.ep.lut);
        float4 t[8192 / 4 / THREADS];
#pragma unroll
        for (int i = 0; i < 8192 / 4 / THREADS; ++i) t[i] = src[tid + i * THREADS];
#pragma unroll
        for (int i = 0; i < 8192 / 4 / THREADS; ++i)
            reinterpret_cast<uint2 *>(tl)[tid + i * THREADS] = make_uint2(pack_h16<DT>(t[i].x, t[i].y), pack_h16<DT>(t[i].z, t[i].w));
        __syncthreads();
        tab = (lds_u16_t) tl;
    }
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int ml = m_wave - m0 + a * 32 + 8 * q + 4 * lh;   // first of the lane's four channels, tile-local
            const float4 bias = *reinterpret_cast<const float4 *>(rows + ml);
            const float bv[4] = {bias.x, bias.y, bias.z, bias.w};
            float y[TN][4];
            if constexpr (EPI == EPI_LUT) {
                // act_fast<EPI_LUT>'s rules; the table reads of the row group all in flight together
                float v[TN][4];
                unsigned short l[TN][4];
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        v[b][j] = __fadd_rn(acc[a][b][4 * q + j], bv[j]);
                        int idx = (int) __fmul_rn(__fadd_rn(v[b][j], 8.0f), 512.0f);
                        idx = idx < 0 ? 0 : idx > 8191 ? 8191 : idx;
                        l[b][j] = tab[idx];
                    }
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float lv = unpack_h16<DT>((unsigned) l[b][j], 0);
                        const float r = v[b][j] < -8.0f ? 0.0f : v[b][j] >= 8.0f ? v[b][j] : lv;
                        y[b][j] = (m0 + ml + j < p.M) ? r : 0.0f;
                    }
            } else {
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float v = act_fast<EPI>(__fadd_rn(acc[a][b][4 * q + j], bv[j]), p.ep);
                        y[b][j] = (m0 + ml + j < p.M) ? v : 0.0f;
                    }
            }
#pragma unroll
            for (int b = 0; b < TN; ++b) {
                const int nl = n_wave - n0 + b * 32 + li;
                *reinterpret_cast<uint2 *>(stage + nl * PITCH + ml * 2) = make_uint2(pack_h16<DT>(y[b][0], y[b][1]), pack_h16<DT>(y[b][2], y[b][3]));
            }
        }
    __syncthreads();
    constexpr int GROUPS = BM / 8;
    const rsrc_t rc = make_rsrc(p.C, RSRC_RANGE);
    const rsrc_t rr = make_rsrc(p.res16, p.res16 ? RSRC_RANGE : 0u);
    const int pitch = (int) p.c_stride_n;
    const bool with_res = p.res16 != nullptr, relu = p.res_relu != 0;
#pragma unroll
    for (int f0 = 0; f0 < BN * GROUPS; f0 += THREADS) {
        const int f = f0 + tid;
        const int nl = f / GROUPS, g = f % GROUPS;
        uint4 v = *reinterpret_cast<const uint4 *>(stage + nl * PITCH + g * 16);
        const int n = n0 + nl, m = m0 + g * 8;
        const bool ok = ((BN * GROUPS) % THREADS == 0 || f < BN * GROUPS) && n < p.N && m < pitch;
        const unsigned off = ok ? (unsigned) (n * pitch + m) * 2u : OOB;
        if (with_res) {   // uniform
            const u32x4 r = __builtin_amdgcn_raw_buffer_load_b128(rr, off, 0, 0);
            unsigned *w = reinterpret_cast<unsigned *>(&v);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float lo = __fadd_rn(unpack_h16<DT>(w[i], 0), unpack_h16<DT>(r[i], 0));
                float hi = __fadd_rn(unpack_h16<DT>(w[i], 1), unpack_h16<DT>(r[i], 1));
                if (relu) { lo = lo > 0.0f ? lo : 0.0f; hi = hi > 0.0f ? hi : 0.0f; }
                w[i] = pack_h16<DT>(lo, hi);
            }
        }
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{v.x, v.y, v.z, v.w}, rc, off, 0, 0);
    }
}

__device__ __forceinline__ unsigned to_bits(float v) { return __float_as_uint(v); }
__device__ __forceinline__ unsigned to_bits(int v) { return (unsigned) v; }

// cache policy bits of the raw-buffer instructions on gfx950: sc0 (bit 0) and sc1 (bit 4) together give an access system
// scope: a store is written through to memory before it is acknowledged, a load does not hit a line that another XCD's
// store has made stale.  The in-launch split-K reduction puts them on the partial sums it publishes and reads back.
constexpr int AUX_SYSTEM_SCOPE = 0x11;

// split-K: raw partial sums [split][batch][M][N]; the finishing kernel applies the epilogue.  PUBLISH: the sums are read
// back by another workgroup of the same launch (system-scope stores); otherwise by the finishing launch.
template <int TM, int TN, bool PUBLISH, class ACC>
__device__ __forceinline__ void write_partial(const IgemmParams &p, ACC (&acc)[TM][TN], int slice, int m_wave,
                                              int n_wave, int li, int lh) {
    const int width = p.N - p.part_begin;   // partial sums cover the columns from part_begin on
    const rsrc_t rp = make_rsrc(reinterpret_cast<const char *>(p.partial) + (size_t) slice * p.M * width * 4, RSRC_RANGE);
    const bool m_edge = m_wave + TM * 32 > p.M;
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        const int n = n_wave + b * 32 + li;
        const unsigned cv = n < p.N ? (unsigned) (n - p.part_begin + 4 * lh * width) * 4u : OOB;
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m_uni = m_wave + a * 32 + 8 * (r / 4) + (r % 4);
                const bool row_ok = !m_edge || m_uni + 4 * lh < p.M;
                const auto val = acc[a][b][r];   // element copy first: bit-casting the vector element in place miscompiles
                __builtin_amdgcn_raw_buffer_store_b32(to_bits(val), rp, row_ok ? cv : OOB,
                                                      (unsigned) m_uni * (unsigned) width * 4u, PUBLISH ? AUX_SYSTEM_SCOPE : 0);
            }
    }
}

// ---- a second, 1x1 product over the finished tile (the PW2 variant of the kernel, fp32, tile 64 x 64) ---------------------
// The workgroup's tile holds every row of the first product (M <= 64) for its 64 columns, so it is the whole B operand
// of a 1x1 convolution over that result for these columns: out[m2][64] = w2[m2][M] * act(tile + bias).  The tile goes to
// LDS in the B layout of the K loop ([unit of 4 rows][column][16 B]; a lane's accumulator registers 4q .. 4q+3 are four
// consecutive rows of one column, i.e. exactly one unit), and every wavefront then walks the rows of w2 in blocks of
// 64 (32 per wavefront), its B operand read from that tile one step ahead and its A operands loaded straight from
// memory, where they lie in the MFMA's own layout (lane li = row, lanes 32-63 the odd unit of a step; w2 is packed
// that way once): no barrier in this loop.  The reduction runs in the order of the K loop (unit pairs ascending, the four elements of a
// unit one MFMA each), so the result has the bits of the two launches it replaces when those use this tile.
// tl: LDS of at least 16 * 64 * 16 bytes that no wavefront reads any more (the caller has synchronised).
template <int EPI, bool RES>
__device__ __forceinline__ void pw2_stage(const IgemmParams &p, const f32x16 &acc1, uint4 *tl, const float *sbias, int n0, int wm, int wn,
                                          int li, int lh) {
    const unsigned lh16 = (unsigned) lh * 16u;
    const int cmid = p.M;
    // the first product's bias, rows 8 (r / 4) + 4 lh + r % 4 of the wavefront's 32: requested before the K loop, in LDS,
    // -0.0f (the addend that changes nothing, not even the sign of a zero sum) where there is none
    float b1[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 t = *reinterpret_cast<const float4 *>(sbias + wm * 32 + 8 * q + 4 * lh);
        b1[4 * q + 0] = t.x; b1[4 * q + 1] = t.y; b1[4 * q + 2] = t.z; b1[4 * q + 3] = t.w;
    }
    // A of the second product, re-laid once by pack_pw2_launch into the order this loop reads it: for every block of 64
    // rows, half wm and step s the 64 lanes' 16 bytes side by side (lane (li, lh): row block * 64 + wm * 32 + li, unit
    // 2 s + lh; zeros beyond m2 rows and M columns), so a load instruction is one contiguous KiB
    const int mblocks = (p.m2 + 63) / 64;
    const rsrc_t rw2 = make_rsrc(p.w2, (unsigned) (mblocks * 64 * 64 * 4));
    const unsigned lane16 = (unsigned) (lh * 32 + li) * 16u;
    uint4 wa[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) wa[s] = buf_load_b128(rw2, lane16, (unsigned) (wm * 8 + s) * 1024u);
    // the first product's activation is none, Relu or Clip (the launcher refuses others): apply_act's comparisons as
    // selects under two uniform flags, so that the sixteen values take no branch
    const bool lo_on = p.ep.act == RELU || p.ep.act == CLIP, hi_on = p.ep.act == CLIP;
    const float lo = p.ep.act == CLIP ? p.ep.clip_min : 0.0f, hi = p.ep.clip_max;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = 4 * q + j;
            float x = __fadd_rn(acc1[r], b1[r]);
            x = (lo_on & !(x > lo)) ? lo : x;
            x = (hi_on & !(x < hi)) ? hi : x;
            v[j] = wm * 32 + 8 * q + 4 * lh + j < cmid ? x : 0.0f;
        }
        tl[(wm * 8 + 2 * q + lh) * 64 + wn * 32 + li] = make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3]));
    }
    __syncthreads();
    // B of the second product stays in LDS: the 16 bytes of a step are read one step ahead (eight registers, not the 32
    // of the whole operand, which cost the kernel a wavefront per SIMD)
    const uint4 *tbp = tl + lh * 64 + wn * 32 + li;
    uint4 tb_next = tbp[0];

    const rsrc_t rc = make_rsrc(p.C, RSRC_RANGE);
    const rsrc_t rres = make_rsrc(RES ? p.res : nullptr, RES ? RSRC_RANGE : 0u);
    const rsrc_t rb2 = make_rsrc(p.bias2, p.bias2 ? (unsigned) (p.m2 * 4) : 0u);
    const bool bias2_on = p.bias2 != nullptr;
    const unsigned row_bytes = (unsigned) p.c_stride_m * 4u;
    const int n = n0 + wn * 32 + li;
    const unsigned col_voff = n < p.N ? out_col_offset(p, n, 4) + (unsigned) (4 * lh) * row_bytes : OOB;
    // One operand set: the 16 bytes of step s are requested again, for the next block of rows, as soon as the step's
    // four MFMAs have been issued, so every load has most of a block's matrix work (and the stores) to arrive.  A block
    // past the end loads nothing (its rows are beyond m2).
    for (int mb = 0; mb < mblocks; ++mb) {
        const int m_wave = mb * 64 + wm * 32;   // uniform
        const bool m_edge = m_wave + 32 > p.m2;
        float b2[16], rv[RES ? 16 : 1];
#pragma unroll
        for (int r = 0; r < 16; ++r) b2[r] = buf_load_f32(rb2, lh16, (unsigned) (m_wave + 8 * (r / 4) + (r % 4)) * 4u);
        if constexpr (RES) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m_uni = m_wave + 8 * (r / 4) + (r % 4);
                rv[r] = buf_load_f32(rres, (!m_edge || m_uni + 4 * lh < p.m2) ? col_voff : OOB, (unsigned) m_uni * row_bytes);
            }
        }
        f32x16 acc2;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc2[r] = 0.0f;
        const unsigned next_voff = mb + 1 < mblocks ? lane16 : OOB;
        const unsigned next_soff = (unsigned) (((mb + 1) * 2 + wm) * 8) * 1024u;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint4 tb = tb_next;
            tb_next = tbp[((s + 1) & 7) * 128];   // step s + 1, or step 0 of the next block of rows
#pragma unroll
            for (int part = 0; part < 4; ++part) Traits<DT_F32>::mma_part(acc2, wa[s], tb, part);
            wa[s] = buf_load_b128(rw2, next_voff, next_soff + 1024u * s);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m_uni = m_wave + 8 * (r / 4) + (r % 4);
            const bool row_ok = !m_edge || m_uni + 4 * lh < p.m2;
            float v = acc2[r];
            v = bias2_on ? __fadd_rn(v, b2[r]) : v;
            v = act_fast<EPI>(v, p.ep2);
            if constexpr (RES) v = add_res(v, rv[r], p.res_relu, (col_voff + (unsigned) m_uni * row_bytes) >> 2, p.res_body);
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rc, row_ok ? col_voff : OOB, (unsigned) m_uni * row_bytes, 0);
        }
    }
}

// ---- the kernel --------------------------------------------------------------------------------
template <int DT, int BL, int BM, int BN, int WM, int WN, int PF = 1, bool RES = false, bool PW2 = false>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(PW2 ? 4 : 1))) void igemm_kernel(const IgemmParams p) {
    static_assert(!PW2 || (DT == DT_F32 && BM == 64 && BN == 64 && WM == 2 && WN == 2), "the second product exists for fp32 tiles of 64 x 64");
    static_assert(!RES || DT == DT_F32 || DT == DT_I8, "the residual store exists for fp32 and int8 operands (fp32 results)");
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    static_assert(TM >= 1 && TN >= 1 && BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "tile / wave grid mismatch");
    static_assert(THREADS % BN == 0 || BN % THREADS == 0, "B loader mapping");
    constexpr int KPU = Traits<DT>::KPU;
    constexpr int ESZ = DT == DT_I8 ? 1 : 4;   // bytes per stored operand element
    constexpr int UPT = 4;                     // 16-byte units per K tile
    constexpr int A_SLOTS = BM * UPT, B_SLOTS = BN * UPT;
    // A reaches LDS from threads that hold the UPT units of one row side by side: one spare slot per unit row
    // puts those UPT stores in different banks
    constexpr int A_LD = BM + 1, A_LDS = A_LD * UPT;
    // The vector loader (BL_KVEC) gives the UPT units of one column to neighbouring lanes as well: they are
    // contiguous in memory (one 64-byte run per pixel instead of 64 scattered 16-byte pieces per load), and the
    // filter tap of a unit becomes a per-lane quantity.
    constexpr bool LANE_UNITS = BL == BL_KVEC || BL == BL_KVEC_TAP;
    constexpr int B_LD = LANE_UNITS ? BN + 1 : BN, B_LDS = B_LD * UPT;
    constexpr int A_PER_T = (A_SLOTS + THREADS - 1) / THREADS;
    constexpr int B_PER_T = B_SLOTS / THREADS;
    static_assert(B_PER_T >= 1, "BN >= 64");
    typedef typename Traits<DT>::acc_t acc_t;

    __shared__ uint4 lds[2][A_LDS + B_LDS];
    // the tile's rows of the store's per-row constants: the bias (fp32 / 16-bit operand kernels; with PW2 the first
    // product's), or weight_aux / 127 followed by the int32 bias as a float (int8).  Requested with the first operand
    // tiles, in LDS when the K loop is over
    constexpr bool BIAS_LDS = true;
    __shared__ __attribute__((aligned(16))) float s_bias[DT == DT_I8 ? 2 * BM : BM];

    const int tid = threadIdx.x;
    // the wavefront index is uniform; saying so keeps everything derived from it in scalar registers
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    // XCD-aware tile order: consecutive workgroup ids go round-robin over the 8 XCDs (each with its
    // own L2); give every XCD a contiguous run of tiles so neighbours in (m, n) share an L2.
    const int tiles_m = (p.M + BM - 1) / BM;
    // A launch with dp_tiles > 0 has two kinds of workgroups: the first dp_tiles take one whole tile each (all of K,
    // result written directly), the others take one of `split` K slices of one of the tail_tiles tiles left over and
    // write partial sums.  Slices of one tile are tail_tiles workgroup ids apart, so they land on different CUs.
    int lid, slice = blockIdx.y;
    bool whole_k = false;
    {
        const int bid = blockIdx.x;
        if (p.dp_tiles > 0 && bid >= p.dp_tiles) {
            const int r = bid - p.dp_tiles;
            slice = r / p.tail_tiles;
            lid = p.dp_tiles + (r - slice * p.tail_tiles);
        } else {
            const int nb = p.dp_tiles > 0 ? p.dp_tiles : (int) gridDim.x;
            const int q = nb >> 3, rmd = nb & 7, xcd = bid & 7, idx = bid >> 3;
            lid = xcd * q + (xcd < rmd ? xcd : rmd) + idx;
            whole_k = p.dp_tiles > 0;
        }
    }
    int tile_n = (int) div31((unsigned) lid, p.div_tiles_m), tile_m = lid - tile_n * tiles_m;
    if (p.n_fast && p.dp_tiles == 0) {   // uniform: rows of A stay in the XCD's L2 while it sweeps the column blocks
        const int tiles_n = (p.N + BN - 1) / BN;
        tile_m = (int) div31((unsigned) lid, p.div_tiles_n);
        tile_n = lid - tile_m * tiles_n;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int batch = blockIdx.z;
    const int u_begin = whole_k ? 0 : slice * p.k_split_units;
    const int u_end = whole_k ? p.k_units : min(p.k_units, u_begin + p.k_split_units);
    const int k_tiles = (u_end - u_begin + UPT - 1) / UPT;
    const int klim = min(p.K, u_end * KPU);

    // The last K tile of this slice is ragged when it is cut by the end of K or of the slice; only then do
    // loads and LDS stores test reduction indices one by one (the CHK variants below).
    const bool ragged = ((u_end - u_begin) % UPT) != 0 || klim < u_end * KPU;

    // exact extent: the dwords of a row-end vector that fall past the matrix read as zero
    const char *a_base = reinterpret_cast<const char *>(p.A) + (size_t) batch * p.a_batch_stride * ESZ;
    // the B buffer starts pad rows/columns before the tensor so that pixel offsets are never negative
    // and ends with the tensor: channel padding of the last image reads as zero
    const char *b_base = reinterpret_cast<const char *>(p.B) + (size_t) batch * p.b_batch_stride * ESZ -
                         (size_t) p.b_shift_bytes;
    const unsigned a_bytes = (unsigned) p.a_slice_bytes, b_bytes = (unsigned) (p.b_slice_bytes + p.b_shift_bytes);

    // per-thread A slots: (row, unit-in-tile) fixed for the whole K loop
    unsigned a_voff[A_PER_T];
    int a_unit[A_PER_T];
#pragma unroll
    for (int t = 0; t < A_PER_T; ++t) {
        const int f = tid + t * THREADS;
        const int ml = f / UPT, ua = f % UPT;
        const bool ok = ((A_SLOTS % THREADS == 0) || f < A_SLOTS) && m0 + ml < p.M;
        a_unit[t] = ua;
        a_voff[t] = ok ? (unsigned) ((m0 + ml) * p.lda + ua * KPU) * (unsigned) ESZ : OOB;
    }
    // per-thread B column(s): one for all of the thread's units, or (LANE_UNITS) one per slot
    constexpr int NCOL = LANE_UNITS ? B_PER_T : 1;
    ColState cols[NCOL];
#pragma unroll
    for (int t = 0; t < NCOL; ++t)
        cols[t] = make_col<BL>(p, n0 + (LANE_UNITS ? (tid + t * THREADS) / UPT : tid % BN));
    const ColState &col = cols[0];
    const unsigned lane_unit_off = (unsigned) (tid % UPT) * 16u;

    acc_t acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;

    // PF K tiles are in flight between global memory and LDS, each in a register set of its own (tile t in
    // set t % PF).  One set covers one memory latency per K tile; short tiles (two int8 MFMAs per wavefront)
    // need several.
    RawUnit<DT> qa_[PF][A_PER_T], qb_[PF][B_PER_T];

    constexpr int PARTS = Traits<DT>::PARTS;
    constexpr int BE = BL == BL_TAPC ? 1 : KPU;                      // scalar descriptions per B unit
    constexpr int B_ITEMS = LANE_UNITS ? 0 : B_PER_T * BE;
    constexpr int BLOCKS = (UPT / 2) * TM * TN;       // 32x32 blocks x unit pairs per K tile
    constexpr int STEPS = BLOCKS * PARTS;             // MFMA instructions per K tile and wavefront
    constexpr int HALF = STEPS / 2;
    constexpr int READS = (UPT / 2) * (TM + TN);      // LDS operand reads per K tile and wavefront
    struct Operands { uint4 a[UPT / 2][TM], b[UPT / 2][TN]; };

    BPrep bp[B_ITEMS > 0 ? B_ITEMS : 1];              // scalar descriptions of the next B loads
    const unsigned hw4 = (unsigned) p.HW * 4u;

    auto b_unit_of = [&](int t) __attribute__((always_inline)) { return __builtin_amdgcn_readfirstlane((tid + t * THREADS) / BN); };
    auto prep_item = [&](int kt, int idx) __attribute__((always_inline)) {
        const int t = idx / BE, e = idx % BE;
        bp[idx] = prep_b<DT, BL>(p, u_begin + kt * UPT + b_unit_of(t), e, klim);
    };
    // issue every global load of K tile kt (B descriptions must have been prepared for kt).  A tile past the
    // end of the slice is switched off as a whole through empty buffer descriptors (a scalar select): its
    // loads return zero without touching memory.  CHK adds the per-unit tests a ragged last tile needs.
    auto issue = [&](int kt, auto chk, auto slot) __attribute__((always_inline)) {
        constexpr bool CHK = decltype(chk)::value;
        RawUnit<DT> (&qa)[A_PER_T] = qa_[decltype(slot)::value];
        RawUnit<DT> (&qb)[B_PER_T] = qb_[decltype(slot)::value];
        const int ub = u_begin + kt * UPT;
        const bool live = kt < k_tiles;
        const rsrc_t ra = make_rsrc(a_base, live ? a_bytes : 0u);
        const rsrc_t rb = make_rsrc(b_base, live ? b_bytes : 0u);
#pragma unroll
        for (int t = 0; t < A_PER_T; ++t)
            load_a_unit<DT, CHK>(qa[t], ra, a_voff[t], (unsigned) (ub * KPU * ESZ), (ub + a_unit[t]) * KPU, klim);
        if constexpr (BL == BL_KVEC_TAP) {
            // the UPT units of the tile share one filter tap: tap, offset and mask bit are scalar, a lane only
            // adds its unit's 16 bytes (kept in lane_unit_off) and tests the tap in its column's mask
            const unsigned tap = fast_div((unsigned) ub, p.magic_upt, p.pass_upt);
            const unsigned cb0 = (unsigned) ub - tap * (unsigned) p.units_per_tap;
            const unsigned ti = fast_div(tap, p.magic_kw, p.pass_kw);
            const unsigned tj = tap - ti * (unsigned) p.kw;
            const unsigned soff = (ti * (unsigned) p.W + tj) * (unsigned) p.pix_stride + cb0 * 16u;
            const unsigned bit = 1u << (tap & 31u);
            const bool hi = tap >= 32u;
            const bool k_ok = !CHK || (int) (((unsigned) ub + (unsigned) (tid % UPT)) * KPU) < klim;
#pragma unroll
            for (int t = 0; t < B_PER_T; ++t) {
                const unsigned word = hi ? cols[t].mask_hi : cols[t].mask_lo;
                const bool ok = k_ok && (word & bit) != 0u;
                const uint4 q = buf_load_b128(rb, ok ? cols[t].pixoff + lane_unit_off : OOB, soff);
                if constexpr (DT == DT_I8) qb[t].q = q;
                else {
                    qb[t].v[0] = __uint_as_float(q.x); qb[t].v[1] = __uint_as_float(q.y);
                    qb[t].v[2] = __uint_as_float(q.z); qb[t].v[3] = __uint_as_float(q.w);
                }
            }
        } else if constexpr (BL == BL_KVEC) {
            // this lane's unit: filter tap and channel block, then one 16-byte load per column
            const unsigned u = (unsigned) ub + (unsigned) (tid % UPT);
            const unsigned tap = fast_div(u, p.magic_upt, p.pass_upt);
            const unsigned cb = u - tap * (unsigned) p.units_per_tap;
            const unsigned ti = fast_div(tap, p.magic_kw, p.pass_kw);
            const unsigned tj = tap - ti * (unsigned) p.kw;
            const unsigned off = (ti * (unsigned) p.W + tj) * (unsigned) p.pix_stride + cb * 16u;
            const bool k_ok = !CHK || (int) (u * KPU) < klim;
#pragma unroll
            for (int t = 0; t < B_PER_T; ++t) {
                // both validity tests, then a select: no branch in the K loop
                const unsigned word = tap >= 32u ? cols[t].mask_hi : cols[t].mask_lo;
                const bool by_mask = ((word >> (tap & 31u)) & 1u) != 0u;
                const bool by_coord = (unsigned) (cols[t].ih0 + (int) ti) < (unsigned) p.H &&
                                      (unsigned) (cols[t].iw0 + (int) tj) < (unsigned) p.W;
                const bool ok = k_ok & (p.use_tapmask ? by_mask : by_coord);
                const uint4 q = buf_load_b128(rb, ok ? cols[t].pixoff + off : OOB, 0);
                if constexpr (DT == DT_I8) qb[t].q = q;
                else {
                    qb[t].v[0] = __uint_as_float(q.x); qb[t].v[1] = __uint_as_float(q.y);
                    qb[t].v[2] = __uint_as_float(q.z); qb[t].v[3] = __uint_as_float(q.w);
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < B_PER_T; ++t) {
                const int u = ub + b_unit_of(t);
                if constexpr (BL == BL_TAPC) {
                    // the unit's KPU channels share the filter tap: one validity test, channel stride in the scalar offset
                    const unsigned voff = b_voff<BL, CHK>(p, col, bp[t], u);
#pragma unroll
                    for (int e = 0; e < KPU; ++e) qb[t].v[e] = buf_load_f32(rb, voff, bp[t].soff + (unsigned) e * hw4);
                } else {
#pragma unroll
                    for (int e = 0; e < KPU; ++e)
                        qb[t].v[e] = buf_load_f32(rb, b_voff<BL, CHK>(p, col, bp[t * KPU + e], u * KPU + e), bp[t * KPU + e].soff);
                }
            }
        }
    };
    auto stage = [&](int buf, int kt, auto chk, auto slot) __attribute__((always_inline)) {
        constexpr bool CHK = decltype(chk)::value;
        RawUnit<DT> (&qa)[A_PER_T] = qa_[decltype(slot)::value];
        RawUnit<DT> (&qb)[B_PER_T] = qb_[decltype(slot)::value];
#pragma unroll
        for (int t = 0; t < A_PER_T; ++t) {
            const int f = tid + t * THREADS;
            const int ml = f / UPT, ua = f % UPT;
            if constexpr (CHK) clear_a_tail<DT>(qa[t], (u_begin + kt * UPT + a_unit[t]) * KPU, klim);
            if ((A_SLOTS % THREADS == 0) || f < A_SLOTS) lds[buf][ua * A_LD + ml] = pack_unit<DT>(qa[t]);
        }
#pragma unroll
        for (int t = 0; t < B_PER_T; ++t) {
            const int f = tid + t * THREADS;
            if constexpr (LANE_UNITS) lds[buf][A_LDS + (f % UPT) * B_LD + (f / UPT)] = pack_unit<DT>(qb[t]);
            else lds[buf][A_LDS + (f / BN) * B_LD + (f % BN)] = pack_unit<DT>(qb[t]);
        }
    };
    auto read_operand = [&](Operands &o, int buf, int idx) __attribute__((always_inline)) {   // idx-th of the READS LDS reads
        const int s = idx / (TM + TN), t = idx % (TM + TN);
        if (t < TM) o.a[s][t] = lds[buf][(2 * s + lh) * A_LD + wm * (BM / WM) + t * 32 + li];
        else o.b[s][t - TM] = lds[buf][A_LDS + (2 * s + lh) * B_LD + wn * (BN / WN) + (t - TM) * 32 + li];
    };

    // Pipeline.  While the MFMAs of K tile kt run (its operands are already in registers):
    //   step 0            LDS store of tile kt+1 (loaded PF tiles ago), then all global loads of tile kt+1+PF
    //   steps 1..         scalar descriptions of the B loads of the tile after that, spread over the MFMAs
    //   after HALF steps  barrier
    //   second half       LDS reads of tile kt+1 into the other operand set, spread over the MFMAs
    // A wavefront therefore always has matrix work queued while it waits for LDS, the barrier or
    // memory, and a global load has PF tiles of MFMAs to complete.  Past the last tile loads are
    // fully masked (zero, no memory traffic), so the body has no branches.
    Operands op0, op1;
    constexpr std::true_type CHECKED{};
    constexpr std::false_type UNCHECKED{};
#pragma unroll
    for (int i = 0; i < B_ITEMS; ++i) prep_item(0, i);
    issue(0, CHECKED, std::integral_constant<int, 0>{});
    stage(0, 0, CHECKED, std::integral_constant<int, 0>{});
    // tiles 1 .. PF: tile t into set t % PF
    [&]<int... T>(std::integer_sequence<int, T...>) __attribute__((always_inline)) {
        ((void) ([&]() __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < B_ITEMS; ++i) prep_item(T + 1, i);
            issue(T + 1, CHECKED, std::integral_constant<int, (T + 1) % PF>{});
        }()), ...);
    }(std::make_integer_sequence<int, PF>{});
    // the tile's bias rows, behind the first operand loads (nothing waits for them before the K loop is over)
    float bias_row = -0.0f;   // the addend that changes nothing
    float aux_row = 0.0f;
    {
        const unsigned row_off = tid < BM ? (unsigned) (m0 + tid) * 4u : OOB;   // rows beyond M read as zero
        if constexpr (DT == DT_I8) {
            aux_row = buf_load_f32(make_rsrc(p.weight_aux, p.weight_aux ? (unsigned) (p.M * 4) : 0u), row_off, 0);
            bias_row = (float) (int) __builtin_amdgcn_raw_buffer_load_b32(make_rsrc(p.bias32, p.bias32 ? (unsigned) (p.M * 4) : 0u), row_off, 0, 0);
        } else {
            const bool on = p.bias_mode == BIAS_M;
            const float bv = buf_load_f32(make_rsrc(p.bias, on ? (unsigned) (p.M * 4) : 0u), row_off, 0);
            bias_row = on ? bv : -0.0f;
        }
    }
#pragma unroll
    for (int i = 0; i < B_ITEMS; ++i) prep_item(PF + 1, i);   // for the first load of the loop: tile 1 + PF
    __syncthreads();
#pragma unroll
    for (int i = 0; i < READS; ++i) read_operand(op0, 0, i);

    auto body = [&](Operands &cur, Operands &nxt, int kt, auto chk, auto slot) __attribute__((always_inline)) {
        const int nbuf = (kt + 1) & 1;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            const int blk = st / PARTS, part = st % PARTS;
            const int s = blk / (TM * TN), a = (blk / TN) % TM, b = blk % TN;
            Traits<DT>::mma_part(acc[a][b], cur.a[s][a], cur.b[s][b], part);
            if (st == 0) {
                stage(nbuf, kt + 1, chk, slot);
                issue(kt + 1 + PF, chk, slot);
            }
#pragma unroll
            for (int i = 0; i < B_ITEMS; ++i)
                if (STEPS > 1 ? (1 + (i * (STEPS - 1)) / B_ITEMS == st) : true) prep_item(kt + 2 + PF, i);   // one body ahead of its issue
            if (st >= HALF) {
#pragma unroll
                for (int i = 0; i < READS; ++i)
                    if (HALF + (i * (STEPS - HALF)) / READS == st) read_operand(nxt, nbuf, i);
            }
            if (st == HALF - 1) __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // Body kt stores tile kt+1 to LDS (register set (kt+1) % PF) and loads tile kt+1+PF into the same set; the
    // ragged tile k_tiles-1 is therefore touched by bodies k_tiles-2-PF and k_tiles-2.  Everything before runs
    // without per-element tests.  The loop is unrolled over U bodies so that operand sets and register sets are
    // compile-time choices.
    constexpr int U = (PF % 2 == 0) ? PF : 2 * PF;
    auto group = [&](int kt0, auto chk, auto guarded) __attribute__((always_inline)) {
        [&]<int... J>(std::integer_sequence<int, J...>) __attribute__((always_inline)) {
            ((void) ([&]() __attribute__((always_inline)) {
                if (!decltype(guarded)::value || kt0 + J < k_tiles)
                    body(J % 2 == 0 ? op0 : op1, J % 2 == 0 ? op1 : op0, kt0 + J, chk, std::integral_constant<int, (J + 1) % PF>{});
            }()), ...);
        }(std::make_integer_sequence<int, U>{});
    };
    const int n_plain = (ragged ? max(0, k_tiles - 2 - PF) : k_tiles) / U * U;
    int kt = 0;
    for (; kt < n_plain; kt += U) group(kt, UNCHECKED, std::false_type{});
    for (; kt + U <= k_tiles; kt += U) group(kt, CHECKED, std::false_type{});
    if (kt < k_tiles) group(kt, CHECKED, std::true_type{});
    if (tid < BM) {
        if constexpr (DT == DT_I8) {
            s_bias[tid] = __fdiv_rn(aux_row, 127.0f);   // conv.c:1049-1056: the factor is weight_aux / 127, rounded once
            s_bias[BM + tid] = bias_row;
        } else {
            s_bias[tid] = bias_row;
        }
    }
    if constexpr (!PW2) __syncthreads();

    if constexpr (PW2) {
        // the launcher gives this variant one row tile, all of K and no batch: the tile is the whole first product
        static_assert(sizeof(lds) >= 16 * 64 * 16, "the tile as a B operand fits the operand buffers");
        __syncthreads();   // every wavefront is done with the operand buffers (and the bias rows are in place)
        uint4 *tl = &lds[0][0];
        switch (p.ep2.act) {
            case NOT_ACT:
            case RELU6: pw2_stage<EPI_NONE, RES>(p, acc[0][0], tl, s_bias, n0, wm, wn, li, lh); break;
            case RELU: pw2_stage<EPI_RELU, RES>(p, acc[0][0], tl, s_bias, n0, wm, wn, li, lh); break;
            case CLIP: pw2_stage<EPI_CLIP, RES>(p, acc[0][0], tl, s_bias, n0, wm, wn, li, lh); break;
            default: pw2_stage<EPI_GENERIC, RES>(p, acc[0][0], tl, s_bias, n0, wm, wn, li, lh); break;
        }
        return;
    }
    const int m_wave = m0 + wm * (BM / WM), n_wave = n0 + wn * (BN / WN);
    if (p.partial && !whole_k) {
        if (DT == DT_I8 || !p.arrive) {   // a finishing launch adds the slices up
            write_partial<TM, TN, false>(p, acc, slice * gridDim.z + batch, m_wave, n_wave, li, lh);
            return;
        }
        write_partial<TM, TN, true>(p, acc, slice * gridDim.z + batch, m_wave, n_wave, li, lh);
        // The reduction inside the launch.  Partial sums and counters live in uncached memory and are stored and
        // loaded with system scope (AUX_SYSTEM_SCOPE): once this workgroup's stores are acknowledged (written
        // through, vmcnt(0)) it counts itself in with a device-scope atomic, and the last of a tile's slices to arrive
        // adds all of them up in slice order (the order of the finishing kernel: the same bits) with loads that
        // bypass the caches, and goes on to the epilogue as if it had computed the whole tile.  Nobody waits for
        // anybody, so the launch cannot hang; the counter is back at zero for the next launch.
        __shared__ int s_last;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            int *ctr = p.arrive + lid + batch * (int) gridDim.x;
            const int old = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int last = old == p.n_slices - 1;
            if (last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = last;
        }
        __syncthreads();
        if (!s_last) return;
        if constexpr (DT != DT_I8) {
            const int width = p.N - p.part_begin;
            const bool m_edge = m_wave + TM * 32 > p.M;
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;
            for (int s = 0; s < p.n_slices; ++s) {
                const rsrc_t rp = make_rsrc(reinterpret_cast<const char *>(p.partial) +
                                            (size_t) (s * gridDim.z + batch) * p.M * width * 4, RSRC_RANGE);
                // half a 32x32 block at a time: eight loads in flight, not sixteen per block of the tile, which would
                // cost the kernels registers and with them occupancy
#pragma unroll
                for (int a = 0; a < TM; ++a)
#pragma unroll
                    for (int b = 0; b < TN; ++b) {
                        const int n = n_wave + b * 32 + li;
                        const unsigned cv = n < p.N ? (unsigned) (n - p.part_begin + 4 * lh * width) * 4u : OOB;
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            float v[8];
#pragma unroll
                            for (int q = 0; q < 8; ++q) {
                                const int r = 8 * h + q;
                                const int m_uni = m_wave + a * 32 + 8 * (r / 4) + (r % 4);
                                const bool row_ok = !m_edge || m_uni + 4 * lh < p.M;
                                v[q] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(
                                    rp, row_ok ? cv : OOB, (unsigned) m_uni * (unsigned) width * 4u, AUX_SYSTEM_SCOPE));
                            }
#pragma unroll
                            for (int q = 0; q < 8; ++q) acc[a][b][8 * h + q] = __fadd_rn(acc[a][b][8 * h + q], v[q]);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
            }
        }
    }
    if constexpr (DT == DT_I8) {
        // int8 NHWC output without the raw-accumulator copy: 128-bit stores through LDS (batch is 1 on this path)
        if (p.out_s8 && p.out_mode == OUT_PLAIN && p.c_stride_m == 1 && !p.acc_out) {
            static_assert(sizeof(lds) >= (size_t) BN * (BM + 16), "output staging fits the operand buffers");
            constexpr bool QL = sizeof(lds) >= (size_t) BN * (BM + 16) + 8192;   // room for the quantised activation table
            unsigned char *stage = reinterpret_cast<unsigned char *>(&lds[0][0]);
            __syncthreads();   // every wavefront is done with the operand buffers
            switch (p.ep.act) {
                case NOT_ACT:
                case RELU6: write_tile_nhwc_s8<EPI_NONE, BM, BN, TM, TN, QL>(p, acc, stage, m0, n0, m_wave, n_wave, li, lh, tid, s_bias); break;
                case RELU: write_tile_nhwc_s8<EPI_RELU, BM, BN, TM, TN, QL>(p, acc, stage, m0, n0, m_wave, n_wave, li, lh, tid, s_bias); break;
                case CLIP: write_tile_nhwc_s8<EPI_CLIP, BM, BN, TM, TN, QL>(p, acc, stage, m0, n0, m_wave, n_wave, li, lh, tid, s_bias); break;
                case SILU:
                case ONHIP_ACT_GELU_LUT: write_tile_nhwc_s8<EPI_LUT, BM, BN, TM, TN, QL>(p, acc, stage, m0, n0, m_wave, n_wave, li, lh, tid, s_bias); break;
                default: write_tile_nhwc_s8<EPI_GENERIC, BM, BN, TM, TN, QL>(p, acc, stage, m0, n0, m_wave, n_wave, li, lh, tid, s_bias); break;
            }
            return;
        }
    }
    switch (p.ep.act) {
        case NOT_ACT:
        case RELU6: write_tile<DT, EPI_NONE, TM, TN, RES, BIAS_LDS>(p, acc, batch, m_wave, n_wave, li, lh, s_bias + wm * (BM / WM), s_bias + BM + wm * (BM / WM)); break;
        case RELU: write_tile<DT, EPI_RELU, TM, TN, RES, BIAS_LDS>(p, acc, batch, m_wave, n_wave, li, lh, s_bias + wm * (BM / WM), s_bias + BM + wm * (BM / WM)); break;
        case CLIP: write_tile<DT, EPI_CLIP, TM, TN, RES, BIAS_LDS>(p, acc, batch, m_wave, n_wave, li, lh, s_bias + wm * (BM / WM), s_bias + BM + wm * (BM / WM)); break;
        case SILU:
        case ONHIP_ACT_GELU_LUT: write_tile<DT, EPI_LUT, TM, TN, RES, BIAS_LDS>(p, acc, batch, m_wave, n_wave, li, lh, s_bias + wm * (BM / WM), s_bias + BM + wm * (BM / WM)); break;
        default: write_tile<DT, EPI_GENERIC, TM, TN, RES, BIAS_LDS>(p, acc, batch, m_wave, n_wave, li, lh, s_bias + wm * (BM / WM), s_bias + BM + wm * (BM / WM)); break;
    }
}

// sums the split-K partials in slice order and applies the epilogue: one thread per output element; a
// workgroup is 64 columns x 4 rows (one wavefront per row) and the grid (column blocks, row blocks, batch),
// so no index has to be divided
template <bool IS_INT>
__global__ __launch_bounds__(256) void splitk_finish_kernel(const IgemmParams p, int split, int batches) {
    const int n = p.part_begin + blockIdx.x * 64 + threadIdx.x;
    const int m = blockIdx.y * 4 + threadIdx.y, batch = blockIdx.z;
    if (n >= p.N || m >= p.M) return;
    const int width = p.N - p.part_begin;
    const size_t slice = (size_t) batches * p.M * width;                  // elements per K slice
    const size_t idx = ((size_t) batch * p.M + m) * width + (n - p.part_begin);
    const size_t off4 = (size_t) batch * p.c_batch_stride + (size_t) m * p.c_stride_m + out_col_offset(p, n, 1);
    char *cbase = reinterpret_cast<char *>(p.C);
    if constexpr (IS_INT) {
        // four loads in flight per step: the slices are a cache-line stride apart and one load at a time would
        // pay the memory latency `split` times over
        const int *part = reinterpret_cast<const int *>(p.partial) + idx;
        int acc = 0, s = 0;
        for (; s + 4 <= split; s += 4) {
            const int a0 = part[(size_t) s * slice], a1 = part[(size_t) (s + 1) * slice];
            const int a2 = part[(size_t) (s + 2) * slice], a3 = part[(size_t) (s + 3) * slice];
            acc += a0 + a1 + a2 + a3;
        }
        for (; s < split; ++s) acc += part[(size_t) s * slice];
        if (p.acc_out) p.acc_out[off4] = acc;
        float f = __fmul_rn((float) acc, p.in_scale);
        if (p.bias32) f = __fadd_rn(f, (float) p.bias32[m]);
        const float y = apply_act(__fmul_rn(f, __fdiv_rn(p.weight_aux[m], 127.0f)), p.ep);
        if (p.out_s8) reinterpret_cast<int8_t *>(cbase)[off4] = (int8_t) requant_s8(y, p.out_inv_scale);
        else reinterpret_cast<float *>(cbase)[off4] = y;
    } else {
        const float *part = p.partial + idx;
        float acc = 0.0f;
        int s = 0;
        // the loads of up to sixteen slices are in flight together (a small problem is one memory round trip, not one
        // per group of four); the sums are added one after the other in slice order whatever the grouping
        for (; s + 16 <= split; s += 16) {
            float a[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) a[i] = part[(size_t) (s + i) * slice];
#pragma unroll
            for (int i = 0; i < 16; ++i) acc = __fadd_rn(acc, a[i]);
        }
        if (s + 8 <= split) {
            float a[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) a[i] = part[(size_t) (s + i) * slice];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = __fadd_rn(acc, a[i]);
            s += 8;
        }
        if (s + 4 <= split) {
            const float a0 = part[(size_t) s * slice], a1 = part[(size_t) (s + 1) * slice];
            const float a2 = part[(size_t) (s + 2) * slice], a3 = part[(size_t) (s + 3) * slice];
            acc = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(acc, a0), a1), a2), a3);
            s += 4;
        }
        if (s < split) {   // up to three left: requested together as well
            const float a0 = part[(size_t) s * slice];
            const float a1 = s + 1 < split ? part[(size_t) (s + 1) * slice] : 0.0f;
            const float a2 = s + 2 < split ? part[(size_t) (s + 2) * slice] : 0.0f;
            acc = __fadd_rn(acc, a0);
            if (s + 1 < split) acc = __fadd_rn(acc, a1);
            if (s + 2 < split) acc = __fadd_rn(acc, a2);
        }
        if (p.bias_mode == BIAS_M) acc = __fadd_rn(acc, p.bias[m]);
        else if (p.bias_mode == BIAS_N) acc = __fadd_rn(acc, p.bias[n]);
        float y = apply_act(acc, p.ep);
        if (p.res) y = add_res(y, p.res[off4], p.res_relu, (unsigned) off4, p.res_body);
        reinterpret_cast<float *>(cbase)[off4] = y;
    }
}

// ---- launch ------------------------------------------------------------------------------------------
template <int DT, int BL, int BM, int BN, int WM, int WN, int PF = 1, bool RES = false>
static int launch_one(const IgemmLaunch &cfg, const IgemmParams &p_in, hipStream_t stream) {
    IgemmParams p = p_in;
    const int tiles_m = (p.M + BM - 1) / BM;
    const int tiles = tiles_m * ((p.N + BN - 1) / BN);
    p.div_ohw = make_div31((unsigned) (p.OHW > 0 ? p.OHW : 1));
    p.div_ow = make_div31((unsigned) (p.OW > 0 ? p.OW : 1));
    p.div_tiles_m = make_div31((unsigned) tiles_m);
    p.div_tiles_n = make_div31((unsigned) ((p.N + BN - 1) / BN));
    dim3 grid(tiles, cfg.split, cfg.batch);
    if (p.dp_tiles > 0) {   // whole tiles first, then the K slices of the leftover tiles (igemm_kernel)
        if (cfg.batch != 1 || p.dp_tiles + p.tail_tiles != tiles || !p.partial || p.part_begin != p.dp_tiles / tiles_m * BN)
            return set_error(ONHIP_ERR_ARG, "igemm: inconsistent leftover-tile launch");
        grid = dim3(p.dp_tiles + p.tail_tiles * cfg.split, 1, 1);
    }
    if (RES != (p.res != nullptr)) return set_error(ONHIP_ERR_ARG, "igemm: residual operand and kernel variant do not match");
    hipLaunchKernelGGL((igemm_kernel<DT, BL, BM, BN, WM, WN, PF, RES>), grid, dim3(THREADS), 0, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    if (p.partial && !p.arrive) {
        if (p.M > 4 * 65535 || cfg.batch > 65535)
            return set_error(ONHIP_ERR_ARG, "igemm: split-K with %d rows, %d batches", p.M, cfg.batch);
        const dim3 fgrid((p.N - p.part_begin + 63) / 64, (p.M + 3) / 4, cfg.batch);
        if (DT == DT_I8)
            hipLaunchKernelGGL((splitk_finish_kernel<true>), fgrid, dim3(64, 4), 0, stream, p, cfg.split, cfg.batch);
        else
            hipLaunchKernelGGL((splitk_finish_kernel<false>), fgrid, dim3(64, 4), 0, stream, p, cfg.split, cfg.batch);
        ONHIP_CHECK_HIP(hipGetLastError());
    }
    return ONHIP_OK;
}

template <int DT, int BL, int PF = 1, bool RES = false>
int launch_tile(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    const int key = cfg.bm * 1000 + cfg.bn;
    switch (key) {
        case 128128: return launch_one<DT, BL, 128, 128, 2, 2, (PF > 2 ? 2 : PF), RES>(cfg, p, stream);
        case 64128: return launch_one<DT, BL, 64, 128, 2, 2, PF, RES>(cfg, p, stream);
        case 64064: return launch_one<DT, BL, 64, 64, 2, 2, PF, RES>(cfg, p, stream);
        case 32128: return launch_one<DT, BL, 32, 128, 1, 4, PF, RES>(cfg, p, stream);
        default: return set_error(ONHIP_ERR_ARG, "igemm: no kernel for tile %dx%d", cfg.bm, cfg.bn);
    }
}

}  // namespace onhip
