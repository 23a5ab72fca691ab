// Internal declarations shared by the gfx950 kernels and the C ABI layer.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/onenew_hip.h"

namespace onhip {

// ---- error plumbing ---------------------------------------------------------------------------
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
#define ONHIP_CHECK_HIP(expr)                                                                     \
    do {                                                                                          \
        hipError_t e_ = (expr);                                                                   \
        if (e_ != hipSuccess)                                                                     \
            return ::onhip::set_error(ONHIP_ERR_RUNTIME, "%s failed: %s (%s:%d)", #expr,          \
                                      hipGetErrorString(e_), __FILE__, __LINE__);                 \
    } while (0)

// ---- epilogue description, common to every kernel ---------------------------------------------------
struct Epilogue {
    int act;                 // ACT_TYPE_E
    float clip_min, clip_max;
    float leaky_alpha;
    float hs_alpha, hs_beta;
    const float *lut;        // 8192-entry table for SILU (conv) / GELU (matmul), or nullptr
    // int8 outputs only: the same table already passed through the output quantiser (one byte per entry), so that the
    // store gathers a byte from 8 KiB instead of a float from 32 KiB and quantises it; nullptr = use `lut`
    const signed char *qlut;
};

#define ONHIP_ACT_GELU_LUT 100  // internal: table GELU of device/x86/Gelu/gelu.c, matmul epilogue only

// Activation with the rounding points of device/x86/Conv/conv.c:1216-1304 (no contraction).
__device__ __forceinline__ float apply_act(float v, const Epilogue &e) {
    switch (e.act) {
        case RELU:
            return v > 0.0f ? v : 0.0f;
        case SILU:
        case ONHIP_ACT_GELU_LUT: {
            if (v < -8.0f) return 0.0f;
            if (v >= 8.0f) return v;
            int idx = (int) __fmul_rn(__fadd_rn(v, 8.0f), 512.0f);
            // v just below 8 rounds v + 8 up to 16: the reference reads one past the table there
            idx = idx > 8191 ? 8191 : idx;
            return e.lut[idx];
        }
        case CLIP: {
            float t = v > e.clip_min ? v : e.clip_min;
            return t < e.clip_max ? t : e.clip_max;
        }
        case LEAKYRELU:
            return v > 0.0f ? v : __fmul_rn(e.leaky_alpha, v);
        case HARDSILU: {
            float t = __fadd_rn(__fmul_rn(e.hs_alpha, v), e.hs_beta);
            t = t > 0.0f ? t : 0.0f;
            t = t < 1.0f ? t : 1.0f;
            return __fmul_rn(v, t);
        }
        default:
            return v;  // NOT_ACT and RELU6 (no branch in the reference)
    }
}

// The activation kind as a template parameter, so the common ones cost one or two instructions and no
// branch in an unrolled epilogue; EPI_GENERIC falls back to apply_act.
enum { EPI_NONE = 0, EPI_RELU = 1, EPI_CLIP = 2, EPI_GENERIC = 3, EPI_LUT = 4 };

inline int epi_of_act(int act) {
    return (act == NOT_ACT || act == RELU6) ? EPI_NONE : act == RELU ? EPI_RELU : act == CLIP ? EPI_CLIP : EPI_GENERIC;
}

template <int EPI>
__device__ __forceinline__ float act_fast(float v, const Epilogue &e) {
    if constexpr (EPI == EPI_NONE) return v;
    else if constexpr (EPI == EPI_RELU) return v > 0.0f ? v : 0.0f;
    else if constexpr (EPI == EPI_CLIP) {
        const float t = v > e.clip_min ? v : e.clip_min;
        return t < e.clip_max ? t : e.clip_max;
    } else if constexpr (EPI == EPI_LUT) {
        // the table activations of apply_act without branches: the load is unconditional (index clamped into
        // the table) and the two outer ranges are selected afterwards
        int idx = (int) __fmul_rn(__fadd_rn(v, 8.0f), 512.0f);
        idx = idx < 0 ? 0 : idx > 8191 ? 8191 : idx;
        const float l = e.lut[idx];
        return v < -8.0f ? 0.0f : v >= 8.0f ? v : l;
    } else return apply_act(v, e);
}

// relu.c:27-52: the first n - n % 32 elements go through _mm256_max_ps(0, x), which is "0 > x ? 0 : x" (a NaN or a
// negative zero comes back unchanged); the rest through "x > 0 ? x : 0"
__device__ __forceinline__ float relu_body(float v) { return 0.0f > v ? 0.0f : v; }
__device__ __forceinline__ float relu_tail(float v) { return v > 0.0f ? v : 0.0f; }
// the Add and the Relu after a convolution, applied to one finished element at index `elem` of the output tensor
__device__ __forceinline__ float add_res(float v, float r, int relu, unsigned elem, unsigned body) {
    v = __fadd_rn(v, r);
    const float vb = relu_body(v), vt = relu_tail(v);
    return relu ? (elem < body ? vb : vt) : v;
}

// (int) roundf(t), ties away from zero, for |t| <= 128.5 in three instructions: adding the largest float below one half
// with t's sign and truncating gives the same integer for every such float (checked exhaustively on the CPU, all
// 2.2e9 of them: a tie k + 0.5 lands within a quarter ulp below k + 1 and rounds up to it, nothing else crosses an
// integer); roundf itself is a dozen instructions
__device__ __forceinline__ int round_half_away_small(float t) {
    const float half = __uint_as_float((__float_as_uint(t) & 0x80000000u) | 0x3effffffu);
    return (int) __fadd_rn(t, half);
}

// activation quantiser of conv.c:961-973: t = x * (1/scale), clamp, roundf (ties away from zero)
__device__ __forceinline__ int quant_s8(float x, float inv_scale) {
    float t = __fmul_rn(x, inv_scale);
    t = (t < -128.0f) ? -128.0f : (t > 127.0f) ? 127.0f : t;
    return round_half_away_small(t);
}

// ---- implicit-GEMM kernel family (igemm.hip) ---------------------------------------------------------
//
// C[M, N] = A[M, K] * B[K, N] on MFMA 32x32 tiles.  A rows are K-contiguous (weights, or the left
// MatMul operand).  B is produced on the fly by one of two loaders.

enum { BL_GATHER = 0,  // element gather from NCHW activations (implicit im2col), any filter / stride / padding
       BL_KVEC = 1,    // 16-byte vectors along K from NHWC int8 activations
       BL_PLAIN = 2,   // 1x1 filter without padding, or a row-major [K, N] matrix: no tap arithmetic
       BL_TAPC = 3,    // NCHW activations against tap-major packed weights: K = (tap, channel), one tap per unit
       BL_KVEC_TAP = 4 };  // BL_KVEC whose K tiles never straddle a filter tap (units per tap a multiple of the
                           // tile, at most 64 taps): tap arithmetic is scalar and the K loop has no branches

enum { OUT_CONV = 0,   // n = img * OHW + pix  ->  img * c_img_stride + m * c_stride_m + pix
       OUT_PLAIN = 1 };// m * c_stride_m + n * c_stride_n

enum { BIAS_NONE = 0, BIAS_M = 1, BIAS_N = 2 };

// floor(x / d) for 0 <= x < 2^31 as (mulhi(x, magic) >> shift) + (x & pass): with L = ceil(log2 d),
// magic = floor(2^(31+L) / d) + 1 and shift = L - 1 the quotient is exact; d == 1 is magic 0, pass ~0.
struct Div31 {
    unsigned magic, shift, pass;
};
inline Div31 make_div31(unsigned d) {
    Div31 r = {0u, 0u, 0xFFFFFFFFu};
    if (d <= 1) return r;
    unsigned L = 0;
    while ((1ull << L) < d) ++L;
    r.magic = (unsigned) ((1ull << (31 + L)) / d) + 1u;
    r.shift = L - 1;
    r.pass = 0;
    return r;
}

struct IgemmParams {
    int M, N, K;              // K counts real reduction elements (gather) or padded units*kpu (kvec)
    int k_units;               // 16-byte units along K (multiple of 2 per MFMA step is NOT required)
    int k_split_units;         // units handled by one blockIdx.y slice (split-K); == k_units if unsplit
    int part_begin;            // first column the split-K partial sums cover (0 unless only leftover tiles are split)
    int dp_tiles, tail_tiles;  // dp_tiles > 0: that many workgroups take whole tiles, the tail_tiles tiles after them are
                               // cut into K slices (see igemm_kernel)
    // A
    const void *A;
    long long a_batch_stride;  // elements; 0 = shared
    int lda;                   // elements between rows
    // B
    const void *B;
    long long b_batch_stride;  // elements
    // gather geometry (BL_GATHER)
    int H, W, OW, OHW, HW;
    int kh, kw, khkw, sh, sw, pt, pl;
    unsigned magic_khkw, magic_kw;   // multiply-high constants for / (kh*kw) and / kw
    unsigned pass_khkw, pass_kw;     // ~0u when the divisor is 1 (quotient = dividend), else 0
    long long b_img_stride;    // Cin * H * W
    long long b_shift_bytes;   // the B buffer descriptor starts this many bytes before the tensor (pad rows/cols)
    long long a_slice_bytes, b_slice_bytes, c_slice_bytes;  // extent one batch slice can address (< 2 GiB)
    // vector geometry (BL_KVEC)
    int units_per_tap;         // units per filter tap (Cp / 16 for NHWC int8); k_units for a plain matrix
    int tap_spans_pixels;      // K-vector loaders: a tap's units_per_tap * 16 bytes of K start at the tap's pixel and run on
                               // into the pixels after it in the row (pix_stride is then less than that): first layers stored
                               // with few channels per pixel, a filter row being one tap
    unsigned magic_upt, pass_upt;
    int use_tapmask;           // kh*kw <= 64: per-lane tap validity is a 64-bit mask built once per tile
    int pix_stride;            // bytes between consecutive n ("pixels"): Cp, or ldb * elem
    // C
    void *C;
    long long c_batch_stride, c_img_stride, c_stride_m, c_stride_n;
    int out_mode;
    // epilogue
    const float *bias;
    int bias_mode;
    Epilogue ep;
    // optional second pass of a residual block folded into the store (fp32 outputs): after the activation the
    // element of `res` at the same place as in C is added (add.c), then, with res_relu, relu.c's rule is applied:
    // the first res_body elements of the tensor go through its vector body, the rest through its scalar tail
    const float *res;
    int res_relu;
    unsigned res_body;
    // W8A32
    float in_scale;            // activation scale s
    const float *weight_aux;   // per output channel max|w|
    const int32_t *bias32;
    int32_t *acc_out;          // optional raw accumulators, same addressing as C
    int out_s8;
    float out_inv_scale;       // 1.0f / output_scale
    // 16-bit storage (bf16 / fp16 operands read as 16-byte vectors): out_h16 != 0 stores the result in the operands'
    // type, NHWC with a channel pitch of c_stride_n; res16, when not null, is a tensor of that type and layout added on
    // the way out (followed by a ReLU when res_relu is set)
    int out_h16;
    const void *res16;
    // int8 kernels with a residual operand: when not null, the fp32 result (after the Add and the Relu) is ALSO stored
    // here as int8 NHWC, element (pixel n, channel m) at n * twin_pitch + m, quantised with twin_inv_scale: the form the
    // int8 convolutions that read the tensor would make of it (M a multiple of 16, so no padding channels exist)
    int8_t *twin;
    int twin_pitch;
    float twin_inv_scale;
    // split-K workspace: partial sums [split][M][N] fp32 (nullptr when unsplit)
    float *partial;
    // reduction inside the launch by the last slice of a tile to arrive: one counter per tile (uncached memory, like
    // `partial` then) and the number of slices; nullptr = a finishing launch adds the slices up
    int *arrive;
    int n_slices;
    // exact division of any x < 2^31 by OHW, OW and the number of row tiles (filled in by the launcher)
    Div31 div_ohw, div_ow, div_tiles_m;
    // n_fast != 0 (tiled kernel, launches without leftover-tile slices): tiles are numbered along N first, so that an XCD's
    // run of tiles covers a band of rows of A against every column block of B.  For products whose A (many rows) does not
    // fit an L2 while B (a weight matrix) does: each XCD then reads its rows of A once instead of all of A per column block.
    int n_fast;
    Div31 div_tiles_n;
    // a second, 1x1 product over the finished tile (igemm_kernel's PW2 variant, one row tile: M <= 64): the M rows of the
    // first product, with `bias` and `ep` applied, are the reduction of w2 ([m2][M], in pack_pw2_launch's order).  C, the
    // c_* strides and res then describe the m2-row result, bias2 and ep2 its epilogue; the M-row tensor between the two
    // never exists
    const float *w2;
    const float *bias2;
    int m2;
    Epilogue ep2;
};

enum { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2, DT_I8 = 3 };

struct IgemmLaunch {
    int dtype;      // DT_*
    int bl;         // BL_*
    int bm, bn;     // tile
    int batch;      // grid.z
    int split;      // grid.y
    int ring;       // direct-to-LDS kernel: 0 = ring of stage buffers within 64 KiB of LDS, 1 = the long ring
};

int igemm_launch(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);
// fp32 convolution followed by a 1x1 convolution over its result in one launch (igemm_f32_pw.hip): p as for the tap-major
// packed loader with M <= 64 rows, plus w2 / bias2 / m2 / ep2
int igemm_launch_f32_pw(const IgemmParams &p, hipStream_t stream);
// fp32 kernel for plain problems with B rows contiguous along N (igemm_rowb.hip): tiles 64x128, 128x128, 64x256
bool rowb_f32_ok(const IgemmLaunch &cfg, const IgemmParams &p);
int rowb_f32_launch(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);
// int8 kernel with operand tiles loaded from global memory straight into LDS (igemm_dma.hip): NHWC int8 activations whose
// padded channel count is a multiple of 64, tiles 128x128, 128x64, 64x128, 64x64, no split-K
bool dma_ok(const IgemmLaunch &cfg, const IgemmParams &p);
bool dma_tile_ok(int bm, int bn);
int dma_launch(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);

// ---- other kernels -------------------------------------------------------------------------------------
int depthwise_f32_launch(const onhip_conv_desc_t &d, int OH, int OW, const float *x, const float *w,
                         const float *bias, const Epilogue &ep, float *y, hipStream_t stream);
int depthwise_w8a32_launch(const onhip_conv_desc_t &d, int OH, int OW, const float *x, const int8_t *w8,
                           const int32_t *bias32, const float *weight_aux, const Epilogue &ep, void *y,
                           int32_t *acc32, hipStream_t stream);
// dw_s8.hip: depthwise convolution on int8 NHWC activations (the chain form's twin of depthwise_w8a32_launch)
bool dw_s8_ok(const onhip_conv_desc_t &d, int OH, int OW);
int dw_s8_launch(const onhip_conv_desc_t &d, int OH, int OW, const int8_t *xq, const int8_t *w8, const int32_t *bias32,
                 const float *weight_aux, const Epilogue &ep, void *y, hipStream_t stream);
int quantize_nhwc_launch(const float *x, int n, int c, int h, int w, int cp, float inv_scale, int8_t *q,
                         hipStream_t stream);
int pack_wf32_launch(const float *w, int cout, int cin, int khkw, int cp, float *packed, hipStream_t stream);
int pack_pw2_launch(const float *w, int m2, int cmid, float *packed, hipStream_t stream);   // ceil(m2 / 64) * 16 KiB
int build_qlut_launch(const float *lut, float out_inv_scale, signed char *qlut, hipStream_t stream);
int forget_quantised_tables(const void *base, size_t bytes);   // api.hip: the cache of tables behind an output quantiser
// i8patch.hip: int8 NHWC 3x3 convolutions with few channels from an LDS-resident input patch
struct IgemmParams;
bool i8patch_ok(const IgemmParams &p, bool any_shape);
int i8patch_launch(const IgemmParams &p, hipStream_t stream);
bool i8direct_ok(const IgemmParams &p);
int i8direct_launch(const IgemmParams &p, hipStream_t stream);

// irblock.hip: 1x1 expansion -> depthwise 3x3 -> 1x1 projection in one launch
int irblock_pack_launch(const float *w_exp, const float *w_proj, int cin, int ce, int co, float *packed, hipStream_t stream);
int irblock_band_rows(const onhip_conv_desc_t &dw, int OH, int OW, int cin);
bool irblock_cin_ok(int cin);
int irblock_f32_launch(const onhip_conv_desc_t &ex, const onhip_conv_desc_t &dw, const onhip_conv_desc_t &pw, int OH, int OW, const float *x,
                       const float *packed, const float *exp_b, const float *dw_w, const float *dw_b, const float *pw_b, const float *res,
                       const Epilogue &exp_ep, const Epilogue &dw_ep, const Epilogue &pw_ep, float *y, hipStream_t stream);

// stem.hip: first-layer convolutions (three input channels) from an LDS patch
bool stem_f32_shape(const onhip_conv_desc_t &d);
bool stem_f32_ok(const onhip_conv_desc_t &d, int OH, int OW);
int stem_pack_launch(const onhip_conv_desc_t &d, const float *w, float *packed, hipStream_t stream);
int stem_f32_launch(const onhip_conv_desc_t &d, int OH, int OW, const float *x, const float *w, int packed, const float *bias,
                    const Epilogue &ep, float *y, hipStream_t stream);
// attention.hip
int attention_f32_launch(const onhip_attention_desc_t &d, const float *q, const float *k, const float *v, float *out,
                         hipStream_t stream);
int attention_h16_launch(int dt, const onhip_attention_desc_t &d, const void *q, const void *k, const void *v, void *out,
                         hipStream_t stream);
// 16-bit storage (h16.hip): dt is DT_BF16 or DT_F16
int pack_w16_launch(int dt, const float *w, long long rows, int cin, int taps, int cp, long long s_row, long long s_ch,
                    long long s_tap, void *packed, hipStream_t stream);
int first_from_nchw_launch(int dt, const float *x, int n, int c, int h, int w, int wp, int cpp, int pad_l, void *y, hipStream_t stream);
int first_pack_w16_launch(int dt, const float *w, int cout, int cin, int kh, int kw, int cpp, void *packed, hipStream_t stream);
int nchw_to_nhwc16_launch(int dt, const float *x, int n, int c, int h, int w, int cp, void *y, hipStream_t stream);
int nhwc16_to_nchw_launch(int dt, const void *x, int n, int c, int h, int w, int cp, float *y, hipStream_t stream);
int rows_to_h16_launch(int dt, const float *x, long long rows, int k, int kp, void *y, hipStream_t stream);
int rows_from_h16_launch(int dt, const void *x, long long rows, int k, int kp, float *y, hipStream_t stream);
int pack_w8_launch(const int8_t *w8, int cout, int cin, int kh, int kw, int cp, int k_units, int8_t *packed,
                   hipStream_t stream);
int gemm_nt_launch(int m, int k, int n, const float *a, const float *w, const float *bias, float *out,
                   hipStream_t stream);
int copy_f32_launch(const float *src, float *dst, long long n, hipStream_t stream);

}  // namespace onhip
