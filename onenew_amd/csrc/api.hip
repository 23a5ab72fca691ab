// Kernel-level C ABI (include/onenew_hip.h): argument checks, geometry set-up and kernel choice.
// Device pointers in, asynchronous launches on the caller's stream, no allocation except the
// lazily grown split-K scratch.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "onhip_internal.hpp"

namespace onhip {

static thread_local char g_err[512] = "";

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static unsigned magic_for(unsigned d) { return d <= 1 ? 0u : (unsigned) (0x100000000ULL / d) + 1u; }
static unsigned pass_for(unsigned d) { return d <= 1 ? 0xFFFFFFFFu : 0u; }

static Epilogue make_epilogue(const onhip_conv_desc_t &d, const float *lut) {
    Epilogue e;
    // conv.c:18-27: a convolution without bias returns before the activation
    e.act = d.has_bias ? d.act_type : NOT_ACT;
    e.clip_min = d.clip_min;
    e.clip_max = d.clip_max;
    e.leaky_alpha = d.leaky_relu_alpha;
    e.hs_alpha = d.hard_sigmoid_alpha;
    e.hs_beta = d.hard_sigmoid_beta;
    e.lut = lut;
    return e;
}

static int check_conv(const onhip_conv_desc_t *d, int32_t *oh, int32_t *ow) {
    if (!d) return set_error(ONHIP_ERR_ARG, "conv: null descriptor");
    if (d->n < 1 || d->cin < 1 || d->cout < 1 || d->h < 1 || d->w < 1 || d->kh < 1 || d->kw < 1 || d->stride_h < 1 ||
        d->stride_w < 1 || d->pad_t < 0 || d->pad_l < 0 || d->pad_b < 0 || d->pad_r < 0)
        return set_error(ONHIP_ERR_ARG, "conv: bad geometry n=%d cin=%d cout=%d %dx%d k=%dx%d s=%d,%d", d->n, d->cin,
                         d->cout, d->h, d->w, d->kh, d->kw, d->stride_h, d->stride_w);
    const int hh = d->h + d->pad_t + d->pad_b - d->kh, ww = d->w + d->pad_l + d->pad_r - d->kw;
    if (hh < 0 || ww < 0) return set_error(ONHIP_ERR_ARG, "conv: kernel larger than padded input");
    *oh = hh / d->stride_h + 1;
    *ow = ww / d->stride_w + 1;
    if (d->group != 1 && d->cin != d->cout)
        return set_error(ONHIP_ERR_ARG, "conv: group=%d needs cin == cout (depthwise, multiplier 1)", d->group);
    if (d->group != 1 && !d->has_bias)
        return set_error(ONHIP_ERR_ARG, "conv: depthwise without bias is not defined by the reference");
    if (d->pad_t >= d->kh || d->pad_b >= d->kh || d->pad_l >= d->kw || d->pad_r >= d->kw) {
        // allowed, just unusual (1x1 with padding): nothing to reject
    }
    const long long in_elems = (long long) d->n * d->cin * d->h * d->w;
    const long long out_elems = (long long) d->n * d->cout * *oh * *ow;
    if (in_elems >= (1LL << 31) || out_elems >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "conv: tensors of 2^31 elements or more are not supported");
    if (d->has_bias && d->act_type != NOT_ACT && d->act_type != RELU && d->act_type != RELU6 && d->act_type != SILU &&
        d->act_type != CLIP && d->act_type != HARDSILU && d->act_type != LEAKYRELU)
        return set_error(ONHIP_ERR_ARG, "conv: unknown act_type %d", d->act_type);
    return ONHIP_OK;
}

// ---- split-K scratch: one lazily grown device buffer per process ---------------------------------
static std::mutex g_scratch_mu;
static void *g_scratch = nullptr;
static size_t g_scratch_bytes = 0;

static int get_scratch(size_t bytes, void **out) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (bytes > g_scratch_bytes) {
        if (g_scratch) {
            ONHIP_CHECK_HIP(hipDeviceSynchronize());
            ONHIP_CHECK_HIP(hipFree(g_scratch));
            g_scratch = nullptr;
            g_scratch_bytes = 0;
        }
        const size_t want = bytes < (64u << 20) ? (64u << 20) : bytes;
        ONHIP_CHECK_HIP(hipMalloc(&g_scratch, want));
        g_scratch_bytes = want;
    }
    *out = g_scratch;
    return ONHIP_OK;
}

// Split K when the tile grid cannot occupy the chip: aim for about two workgroups per CU.
static int plan_split(IgemmLaunch &cfg, IgemmParams &p) {
    const long long tiles = (long long) ((p.M + cfg.bm - 1) / cfg.bm) * ((p.N + cfg.bn - 1) / cfg.bn) * cfg.batch;
    cfg.split = 1;
    p.k_split_units = p.k_units;
    p.partial = nullptr;
    const int k_tiles = (p.k_units + 3) / 4;
    if (tiles >= 192 || k_tiles < 8) return ONHIP_OK;
    int split = (int) ((512 + tiles - 1) / tiles);
    if (split > k_tiles / 4) split = k_tiles / 4;
    if (split > 32) split = 32;
    if (split < 2) return ONHIP_OK;
    const int tiles_per = (k_tiles + split - 1) / split;
    split = (k_tiles + tiles_per - 1) / tiles_per;
    void *buf = nullptr;
    const size_t bytes = (size_t) split * cfg.batch * p.M * p.N * 4;
    if (bytes > (512u << 20)) return ONHIP_OK;
    int rc = get_scratch(bytes, &buf);
    if (rc) return rc;
    cfg.split = split;
    p.k_split_units = tiles_per * 4;
    p.partial = reinterpret_cast<float *>(buf);
    return ONHIP_OK;
}

static int dtype_of_compute(int compute, int *dt) {
    switch (compute) {
        case ONHIP_COMPUTE_F32: *dt = DT_F32; return ONHIP_OK;
        case ONHIP_COMPUTE_BF16: *dt = DT_BF16; return ONHIP_OK;
        case ONHIP_COMPUTE_F16: *dt = DT_F16; return ONHIP_OK;
        default: return set_error(ONHIP_ERR_ARG, "unknown compute mode %d", compute);
    }
}

static int kpu_of(int dt) { return dt == DT_F32 ? 4 : dt == DT_I8 ? 16 : 8; }

}  // namespace onhip

using namespace onhip;

extern "C" {

const char *onhip_last_error(void) { return g_err; }

int onhip_init(int device) {
    ONHIP_CHECK_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    ONHIP_CHECK_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(ONHIP_ERR_RUNTIME, "device %d is %s; this library holds gfx950 code only", device,
                         prop.gcnArchName);
    return ONHIP_OK;
}

int onhip_conv_out_shape(const onhip_conv_desc_t *d, int32_t *oh, int32_t *ow) {
    if (!oh || !ow) return set_error(ONHIP_ERR_ARG, "conv: null output pointer");
    return check_conv(d, oh, ow);
}

int onhip_conv2d_f32(const onhip_conv_desc_t *d, const float *x, const float *w, const float *bias,
                     const float *silu_lut, float *y, void *stream) {
    int32_t OH, OW;
    int rc = check_conv(d, &OH, &OW);
    if (rc) return rc;
    if (!x || !w || !y || (d->has_bias && !bias)) return set_error(ONHIP_ERR_ARG, "conv: null tensor pointer");
    if (d->has_bias && d->act_type == SILU && !silu_lut) return set_error(ONHIP_ERR_ARG, "conv: SILU needs the table");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const Epilogue ep = make_epilogue(*d, silu_lut);
    if (d->group != 1) {
        if (d->compute != ONHIP_COMPUTE_F32)
            return set_error(ONHIP_ERR_ARG, "conv: depthwise runs in fp32 only");
        return depthwise_f32_launch(*d, OH, OW, x, w, bias, ep, y, st);
    }
    IgemmLaunch cfg;
    memset(&cfg, 0, sizeof(cfg));
    rc = dtype_of_compute(d->compute, &cfg.dtype);
    if (rc) return rc;
    cfg.bl = BL_GATHER;
    cfg.batch = 1;
    IgemmParams p;
    memset(&p, 0, sizeof(p));
    p.M = d->cout;
    p.N = d->n * OH * OW;
    p.K = d->cin * d->kh * d->kw;
    if ((unsigned long long) p.K * (unsigned) (d->kh * d->kw) >= (1ULL << 32))
        return set_error(ONHIP_ERR_ARG, "conv: reduction length %d too large", p.K);
    const int kpu = kpu_of(cfg.dtype);
    p.k_units = (p.K + kpu - 1) / kpu;
    p.A = w;
    p.lda = p.K;
    p.B = x;
    p.H = d->h; p.W = d->w; p.OW = OW; p.OHW = OH * OW; p.HW = d->h * d->w;
    p.kh = d->kh; p.kw = d->kw; p.khkw = d->kh * d->kw;
    p.sh = d->stride_h; p.sw = d->stride_w; p.pt = d->pad_t; p.pl = d->pad_l;
    p.magic_khkw = magic_for(p.khkw); p.pass_khkw = pass_for(p.khkw);
    p.magic_kw = magic_for(p.kw); p.pass_kw = pass_for(p.kw);
    p.b_img_stride = (long long) d->cin * d->h * d->w;
    if (p.khkw == 1 && !d->pad_t && !d->pad_l && !d->pad_b && !d->pad_r) cfg.bl = BL_PLAIN;
    p.b_shift_bytes = ((long long) d->pad_t * d->w + d->pad_l) * 4;
    p.a_slice_bytes = (long long) p.M * p.K * 4;
    p.b_slice_bytes = (long long) d->n * p.b_img_stride * 4 + 2 * p.b_shift_bytes;
    p.c_slice_bytes = (long long) d->n * d->cout * OH * OW * 4;
    p.C = y;
    p.out_mode = OUT_CONV;
    p.c_img_stride = (long long) d->cout * OH * OW;
    p.c_stride_m = (long long) OH * OW;
    p.bias = bias;
    p.bias_mode = d->has_bias ? BIAS_M : BIAS_NONE;
    p.ep = ep;
    igemm_pick_tile(cfg, p);
    rc = plan_split(cfg, p);
    if (rc) return rc;
    return igemm_launch(cfg, p, st);
}

static void w8a32_layout(const onhip_conv_desc_t *d, int *cp, int *k_units, size_t *packed_bytes, size_t *q_bytes) {
    *cp = (d->cin + 15) / 16 * 16;
    *k_units = d->kh * d->kw * (*cp / 16);
    *packed_bytes = ((size_t) d->cout * *k_units * 16 + 255) / 256 * 256;
    *q_bytes = ((size_t) d->n * d->h * d->w * *cp + 255) / 256 * 256;
}

size_t onhip_conv2d_w8a32_workspace(const onhip_conv_desc_t *d) {
    if (!d || d->group != 1) return 0;
    int cp, ku;
    size_t pb, qb;
    w8a32_layout(d, &cp, &ku, &pb, &qb);
    return pb + qb;
}

int onhip_conv2d_w8a32(const onhip_conv_desc_t *d, const float *x, const int8_t *w8, const int32_t *bias32,
                       const float *weight_aux, const float *silu_lut, void *y, int32_t *acc32, void *workspace,
                       size_t workspace_bytes, void *stream) {
    int32_t OH, OW;
    int rc = check_conv(d, &OH, &OW);
    if (rc) return rc;
    if (!x || !w8 || !y || !weight_aux || (d->has_bias && !bias32))
        return set_error(ONHIP_ERR_ARG, "conv w8a32: null tensor pointer");
    // the reference pads all four sides by pads[0] (conv.c:979-999) while shapes come from the four
    // pads: only uniform padding is self-consistent
    if (d->pad_t != d->pad_l || d->pad_t != d->pad_b || d->pad_t != d->pad_r)
        return set_error(ONHIP_ERR_ARG, "conv w8a32: padding must be uniform");
    if (!(d->input_scale > 0.0f)) return set_error(ONHIP_ERR_ARG, "conv w8a32: input_scale must be positive");
    if (d->out_s8 && !(d->output_scale > 0.0f)) return set_error(ONHIP_ERR_ARG, "conv w8a32: output_scale must be positive");
    if (d->has_bias && d->act_type == SILU && !silu_lut) return set_error(ONHIP_ERR_ARG, "conv: SILU needs the table");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const Epilogue ep = make_epilogue(*d, silu_lut);
    if (d->group != 1) return depthwise_w8a32_launch(*d, OH, OW, x, w8, bias32, weight_aux, ep, y, acc32, st);

    int cp, k_units;
    size_t packed_bytes, q_bytes;
    w8a32_layout(d, &cp, &k_units, &packed_bytes, &q_bytes);
    if (!workspace || workspace_bytes < packed_bytes + q_bytes)
        return set_error(ONHIP_ERR_WORKSPACE, "conv w8a32: workspace of %zu bytes needed, %zu given",
                         packed_bytes + q_bytes, workspace ? workspace_bytes : (size_t) 0);
    if (reinterpret_cast<uintptr_t>(workspace) % 16)
        return set_error(ONHIP_ERR_WORKSPACE, "conv w8a32: workspace must be 16-byte aligned");
    if ((long long) d->n * d->h * d->w * cp >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "conv w8a32: staged activations of 2 GiB or more are not supported");
    int8_t *packed = reinterpret_cast<int8_t *>(workspace);
    int8_t *q = packed + packed_bytes;
    rc = pack_w8_launch(w8, d->cout, d->cin, d->kh, d->kw, cp, k_units, packed, st);
    if (rc) return rc;
    rc = quantize_nhwc_launch(x, d->n, d->cin, d->h, d->w, cp, 1.0f / d->input_scale, q, st);
    if (rc) return rc;

    IgemmLaunch cfg;
    memset(&cfg, 0, sizeof(cfg));
    cfg.dtype = DT_I8;
    cfg.bl = BL_KVEC;
    cfg.batch = 1;
    IgemmParams p;
    memset(&p, 0, sizeof(p));
    p.M = d->cout;
    p.N = d->n * OH * OW;
    p.K = k_units * 16;
    p.k_units = k_units;
    p.A = packed;
    p.lda = k_units * 16;
    p.B = q;
    p.H = d->h; p.W = d->w; p.OW = OW; p.OHW = OH * OW; p.HW = d->h * d->w;
    p.kh = d->kh; p.kw = d->kw; p.khkw = d->kh * d->kw;
    p.sh = d->stride_h; p.sw = d->stride_w; p.pt = d->pad_t; p.pl = d->pad_l;
    p.magic_kw = magic_for(p.kw); p.pass_kw = pass_for(p.kw);
    p.units_per_tap = cp / 16;
    p.magic_upt = magic_for(p.units_per_tap); p.pass_upt = pass_for(p.units_per_tap);
    p.pix_stride = cp;
    p.b_shift_bytes = ((long long) d->pad_t * d->w + d->pad_l) * cp;
    p.a_slice_bytes = (long long) p.M * p.lda;
    p.b_slice_bytes = (long long) d->n * d->h * d->w * cp + 2 * p.b_shift_bytes;
    p.c_slice_bytes = (long long) d->n * d->cout * OH * OW * 4;
    p.C = y;
    p.out_mode = OUT_CONV;
    p.c_img_stride = (long long) d->cout * OH * OW;
    p.c_stride_m = (long long) OH * OW;
    p.ep = ep;
    p.in_scale = d->input_scale;
    p.weight_aux = weight_aux;
    p.bias32 = d->has_bias ? bias32 : nullptr;
    p.acc_out = acc32;
    p.out_s8 = d->out_s8;
    p.out_inv_scale = d->out_s8 ? 1.0f / d->output_scale : 0.0f;
    igemm_pick_tile(cfg, p);
    rc = plan_split(cfg, p);
    if (rc) return rc;
    return igemm_launch(cfg, p, st);
}

int onhip_matmul(const onhip_matmul_desc_t *d, const float *a, const float *b, const float *bias,
                 const float *gelu_lut, float *out, void *stream) {
    if (!d || d->batch < 1 || d->m < 1 || d->k < 1 || d->n < 1) return set_error(ONHIP_ERR_ARG, "matmul: bad shape");
    if (!a || !b || !out) return set_error(ONHIP_ERR_ARG, "matmul: null tensor pointer");
    int batch = d->batch, M = d->m;
    // a shared right operand turns the batch into extra rows of one larger product
    if (d->b_shared) { M = batch * M; batch = 1; }
    if ((long long) batch * M * d->k >= (1LL << 31) || (long long) d->k * d->n >= (1LL << 31) ||
        (long long) batch * M * d->n >= (1LL << 31) || (long long) M * d->batch >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "matmul: operands of 2^31 elements or more are not supported");
    IgemmLaunch cfg;
    memset(&cfg, 0, sizeof(cfg));
    int rc = dtype_of_compute(d->compute, &cfg.dtype);
    if (rc) return rc;
    cfg.bl = BL_PLAIN;
    cfg.batch = batch;
    IgemmParams p;
    memset(&p, 0, sizeof(p));
    p.M = M; p.N = d->n; p.K = d->k;
    const int kpu = kpu_of(cfg.dtype);
    p.k_units = (p.K + kpu - 1) / kpu;
    p.A = a;
    p.lda = d->k;
    p.a_batch_stride = (long long) M * d->k;
    p.B = b;
    p.b_batch_stride = (long long) d->k * d->n;
    // a row-major [K, N] matrix is the 1x1 "image" of N pixels and K channels
    p.H = 1; p.W = d->n; p.OW = d->n; p.OHW = d->n; p.HW = d->n;
    p.kh = p.kw = p.khkw = 1; p.sh = p.sw = 1;
    p.a_slice_bytes = (long long) M * d->k * 4;
    p.b_slice_bytes = (long long) d->k * d->n * 4;
    p.c_slice_bytes = (long long) M * d->n * 4;
    p.C = out;
    p.out_mode = OUT_PLAIN;
    p.c_batch_stride = (long long) M * d->n;
    p.c_stride_m = d->n;
    p.c_stride_n = 1;
    p.bias = bias;
    p.bias_mode = bias ? BIAS_N : BIAS_NONE;
    p.ep.act = gelu_lut ? ONHIP_ACT_GELU_LUT : NOT_ACT;
    p.ep.lut = gelu_lut;
    igemm_pick_tile(cfg, p);
    rc = plan_split(cfg, p);
    if (rc) return rc;
    return igemm_launch(cfg, p, reinterpret_cast<hipStream_t>(stream));
}

int onhip_gemm_f32(int32_t m, int32_t k, int32_t n, const float *a, const float *w, const float *bias, float *out,
                   void *stream) {
    if (m < 1 || k < 1 || n < 1) return set_error(ONHIP_ERR_ARG, "gemm: bad shape %dx%dx%d", m, k, n);
    if (!a || !w || !bias || !out) return set_error(ONHIP_ERR_ARG, "gemm: null tensor pointer");
    return gemm_nt_launch(m, k, n, a, w, bias, out, reinterpret_cast<hipStream_t>(stream));
}

}  // extern "C"
