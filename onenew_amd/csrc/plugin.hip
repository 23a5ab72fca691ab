// Plugin level of the C ABI: the three `eval` bodies the oneNew host binds.  They read the slot
// arrays exactly like the reference kernels do (device/x86/Conv/conv.c:13-104, MatMul/mat_mul.c:10-33,
// Gemm/gemm.c:9-33) and run the kernel-level entry points of api.hip.
//
// Residency.  The oneNew host hands out host pointers (weights in std::vector, activations from
// aligned_alloc).  A slot whose address is device memory (hipMalloc / managed) is used in place;
// a host address is staged: weights, bias and tables are uploaded once and cached by host address
// and size (they live as long as the net, host/ops/conv.h:148-154), activations are copied in and
// the result copied back on every call.  eval is synchronous: the output is complete on return,
// like the reference's CUDA operators (device/cuda/MaxPool/maxpool.cu:76).
#include <stdio.h>
#include <string.h>

#include <map>
#include <mutex>
#include <utility>

#include "onhip_internal.hpp"

namespace onhip {

static std::mutex g_mu;
static bool g_ready = false;
// set by a caller that keeps consuming results on the device in stream order (onhip_plugin_set_async): an eval
// whose output is device memory then returns without waiting for the kernels
static bool g_async = false;
// the stream every eval queues its kernels on: the default stream unless the caller named another
// (onhip_plugin_set_stream)
static hipStream_t g_stream = nullptr;

static int wait_for_output() {
    if (!g_async) ONHIP_CHECK_HIP(hipStreamSynchronize(g_stream));
    return ONHIP_OK;
}

// result back into a host buffer: the blocking copy orders itself after the default stream and after streams created
// without hipStreamNonBlocking; a named stream of the other kind is waited for first
static int copy_out(void *host_out, const void *y, size_t bytes) {
    if (g_stream) ONHIP_CHECK_HIP(hipStreamSynchronize(g_stream));
    ONHIP_CHECK_HIP(hipMemcpy(host_out, y, bytes, hipMemcpyDeviceToHost));
    return ONHIP_OK;
}

struct DevBuf {
    void *ptr = nullptr;
    size_t bytes = 0;
};
// persistent staging buffers: [0] input, [1] second input, [2] output, [3] workspace
static DevBuf g_stage[6];   // 0, 1: inputs; 2: the output; 3: workspace; 4, 5: third and fourth input of a fused MatMul
// uploaded constants keyed by (host address, bytes); the fingerprint of the content detects a host buffer that was
// freed and reused for other data at the same address, or weights updated in place
struct ConstEntry {
    void *dev;
    uint64_t fingerprint;
};
static std::map<std::pair<const void *, size_t>, ConstEntry> g_const;
// 0: every byte is hashed on every call (four independent multiply-xor lanes: memory speed, about 0.05 ms per MiB);
// 1: at most 4096 sampled words, for a caller whose weights never change while the library holds a copy
static int g_weight_check_sampled = 0;

static uint64_t fingerprint(const void *host, size_t bytes) {
    const unsigned char *b = static_cast<const unsigned char *>(host);
    const uint64_t P = 1099511628211ULL;
    uint64_t h = 1469598103934665603ULL ^ bytes;
    const size_t words = bytes / 8;
    if (g_weight_check_sampled) {
        const size_t step = words > 4096 ? words / 4096 : 1;
        for (size_t i = 0; i < words; i += step) {
            uint64_t v;
            memcpy(&v, b + i * 8, 8);
            h = (h ^ v) * P;
        }
    } else {
        uint64_t l0 = h, l1 = h + 1, l2 = h + 2, l3 = h + 3;
        size_t i = 0;
        for (; i + 4 <= words; i += 4) {
            uint64_t v[4];
            memcpy(v, b + i * 8, 32);
            l0 = (l0 ^ v[0]) * P; l1 = (l1 ^ v[1]) * P; l2 = (l2 ^ v[2]) * P; l3 = (l3 ^ v[3]) * P;
        }
        for (; i < words; ++i) {
            uint64_t v;
            memcpy(&v, b + i * 8, 8);
            l0 = (l0 ^ v) * P;
        }
        h = (((l0 * P) ^ l1) * P ^ l2) * P ^ l3;
    }
    for (size_t i = words * 8; i < bytes; ++i) h = (h ^ b[i]) * P;
    if (words) {
        uint64_t v;
        memcpy(&v, b + (words - 1) * 8, 8);
        h = (h ^ v) * P;
    }
    return h;
}

// tap-major copies of k x k convolution weights, keyed by the device address of the original
struct PackedEntry {
    float *dev;
    size_t bytes;
    bool int8;
    const void *other;   // a pack made of two weight tensors (the 1x1 layers of a fused block): the one it is not keyed by
};
static std::map<const void *, PackedEntry> g_packed;

static void drop_packed(const void *w_dev) {
    auto it = g_packed.find(w_dev);
    if (it != g_packed.end()) {
        (void) hipFree(it->second.dev);
        g_packed.erase(it);
    }
    for (it = g_packed.begin(); it != g_packed.end();) {
        if (it->second.other == w_dev) {
            (void) hipFree(it->second.dev);
            it = g_packed.erase(it);
        } else {
            ++it;
        }
    }
}

// *out = packed copy of the device weights w_dev for convolution d, or nullptr if d takes them as they are.
// A weight that lives in device memory is packed when first seen; after changing it in place call
// onhip_plugin_release().
static int packed_weights(const onhip_conv_desc_t *d, const float *w_dev, const float **out, bool int8 = false) {
    *out = nullptr;
    const size_t bytes = int8 ? onhip_conv2d_w8a32_packed_weight_bytes(d) : onhip_conv2d_packed_weight_bytes(d);
    if (!bytes) return ONHIP_OK;
    auto it = g_packed.find(w_dev);
    if (it != g_packed.end() && it->second.bytes == bytes && it->second.int8 == int8) { *out = it->second.dev; return ONHIP_OK; }
    drop_packed(w_dev);
    float *p = nullptr;
    ONHIP_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&p), bytes));
    int rc = int8 ? onhip_conv2d_w8a32_pack_weights(d, reinterpret_cast<const int8_t *>(w_dev),
                                                    reinterpret_cast<int8_t *>(p), g_stream)
                  : onhip_conv2d_pack_weights(d, w_dev, p, g_stream);
    if (rc) { (void) hipFree(p); return rc; }
    g_packed[w_dev] = PackedEntry{p, bytes, int8, nullptr};
    *out = p;
    return ONHIP_OK;
}

// the two 1x1 weight tensors of an inverted-residual block in the layout of onhip_ir_block_f32, packed when first seen,
// keyed by the projection's device address
static int packed_block_weights(const float *ex_w, const float *pw_w, int cin, int ce, int co, const float **out) {
    const size_t bytes = onhip_ir_block_packed_weight_bytes(cin, ce, co);
    auto it = g_packed.find(pw_w);
    if (it != g_packed.end() && it->second.bytes == bytes && it->second.other == ex_w) { *out = it->second.dev; return ONHIP_OK; }
    drop_packed(pw_w);
    float *p = nullptr;
    ONHIP_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&p), bytes));
    const int rc = onhip_ir_block_pack_weights(ex_w, pw_w, cin, ce, co, p, g_stream);
    if (rc) { (void) hipFree(p); return rc; }
    g_packed[pw_w] = PackedEntry{p, bytes, false, ex_w};
    *out = p;
    return ONHIP_OK;
}

// the 1x1 convolution of a fused pair: its weights in the order onhip_conv2d_pw_f32 reads them, next to their device copy
static int packed_pair_weights(const onhip_conv_desc_t *b, const float *w_dev, const float **out) {
    const size_t bytes = onhip_conv2d_pw_packed_weight_bytes(b);
    auto it = g_packed.find(w_dev);
    if (it != g_packed.end() && it->second.bytes == bytes && it->second.other == w_dev) { *out = it->second.dev; return ONHIP_OK; }
    drop_packed(w_dev);
    float *p = nullptr;
    ONHIP_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&p), bytes));
    const int rc = onhip_conv2d_pw_pack_weights(b, w_dev, p, g_stream);
    if (rc) { (void) hipFree(p); return rc; }
    g_packed[w_dev] = PackedEntry{p, bytes, false, w_dev};
    *out = p;
    return ONHIP_OK;
}

static int ensure_ready() {
    if (g_ready) return ONHIP_OK;
    int dev = 0;
    ONHIP_CHECK_HIP(hipGetDevice(&dev));
    int rc = onhip_init(dev);
    if (rc) return rc;
    g_ready = true;
    return ONHIP_OK;
}

static bool is_device_ptr(const void *p) {
    hipPointerAttribute_t attr;
    hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void) hipGetLastError();  // plain host memory: clear the sticky error
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

static int stage_buf(int slot, size_t bytes, void **out) {
    DevBuf &b = g_stage[slot];
    if (bytes > b.bytes) {
        size_t want = (bytes + (1u << 20) - 1) & ~((size_t) (1u << 20) - 1);
        if (slot == 3) {
            // the workspace is a kernel argument of launches a caller may have recorded into a HIP graph (the int8 copy
            // of a W8A32 convolution's activations): an outgrown block stays allocated for those replays, sizes at least
            // double so the retired blocks together stay below the live one
            if (want < 2 * b.bytes) want = 2 * b.bytes;
        } else if (b.ptr) {
            ONHIP_CHECK_HIP(hipFree(b.ptr));   // host staging: only synchronous copies of this library touch it
        }
        b.ptr = nullptr;
        b.bytes = 0;
        ONHIP_CHECK_HIP(hipMalloc(&b.ptr, want));
        b.bytes = want;
    }
    *out = b.ptr;
    return ONHIP_OK;
}

// device address of an input tensor: in place if already on the device, else staged copy
static int input_on_device(int slot, const void *host, size_t bytes, const void **dev) {
    if (is_device_ptr(host)) { *dev = host; return ONHIP_OK; }
    void *d;
    int rc = stage_buf(slot, bytes, &d);
    if (rc) return rc;
    ONHIP_CHECK_HIP(hipMemcpy(d, host, bytes, hipMemcpyHostToDevice));
    *dev = d;
    return ONHIP_OK;
}

// device address of a constant (weight, bias, table): uploaded once
static int const_on_device(const void *host, size_t bytes, const void **dev) {
    if (!host) { *dev = nullptr; return ONHIP_OK; }
    if (is_device_ptr(host)) { *dev = host; return ONHIP_OK; }
    auto key = std::make_pair(host, bytes);
    const uint64_t fp = fingerprint(host, bytes);
    auto it = g_const.find(key);
    if (it != g_const.end()) {
        if (it->second.fingerprint != fp) {
            ONHIP_CHECK_HIP(hipMemcpy(it->second.dev, host, bytes, hipMemcpyHostToDevice));
            it->second.fingerprint = fp;
            drop_packed(it->second.dev);   // a packed copy of the old content is stale
        }
        *dev = it->second.dev;
        return ONHIP_OK;
    }
    void *d = nullptr;
    ONHIP_CHECK_HIP(hipMalloc(&d, bytes < 16 ? 16 : bytes));
    ONHIP_CHECK_HIP(hipMemcpy(d, host, bytes, hipMemcpyHostToDevice));
    g_const[key] = ConstEntry{d, fp};
    *dev = d;
    return ONHIP_OK;
}

static long long numel(const OPERAND_S *o) {
    long long n = 1;
    for (int i = 0; i < SHAPE_LEN; ++i) n *= o->shapes[i];  // unused dims hold 1 (common/utils_c.h:9-16)
    return n;
}

// What travels along the edges of an int8 convolution inside a chain of them (inputs[4] of `eval_link`): in_s8 != 0, the
// input tensor is int8 NHWC with channels padded to 16, quantised with this operator's input_scale by its producer;
// out_s8 != 0, the result is stored that way for consumers whose input_scale is out_scale.
// twin != 0 (fp32 results with a folded Add only): outputs[1] receives the result once more, as int8 NHWC quantised with
// out_scale, for the int8 convolutions among its readers.
struct ConvLink {
    int32_t in_s8, out_s8;
    float out_scale;
    int32_t twin;
};

// fuse 0: the Conv of the reference.  1: inputs[3] holds a tensor of the output's shape that is added to the result
// (the Add of a residual block); 2: and a Relu after that.  link: null, or the int8 forms of the edges.
static int conv_eval_fused(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs, int fuse, const ConvLink *link = nullptr) {
    const CONV_CONFIG_S *cfg = reinterpret_cast<const CONV_CONFIG_S *>(params[0].addr);
    const OPERAND_S *in_t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    const OPERAND_S *w_t = reinterpret_cast<const OPERAND_S *>(params[2].addr);
    // params[3] is the bias descriptor, or the output when there is no bias (conv.c:434-436)
    const OPERAND_S *out_t = reinterpret_cast<const OPERAND_S *>(params[cfg->has_bias ? 4 : 3].addr);
    if (!cfg || !in_t || !w_t || !out_t) return set_error(ONHIP_ERR_ARG, "Conv eval: empty params slot");

    onhip_conv_desc_t d;
    memset(&d, 0, sizeof(d));
    // the reference evaluates image 0 only (host/ops/conv.h:43); a batched output descriptor asks for more
    d.n = out_t->shapes[0] < in_t->shapes[0] ? out_t->shapes[0] : in_t->shapes[0];
    if (d.n < 1) d.n = 1;
    d.cin = in_t->shapes[1]; d.h = in_t->shapes[2]; d.w = in_t->shapes[3];
    d.cout = w_t->shapes[0]; d.kh = w_t->shapes[2]; d.kw = w_t->shapes[3];
    d.stride_h = (int32_t) cfg->strides[0]; d.stride_w = (int32_t) cfg->strides[1];
    d.pad_t = (int32_t) cfg->pads[0]; d.pad_l = (int32_t) cfg->pads[1];
    d.pad_b = (int32_t) cfg->pads[2]; d.pad_r = (int32_t) cfg->pads[3];
    // conv.c:18-29: without bias the dense path runs whatever the group says; with bias any group != 1
    // (including a missing attribute, 0) is depthwise
    d.group = !cfg->has_bias ? 1 : (cfg->group == 1 ? 1 : d.cin);
    d.has_bias = cfg->has_bias ? 1 : 0;
    d.act_type = cfg->act_type;
    d.clip_min = cfg->clip_min; d.clip_max = cfg->clip_max;
    d.leaky_relu_alpha = cfg->leaky_relu_alpha;
    d.hard_sigmoid_alpha = cfg->hard_sigmoid_alpha; d.hard_sigmoid_beta = cfg->hard_sigmoid_beta;
    d.input_scale = cfg->input_scale;
    const bool int8 = cfg->ifmap_quant2 == TYPE_INT8;
    if (d.group != 1 && d.cout != d.cin)
        return set_error(ONHIP_ERR_ARG, "Conv eval: depthwise with cout %d != cin %d", d.cout, d.cin);

    int32_t OH, OW;
    int rc = onhip_conv_out_shape(&d, &OH, &OW);
    if (rc) return rc;
    if (out_t->shapes[1] != d.cout || out_t->shapes[2] != OH || out_t->shapes[3] != OW)
        return set_error(ONHIP_ERR_ARG, "Conv eval: output descriptor %dx%dx%d does not match computed %dx%dx%d",
                         out_t->shapes[1], out_t->shapes[2], out_t->shapes[3], d.cout, OH, OW);
    const int kc = d.group == 1 ? d.cin : 1;
    if (w_t->shapes[1] != kc)
        return set_error(ONHIP_ERR_ARG, "Conv eval: weight has %d input channels, expected %d", w_t->shapes[1], kc);

    const bool in_s8 = link && link->in_s8, out_s8 = link && link->out_s8;
    if (link) {
        if (!int8) return set_error(ONHIP_ERR_ARG, "Conv eval: int8 edges are for int8 convolutions");
        if (d.group != 1 && (fuse || link->twin)) return set_error(ONHIP_ERR_ARG, "Conv eval: a depthwise int8 convolution takes no folded Add");
        if (out_s8 && fuse) return set_error(ONHIP_ERR_ARG, "Conv eval: an int8 result cannot take the Add of a residual block");
        if (out_s8 && !(link->out_scale > 0.0f)) return set_error(ONHIP_ERR_ARG, "Conv eval: int8 result without a scale");
    }
    const size_t in_bytes = in_s8 ? (size_t) d.n * d.h * d.w * ((d.cin + 15) / 16 * 16) : (size_t) d.n * d.cin * d.h * d.w * 4;
    const size_t out_bytes = out_s8 ? (size_t) d.n * OH * OW * ((d.cout + 15) / 16 * 16) : (size_t) d.n * d.cout * OH * OW * 4;
    const size_t w_elems = (size_t) d.cout * kc * d.kh * d.kw;
    const void *x, *w, *b = nullptr, *lut = nullptr, *aux = nullptr;
    rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), in_bytes, &x);
    if (rc) return rc;
    // int8 weights sit at the front of the fp32-sized buffer, the int32 bias in the fp32 bias buffer
    rc = const_on_device(reinterpret_cast<const void *>(inputs[1].addr), int8 ? w_elems : w_elems * 4, &w);
    if (rc) return rc;
    if (d.has_bias) {
        rc = const_on_device(reinterpret_cast<const void *>(inputs[2].addr), (size_t) d.cout * 4, &b);
        if (rc) return rc;
    }
    if (d.has_bias && d.act_type == SILU) {
        rc = const_on_device(reinterpret_cast<const void *>(inputs[BUF_MAXNUM - 1].addr), 8192 * 4, &lut);
        if (rc) return rc;
        if (!lut) return set_error(ONHIP_ERR_ARG, "Conv eval: SILU without a table in inputs[%d]", BUF_MAXNUM - 1);
    }
    const void *addend = nullptr;
    if (fuse) {
        if (!inputs[3].addr) return set_error(ONHIP_ERR_ARG, "Conv eval: no addend in inputs[3]");
        rc = input_on_device(1, reinterpret_cast<const void *>(inputs[3].addr), out_bytes, &addend);
        if (rc) return rc;
    }
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, out_bytes, &y);
        if (rc) return rc;
    }
    // the model-wide GEMM tile the file carries (host/ops/conv.h:65-68 puts USEFUL_INFO_S in the last params slot): a
    // tile this library has kernels for narrows the cost model's choice, anything else (the converter's 16 x 16) does not
    struct HintScope {
        HintScope(const USEFUL_INFO_S *u) { if (u) onhip_set_tile_hint(u->block_info.cuda_gemm_tile_m, u->block_info.cuda_gemm_tile_n); }
        ~HintScope() { onhip_set_tile_hint(0, 0); }
    } hint(reinterpret_cast<const USEFUL_INFO_S *>(params[BUF_MAXNUM - 1].addr));
    if (int8) {
        if (d.cout > 4096) return set_error(ONHIP_ERR_ARG, "Conv eval: weight_aux holds 4096 channels, cout is %d", d.cout);
        rc = const_on_device(cfg->weight_aux, (size_t) d.cout * 4, &aux);
        if (rc) return rc;
        void *ws = nullptr;
        const size_t ws_bytes = onhip_conv2d_w8a32_workspace(&d);
        if (ws_bytes) {
            rc = stage_buf(3, ws_bytes, &ws);
            if (rc) return rc;
        }
        // dense int8 weights are re-laid out for the kernel once, next to their device copy
        const float *wp = nullptr;
        rc = packed_weights(&d, (const float *) w, &wp, true);
        if (rc) return rc;
        bool added = false;   // the addend went into the convolution's store
        if (link || (fuse && wp)) {
            if (!wp && d.group == 1) return set_error(ONHIP_ERR_ARG, "Conv eval: int8 edges need the packed weight form");
            if (!wp) wp = (const float *) w;   // depthwise: the weights as they are
            d.out_s8 = out_s8 ? 1 : 0;
            d.output_scale = link ? link->out_scale : 0.0f;
            int8_t *twin = nullptr;
            if (link && link->twin) {
                twin = reinterpret_cast<int8_t *>(outputs[1].addr);
                if (!twin || !is_device_ptr(twin) || !fuse || out_s8)
                    return set_error(ONHIP_ERR_ARG, "Conv eval: the int8 twin needs a device buffer in outputs[1], a folded Add and an fp32 result");
            }
            rc = onhip_conv2d_w8_link(&d, in_s8 ? nullptr : (const float *) x, in_s8 ? (const int8_t *) x : nullptr, (const int8_t *) wp,
                                      (const int32_t *) b, (const float *) aux, (const float *) lut, (const float *) addend, fuse == 2,
                                      y, twin, ws, ws_bytes, g_stream);
            added = true;
        } else if (wp)
            rc = onhip_conv2d_w8a32_packed(&d, (const float *) x, (const int8_t *) wp, (const int32_t *) b,
                                           (const float *) aux, (const float *) lut, y, nullptr, ws, ws_bytes, g_stream);
        else
            rc = onhip_conv2d_w8a32(&d, (const float *) x, (const int8_t *) w, (const int32_t *) b, (const float *) aux,
                                    (const float *) lut, y, nullptr, ws, ws_bytes, g_stream);
        if (!rc && fuse && !added) {   // unpacked weights: the two operators as one pass over y
            onhip_add_desc_t ad;
            memset(&ad, 0, sizeof(ad));
            ad.ndim = 4;
            const int32_t shape[4] = {d.n, d.cout, OH, OW};
            for (int i = 0; i < 4; ++i) ad.large_shape[i] = ad.small_shape[i] = shape[i];
            ad.relu = fuse == 2 ? 2 : 0;   // the Relu operator's rules by element index, in the same pass
            rc = onhip_add_f32(&ad, (const float *) y, (const float *) addend, (float *) y, g_stream);
        }
    } else if (fuse) {
        const float *wp = nullptr;
        rc = packed_weights(&d, (const float *) w, &wp);
        if (rc) return rc;
        rc = onhip_conv2d_f32_add(&d, (const float *) x, wp ? wp : (const float *) w, wp ? 1 : 0, (const float *) b,
                                  (const float *) lut, (const float *) addend, fuse == 2, (float *) y, g_stream);
    } else {
        // k x k dense weights are re-laid out tap-major once, next to their device copy
        const float *wp = nullptr;
        rc = packed_weights(&d, (const float *) w, &wp);
        if (rc) return rc;
        if (wp)
            rc = onhip_conv2d_f32_packed(&d, (const float *) x, wp, (const float *) b, (const float *) lut, (float *) y,
                                         g_stream);
        else
            rc = onhip_conv2d_f32(&d, (const float *) x, (const float *) w, (const float *) b, (const float *) lut,
                                  (float *) y, g_stream);
    }
    if (rc) return rc;
    if (!out_on_dev) return copy_out(host_out, y, out_bytes);
    else return wait_for_output();
    return ONHIP_OK;
}

// One convolution of a fused block as the library describes it: configuration, input extent, weight operand.
static void block_conv_desc(onhip_conv_desc_t *d, const CONV_CONFIG_S *cfg, int n, int cin, int h, int w, const OPERAND_S *w_t) {
    memset(d, 0, sizeof(*d));
    d->n = n; d->cin = cin; d->h = h; d->w = w;
    d->cout = w_t->shapes[0]; d->kh = w_t->shapes[2]; d->kw = w_t->shapes[3];
    d->stride_h = (int32_t) cfg->strides[0]; d->stride_w = (int32_t) cfg->strides[1];
    d->pad_t = (int32_t) cfg->pads[0]; d->pad_l = (int32_t) cfg->pads[1];
    d->pad_b = (int32_t) cfg->pads[2]; d->pad_r = (int32_t) cfg->pads[3];
    d->group = !cfg->has_bias ? 1 : (cfg->group == 1 ? 1 : cin);   // conv.c:18-29, as in conv_eval_fused
    d->has_bias = cfg->has_bias ? 1 : 0;
    d->act_type = cfg->act_type;
    d->clip_min = cfg->clip_min; d->clip_max = cfg->clip_max;
    d->leaky_relu_alpha = cfg->leaky_relu_alpha;
    d->hard_sigmoid_alpha = cfg->hard_sigmoid_alpha; d->hard_sigmoid_beta = cfg->hard_sigmoid_beta;
    d->compute = ONHIP_COMPUTE_F32;
}

// Conv (1x1) -> Conv (depthwise 3x3) -> Conv (1x1) [-> Add] as one call of onhip_ir_block_f32.  Slots: params[0..4] /
// inputs[0..2] as for the first convolution's `eval`, params[4] the block's result operand; inputs[3] the addend or
// null; params[5] the depthwise CONV_CONFIG_S, params[6] its weight operand, inputs[5] / inputs[6] its weights and bias;
// params[7] the last convolution's CONV_CONFIG_S, params[8] its weight operand, inputs[7] / inputs[8] its weights and
// bias (null without).  query: no tensor is touched; the return value is 1 when the library recommends the one-launch
// kernel for these shapes and 0 otherwise.
static int conv_block_eval_mode(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs, bool query) {
    const CONV_CONFIG_S *cfg[3] = {reinterpret_cast<const CONV_CONFIG_S *>(params[0].addr), reinterpret_cast<const CONV_CONFIG_S *>(params[5].addr),
                                   reinterpret_cast<const CONV_CONFIG_S *>(params[7].addr)};
    const OPERAND_S *in_t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    const OPERAND_S *w_t[3] = {reinterpret_cast<const OPERAND_S *>(params[2].addr), reinterpret_cast<const OPERAND_S *>(params[6].addr),
                               reinterpret_cast<const OPERAND_S *>(params[8].addr)};
    const OPERAND_S *out_t = reinterpret_cast<const OPERAND_S *>(params[4].addr);
    if (!cfg[0] || !cfg[1] || !cfg[2] || !in_t || !w_t[0] || !w_t[1] || !w_t[2] || !out_t) {
        if (query) return 0;
        return set_error(ONHIP_ERR_ARG, "Conv block eval: empty params slot");
    }
    if (cfg[0]->ifmap_quant2 == TYPE_INT8 || cfg[1]->ifmap_quant2 == TYPE_INT8 || cfg[2]->ifmap_quant2 == TYPE_INT8) {
        if (query) return 0;
        return set_error(ONHIP_ERR_ARG, "Conv block eval: fp32 convolutions only");
    }
    onhip_conv_desc_t d[3];
    int n = out_t->shapes[0] < in_t->shapes[0] ? out_t->shapes[0] : in_t->shapes[0];
    n = n < 1 ? 1 : n;
    int32_t oh = 0, ow = 0, h2 = 0, w2 = 0, h3 = 0, w3 = 0;
    block_conv_desc(&d[0], cfg[0], n, in_t->shapes[1], in_t->shapes[2], in_t->shapes[3], w_t[0]);
    bool ok = onhip_conv_out_shape(&d[0], &h2, &w2) == ONHIP_OK;
    if (ok) {
        block_conv_desc(&d[1], cfg[1], n, d[0].cout, h2, w2, w_t[1]);
        ok = onhip_conv_out_shape(&d[1], &h3, &w3) == ONHIP_OK;
    }
    if (ok) {
        block_conv_desc(&d[2], cfg[2], n, d[1].cout, h3, w3, w_t[2]);
        ok = onhip_conv_out_shape(&d[2], &oh, &ow) == ONHIP_OK && out_t->shapes[1] == d[2].cout && out_t->shapes[2] == oh && out_t->shapes[3] == ow;
    }
    if (query) return ok && onhip_ir_block_supported(&d[0], &d[1], &d[2]) >= 2 ? 1 : 0;
    if (!ok) return set_error(ONHIP_ERR_ARG, "Conv block eval: the three convolutions and the result operand do not fit together");
    if (!onhip_ir_block_supported(&d[0], &d[1], &d[2])) return set_error(ONHIP_ERR_ARG, "Conv block eval: not a block the one-launch kernel takes");
    const size_t in_bytes = (size_t) n * d[0].cin * d[0].h * d[0].w * 4, out_bytes = (size_t) n * d[2].cout * oh * ow * 4;
    const void *x, *ex_w, *ex_b, *dw_w, *dw_b, *pw_w, *pw_b = nullptr, *addend = nullptr;
    int rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), in_bytes, &x);
    if (!rc) rc = const_on_device(reinterpret_cast<const void *>(inputs[1].addr), (size_t) d[0].cout * d[0].cin * 4, &ex_w);
    if (!rc) rc = const_on_device(reinterpret_cast<const void *>(inputs[2].addr), (size_t) d[0].cout * 4, &ex_b);
    if (!rc) rc = const_on_device(reinterpret_cast<const void *>(inputs[5].addr), (size_t) d[1].cout * d[1].kh * d[1].kw * 4, &dw_w);
    if (!rc) rc = const_on_device(reinterpret_cast<const void *>(inputs[6].addr), (size_t) d[1].cout * 4, &dw_b);
    if (!rc) rc = const_on_device(reinterpret_cast<const void *>(inputs[7].addr), (size_t) d[2].cout * d[2].cin * 4, &pw_w);
    if (!rc && d[2].has_bias) rc = const_on_device(reinterpret_cast<const void *>(inputs[8].addr), (size_t) d[2].cout * 4, &pw_b);
    if (!rc && inputs[3].addr) rc = input_on_device(5, reinterpret_cast<const void *>(inputs[3].addr), out_bytes, &addend);
    if (rc) return rc;
    if (!ex_w || !ex_b || !dw_w || !dw_b || !pw_w) return set_error(ONHIP_ERR_ARG, "Conv block eval: empty weight or bias slot");
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, out_bytes, &y);
        if (rc) return rc;
    }
    const float *packed = nullptr;
    rc = packed_block_weights((const float *) ex_w, (const float *) pw_w, d[0].cin, d[0].cout, d[2].cout, &packed);
    if (rc) return rc;
    rc = onhip_ir_block_f32(&d[0], &d[1], &d[2], (const float *) x, packed, (const float *) ex_b, (const float *) dw_w, (const float *) dw_b,
                            (const float *) pw_b, (const float *) addend, (float *) y, g_stream);
    if (rc) return rc;
    return out_on_dev ? wait_for_output() : copy_out(host_out, y, out_bytes);
}

// Conv (dense, at most 64 output channels, not a plain 1x1) -> Conv (1x1) [-> Add [-> Relu]] as one call of
// onhip_conv2d_pw_f32.  Slots: params[0..4] / inputs[0..2] as for the first convolution's `eval`, params[4] the pair's result
// operand; inputs[3] the addend or null; params[5] the second convolution's CONV_CONFIG_S, params[6] its weight operand,
// inputs[5] / inputs[6] its weights and bias (null without).  relu: relu.c's rule on the sum (with an addend only).
// query: no tensor is touched; 1 when the library recommends the one-launch kernel for these shapes, else 0.
static int conv_pair_eval_mode(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs, bool query, bool relu) {
    const CONV_CONFIG_S *cfg[2] = {reinterpret_cast<const CONV_CONFIG_S *>(params[0].addr), reinterpret_cast<const CONV_CONFIG_S *>(params[5].addr)};
    const OPERAND_S *in_t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    const OPERAND_S *w_t[2] = {reinterpret_cast<const OPERAND_S *>(params[2].addr), reinterpret_cast<const OPERAND_S *>(params[6].addr)};
    const OPERAND_S *out_t = reinterpret_cast<const OPERAND_S *>(params[4].addr);
    if (!cfg[0] || !cfg[1] || !in_t || !w_t[0] || !w_t[1] || !out_t) {
        if (query) return 0;
        return set_error(ONHIP_ERR_ARG, "Conv pair eval: empty params slot");
    }
    if (cfg[0]->ifmap_quant2 == TYPE_INT8 || cfg[1]->ifmap_quant2 == TYPE_INT8) {
        if (query) return 0;
        return set_error(ONHIP_ERR_ARG, "Conv pair eval: fp32 convolutions only");
    }
    onhip_conv_desc_t d[2];
    int n = out_t->shapes[0] < in_t->shapes[0] ? out_t->shapes[0] : in_t->shapes[0];
    n = n < 1 ? 1 : n;
    int32_t oh = 0, ow = 0, h2 = 0, w2 = 0;
    block_conv_desc(&d[0], cfg[0], n, in_t->shapes[1], in_t->shapes[2], in_t->shapes[3], w_t[0]);
    bool ok = cfg[0]->group == 1 && cfg[1]->group == 1 && w_t[0]->shapes[1] == in_t->shapes[1] && onhip_conv_out_shape(&d[0], &h2, &w2) == ONHIP_OK;
    if (ok) {
        block_conv_desc(&d[1], cfg[1], n, d[0].cout, h2, w2, w_t[1]);
        ok = w_t[1]->shapes[1] == d[0].cout && onhip_conv_out_shape(&d[1], &oh, &ow) == ONHIP_OK && out_t->shapes[1] == d[1].cout &&
             out_t->shapes[2] == oh && out_t->shapes[3] == ow;
    }
    if (query) return ok && onhip_conv2d_pw_supported(&d[0], &d[1]) >= 2 ? 1 : 0;
    if (!ok) return set_error(ONHIP_ERR_ARG, "Conv pair eval: the two convolutions and the result operand do not fit together");
    if (!onhip_conv2d_pw_supported(&d[0], &d[1])) return set_error(ONHIP_ERR_ARG, "Conv pair eval: not a pair the one-launch kernel takes");
    const size_t in_bytes = (size_t) n * d[0].cin * d[0].h * d[0].w * 4, out_bytes = (size_t) n * d[1].cout * oh * ow * 4;
    const void *x, *wa, *ba = nullptr, *wb, *bb = nullptr, *addend = nullptr;
    int rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), in_bytes, &x);
    if (!rc) rc = const_on_device(reinterpret_cast<const void *>(inputs[1].addr), (size_t) d[0].cout * d[0].cin * d[0].kh * d[0].kw * 4, &wa);
    if (!rc && d[0].has_bias) rc = const_on_device(reinterpret_cast<const void *>(inputs[2].addr), (size_t) d[0].cout * 4, &ba);
    if (!rc) rc = const_on_device(reinterpret_cast<const void *>(inputs[5].addr), (size_t) d[1].cout * d[1].cin * 4, &wb);
    if (!rc && d[1].has_bias) rc = const_on_device(reinterpret_cast<const void *>(inputs[6].addr), (size_t) d[1].cout * 4, &bb);
    if (!rc && inputs[3].addr) rc = input_on_device(5, reinterpret_cast<const void *>(inputs[3].addr), out_bytes, &addend);
    if (rc) return rc;
    if (!wa || !wb || (d[0].has_bias && !ba) || (d[1].has_bias && !bb)) return set_error(ONHIP_ERR_ARG, "Conv pair eval: empty weight or bias slot");
    if (relu && !addend) return set_error(ONHIP_ERR_ARG, "Conv pair eval: a Relu after the Add needs the addend in inputs[3]");
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, out_bytes, &y);
        if (rc) return rc;
    }
    const float *wa_packed = nullptr, *wb_packed = nullptr;
    rc = packed_weights(&d[0], (const float *) wa, &wa_packed);
    if (!rc && !wa_packed) rc = set_error(ONHIP_ERR_ARG, "Conv pair eval: the first convolution has no packed weight form");
    if (!rc) rc = packed_pair_weights(&d[1], (const float *) wb, &wb_packed);
    if (rc) return rc;
    rc = onhip_conv2d_pw_f32(&d[0], &d[1], (const float *) x, wa_packed, (const float *) ba, wb_packed, (const float *) bb,
                             (const float *) addend, relu ? 1 : 0, (float *) y, g_stream);
    if (rc) return rc;
    return out_on_dev ? wait_for_output() : copy_out(host_out, y, out_bytes);
}

static int conv_pair_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return conv_pair_eval_mode(params, inputs, outputs, false, false);
}
static int conv_pair_relu_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return conv_pair_eval_mode(params, inputs, outputs, false, true);
}

static int conv_block_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return conv_block_eval_mode(params, inputs, outputs, false);
}

static int conv_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return conv_eval_fused(params, inputs, outputs, 0);
}
static int conv_add_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return conv_eval_fused(params, inputs, outputs, 1);
}
static int conv_add_relu_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return conv_eval_fused(params, inputs, outputs, 2);
}
// inputs[4]: a ConvLink in host memory; inputs[5]: null, or one int32 in host memory, 1 / 2 = the Add (and Relu) of a
// residual block with its other operand in inputs[3]
static int conv_link_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const ConvLink *link = reinterpret_cast<const ConvLink *>(inputs[4].addr);
    if (!link) return set_error(ONHIP_ERR_ARG, "Conv eval: no edge description in inputs[4]");
    const int32_t *fuse = reinterpret_cast<const int32_t *>(inputs[5].addr);
    if (fuse && (*fuse < 0 || *fuse > 2)) return set_error(ONHIP_ERR_ARG, "Conv eval: fold code %d", *fuse);
    return conv_eval_fused(params, inputs, outputs, fuse ? *fuse : 0, link);
}

// mode 0: MatMul.  mode 1: MatMul -> Add of a bias over the last axis (params[3] / inputs[2], n elements; the result's
// operand moves to params[4]).  mode 2: -> Gelu as well, through the table in inputs[11] like the Gelu operator.
// mode 3: mode 1 -> Add of the tensor in inputs[3], which has the result's shape.
static int matmul_eval_mode(int mode, BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const OPERAND_S *a_t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    const OPERAND_S *b_t = reinterpret_cast<const OPERAND_S *>(params[2].addr);
    const OPERAND_S *bias_t = mode ? reinterpret_cast<const OPERAND_S *>(params[3].addr) : nullptr;
    const OPERAND_S *o_t = reinterpret_cast<const OPERAND_S *>(params[mode ? 4 : 3].addr);
    if (!a_t || !b_t || !o_t || (mode && (!bias_t || !inputs[2].addr))) return set_error(ONHIP_ERR_ARG, "MatMul eval: empty params slot");
    if (mode == 2 && !inputs[BUF_MAXNUM - 1].addr) return set_error(ONHIP_ERR_ARG, "MatMul eval: no Gelu table in inputs[11]");
    const int nd = a_t->dim_num_of_shapes;
    if (nd < 2 || nd > SHAPE_LEN || o_t->dim_num_of_shapes < 1 || o_t->dim_num_of_shapes > SHAPE_LEN)
        return set_error(ONHIP_ERR_ARG, "MatMul eval: rank %d", nd);
    onhip_matmul_desc_t d;
    memset(&d, 0, sizeof(d));
    d.batch = 1;
    for (int i = 0; i < nd - 2; ++i) d.batch *= a_t->shapes[i];  // mat_mul.c:24-27
    d.m = a_t->shapes[nd - 2];
    d.k = a_t->shapes[nd - 1];
    d.n = o_t->shapes[o_t->dim_num_of_shapes - 1];
    const long long b_elems = numel(b_t);
    d.b_shared = b_elems == (long long) d.k * d.n;  // mat_mul.c:42-46
    if (!d.b_shared && b_elems != (long long) d.batch * d.k * d.n)
        return set_error(ONHIP_ERR_ARG, "MatMul eval: second operand has %lld elements, expected %lld or %lld", b_elems,
                         (long long) d.k * d.n, (long long) d.batch * d.k * d.n);
    const size_t a_bytes = (size_t) d.batch * d.m * d.k * 4, b_bytes = (size_t) b_elems * 4;
    const size_t o_bytes = (size_t) d.batch * d.m * d.n * 4;
    const void *a, *b;
    int rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), a_bytes, &a);
    if (rc) return rc;
    const void *b_host = reinterpret_cast<const void *>(inputs[1].addr);
    // the second operand is a weight (fixed) or another activation
    if (b_t->is_fixed_val) rc = const_on_device(b_host, b_bytes, &b);
    else rc = input_on_device(1, b_host, b_bytes, &b);
    if (rc) return rc;
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, o_bytes, &y);
        if (rc) return rc;
    }
    const void *bias = nullptr, *lut = nullptr;
    if (mode) {
        if (numel(bias_t) != d.n) return set_error(ONHIP_ERR_ARG, "MatMul eval: bias of %lld elements for %d columns", numel(bias_t), d.n);
        const void *bias_host = reinterpret_cast<const void *>(inputs[2].addr);
        rc = bias_t->is_fixed_val ? const_on_device(bias_host, (size_t) d.n * 4, &bias) : input_on_device(4, bias_host, (size_t) d.n * 4, &bias);
        if (rc) return rc;
    }
    if (mode == 2) {
        rc = const_on_device(reinterpret_cast<const void *>(inputs[BUF_MAXNUM - 1].addr), 8192 * 4, &lut);
        if (rc) return rc;
    }
    if (mode == 3) {
        if (!inputs[3].addr) return set_error(ONHIP_ERR_ARG, "MatMul eval: no addend in inputs[3]");
        const void *addend;
        rc = input_on_device(5, reinterpret_cast<const void *>(inputs[3].addr), o_bytes, &addend);
        if (rc) return rc;
        rc = onhip_matmul_add(&d, (const float *) a, (const float *) b, (const float *) bias, (const float *) addend, (float *) y, g_stream);
    } else {
        rc = onhip_matmul(&d, (const float *) a, (const float *) b, (const float *) bias, (const float *) lut, (float *) y, g_stream);
    }
    if (rc) return rc;
    if (!out_on_dev) return copy_out(host_out, y, o_bytes);
    return wait_for_output();
}

// `eval_link_takes`: reads params[0..2] only (configuration, input operand, weight operand); 1 when this convolution
// can take and leave int8 NHWC activations through `eval_link`, 0 when it cannot (fp32, or a depthwise shape beyond the
// int8 NHWC depthwise kernel)
static int conv_link_takes(BUFFER_INFO_S *params) {
    const CONV_CONFIG_S *cfg = reinterpret_cast<const CONV_CONFIG_S *>(params[0].addr);
    const OPERAND_S *in_t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    const OPERAND_S *w_t = reinterpret_cast<const OPERAND_S *>(params[2].addr);
    if (!cfg || !in_t || !w_t || cfg->ifmap_quant2 != TYPE_INT8) return 0;
    if (!cfg->has_bias || cfg->group == 1) return 1;   // conv.c:18-29: dense
    onhip_conv_desc_t d;
    block_conv_desc(&d, cfg, in_t->shapes[0] < 1 ? 1 : in_t->shapes[0], in_t->shapes[1], in_t->shapes[2], in_t->shapes[3], w_t);
    int32_t oh = 0, ow = 0;
    if (onhip_conv_out_shape(&d, &oh, &ow) != ONHIP_OK) return 0;
    return onhip_conv2d_w8a8_depthwise_supported(&d);
}

static int matmul_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return matmul_eval_mode(0, params, inputs, outputs);
}
static int matmul_bias_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return matmul_eval_mode(1, params, inputs, outputs);
}
static int matmul_bias_gelu_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return matmul_eval_mode(2, params, inputs, outputs);
}
static int matmul_bias_add_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return matmul_eval_mode(3, params, inputs, outputs);
}

// MatMul(q, Transpose(k)) -> Softmax -> MatMul(., v) as one call.  Slots: params[1..3] the operands q, k, v (all
// [..., tokens, head_dim], k NOT transposed), params[4] the result [..., tokens, head_dim]; inputs[0..2], outputs[0] the
// tensors (host or device memory like every eval).  Leading dimensions are (batch, head) pairs.
// inputs[4]: null, or the address of four int32 flags for q, k, v and the result; a non-zero flag says that this tensor
// (rank 4) is stored [batch, tokens, heads, head_dim], i.e. as it is before a head-split Transpose (0, 2, 1, 3) or after
// the head-merge one, and its operand in params carries that shape; the call walks it with strides.
static int matmul_attention_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const OPERAND_S *t[4];
    for (int i = 0; i < 4; ++i) {
        t[i] = reinterpret_cast<const OPERAND_S *>(params[1 + i].addr);
        if (!t[i]) return set_error(ONHIP_ERR_ARG, "attention eval: empty params slot %d", 1 + i);
    }
    const int32_t *flags = reinterpret_cast<const int32_t *>(inputs[4].addr);
    const bool token_major = flags && (flags[0] || flags[1] || flags[2] || flags[3]);
    const int nd = t[0]->dim_num_of_shapes;
    if (nd < 2 || nd > SHAPE_LEN || (token_major && nd != 4)) return set_error(ONHIP_ERR_ARG, "attention eval: rank %d", nd);
    // every tensor's shape as [..., tokens, head_dim], the two middle axes of a token-major one exchanged
    int32_t shape[4][SHAPE_LEN];
    for (int i = 0; i < 4; ++i) {
        if (t[i]->dim_num_of_shapes != nd) return set_error(ONHIP_ERR_ARG, "attention eval: q, k, v and the result must have one rank");
        for (int a = 0; a < nd; ++a) shape[i][a] = t[i]->shapes[a];
        if (token_major && flags[i]) { shape[i][1] = t[i]->shapes[2]; shape[i][2] = t[i]->shapes[1]; }
        if (memcmp(shape[i], shape[0], nd * sizeof(int32_t)))
            return set_error(ONHIP_ERR_ARG, "attention eval: q, k, v and the result must have one shape");
    }
    onhip_attention_desc_t d;
    memset(&d, 0, sizeof(d));
    d.batch = 1;
    for (int i = 0; i < nd - 2; ++i) d.batch *= shape[0][i];
    d.heads = 1;
    d.tokens = shape[0][nd - 2];
    d.head_dim = shape[0][nd - 1];
    d.scale = 1.0f;
    d.compute = ONHIP_COMPUTE_F32;
    const long long plane = (long long) d.tokens * d.head_dim;
    long long *strides[4] = {d.q_strides, d.k_strides, d.v_strides, d.out_strides};
    for (long long *st : strides) { st[0] = plane; st[1] = plane; st[2] = d.head_dim; }
    if (token_major) {
        d.batch = shape[0][0];
        d.heads = shape[0][1];
        for (int i = 0; i < 4; ++i) {
            strides[i][0] = (long long) d.heads * plane;
            strides[i][1] = flags[i] ? d.head_dim : plane;
            strides[i][2] = flags[i] ? (long long) d.heads * d.head_dim : d.head_dim;
        }
    }
    const size_t bytes = (size_t) d.batch * d.heads * plane * 4;
    const void *in[3];
    for (int i = 0; i < 3; ++i) {
        if (!inputs[i].addr) return set_error(ONHIP_ERR_ARG, "attention eval: empty input slot %d", i);
        // q and k in the first two staging buffers, v in the fifth: the third one holds the result (the kernel reads v
        // of one head while it writes the result of another)
        const int rc = input_on_device(i < 2 ? i : 4, reinterpret_cast<const void *>(inputs[i].addr), bytes, &in[i]);
        if (rc) return rc;
    }
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        const int rc = stage_buf(2, bytes, &y);
        if (rc) return rc;
    }
    const int rc = onhip_attention(&d, in[0], in[1], in[2], y, g_stream);
    if (rc) return rc;
    return out_on_dev ? wait_for_output() : copy_out(host_out, y, bytes);
}

static int gemm_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const OPERAND_S *a_t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    const OPERAND_S *o_t = reinterpret_cast<const OPERAND_S *>(params[4].addr);
    if (!a_t || !o_t) return set_error(ONHIP_ERR_ARG, "Gemm eval: empty params slot");
    const int nd = a_t->dim_num_of_shapes;
    if (nd < 2 || nd > SHAPE_LEN || o_t->dim_num_of_shapes < 1 || o_t->dim_num_of_shapes > SHAPE_LEN)
        return set_error(ONHIP_ERR_ARG, "Gemm eval: rank %d", nd);
    // gemm.c:25-33: M and K from the last two dims of the input, N from the output; leading dims ignored
    const int M = a_t->shapes[nd - 2], K = a_t->shapes[nd - 1], N = o_t->shapes[o_t->dim_num_of_shapes - 1];
    if (M < 1 || K < 1 || N < 1) return set_error(ONHIP_ERR_ARG, "Gemm eval: bad shape %dx%dx%d", M, K, N);
    const void *a, *w, *b;
    int rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), (size_t) M * K * 4, &a);
    if (rc) return rc;
    rc = const_on_device(reinterpret_cast<const void *>(inputs[1].addr), (size_t) N * K * 4, &w);
    if (rc) return rc;
    rc = const_on_device(reinterpret_cast<const void *>(inputs[2].addr), (size_t) N * 4, &b);
    if (rc) return rc;
    if (!b) return set_error(ONHIP_ERR_ARG, "Gemm eval: the reference Gemm always adds a bias; inputs[2] is empty");
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const size_t o_bytes = (size_t) M * N * 4;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, o_bytes, &y);
        if (rc) return rc;
    }
    rc = onhip_gemm_f32(M, K, N, (const float *) a, (const float *) w, (const float *) b, (float *) y, g_stream);
    if (rc) return rc;
    if (!out_on_dev) return copy_out(host_out, y, o_bytes);
    else return wait_for_output();
    return ONHIP_OK;
}

// ---- Add / Relu / MaxPool / GlobalAveragePool ----------------------------------------------------------
// an output on the host is computed into a staging buffer and copied back; one on the device is written in place
static int finish_output(void *host_out, void *y, size_t bytes, bool out_on_dev) {
    if (!out_on_dev) return copy_out(host_out, y, bytes);
    else return wait_for_output();
    return ONHIP_OK;
}

static int add_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const OPERAND_S *t0 = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    const OPERAND_S *t1 = reinterpret_cast<const OPERAND_S *>(params[2].addr);
    if (!t0 || !t1 || !inputs[1].addr) return set_error(ONHIP_ERR_ARG, "Add eval: empty slot");
    // add.c:30-46: the operand with fewer elements is the one that is broadcast (the second one on a tie)
    const long long n0 = numel(t0), n1 = numel(t1);
    const bool small_is_0 = n0 < n1;
    const OPERAND_S *lt = small_is_0 ? t1 : t0, *st = small_is_0 ? t0 : t1;
    const void *lp = reinterpret_cast<const void *>(inputs[small_is_0 ? 1 : 0].addr);
    const void *sp = reinterpret_cast<const void *>(inputs[small_is_0 ? 0 : 1].addr);
    const long long nl = small_is_0 ? n1 : n0, ns = small_is_0 ? n0 : n1;
    onhip_add_desc_t d;
    memset(&d, 0, sizeof(d));
    const int rank = lt->dim_num_of_shapes;
    if (nl == ns || ns == 1) {
        // add.c:48-53: shapes are not looked at
        d.ndim = 1;
        d.large_shape[0] = (int32_t) nl;
        d.small_shape[0] = (int32_t) ns;
        if (nl >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "Add eval: tensor too large");
    } else {
        if (rank < 3 || rank > 6) return set_error(ONHIP_ERR_ARG, "Add eval: broadcast over rank %d (3..6 as add.c:128-141)", rank);
        const int srank = st->dim_num_of_shapes;
        if (srank < 1 || srank > rank) return set_error(ONHIP_ERR_ARG, "Add eval: small operand of rank %d", srank);
        d.ndim = rank;
        for (int i = 0; i < rank; ++i) {
            d.large_shape[i] = lt->shapes[i];
            d.small_shape[i] = i < rank - srank ? 1 : st->shapes[i - (rank - srank)];   // add.c:56-70
        }
    }
    const void *ld, *sd;
    int rc = input_on_device(0, lp, (size_t) nl * 4, &ld);
    if (rc) return rc;
    rc = input_on_device(1, sp, (size_t) ns * 4, &sd);
    if (rc) return rc;
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, (size_t) nl * 4, &y);
        if (rc) return rc;
    }
    rc = onhip_add_f32(&d, (const float *) ld, (const float *) sd, (float *) y, g_stream);
    if (rc) return rc;
    return finish_output(host_out, y, (size_t) nl * 4, out_on_dev);
}

static int relu_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const OPERAND_S *t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    if (!t) return set_error(ONHIP_ERR_ARG, "Relu eval: empty slot");
    const long long n = numel(t);
    if (n < 1 || n >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "Relu eval: %lld elements", n);
    const void *x;
    int rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), (size_t) n * 4, &x);
    if (rc) return rc;
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, (size_t) n * 4, &y);
        if (rc) return rc;
    }
    rc = onhip_relu_f32((const float *) x, (float *) y, n, g_stream);
    if (rc) return rc;
    return finish_output(host_out, y, (size_t) n * 4, out_on_dev);
}

static int maxpool_eval_mode(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs, bool s8);
static int maxpool_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return maxpool_eval_mode(params, inputs, outputs, false);
}
static int maxpool_s8_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return maxpool_eval_mode(params, inputs, outputs, true);
}
// s8: the tensors are int8 NHWC with channels padded to 16
static int maxpool_eval_mode(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs, bool s8) {
    const MAX_POOL_CONFIG_S *cfg = reinterpret_cast<const MAX_POOL_CONFIG_S *>(params[0].addr);
    const OPERAND_S *it = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    const OPERAND_S *ot = reinterpret_cast<const OPERAND_S *>(params[2].addr);
    if (!it || !ot) return set_error(ONHIP_ERR_ARG, "MaxPool eval: empty slot");
    onhip_pool_desc_t d;
    // maxpool.c:67-69 loops over the output's batch and channels with the input's strides
    d.n = ot->shapes[0]; d.c = ot->shapes[1]; d.h = it->shapes[2]; d.w = it->shapes[3];
    if (d.n > it->shapes[0] || d.c != it->shapes[1])
        return set_error(ONHIP_ERR_ARG, "MaxPool eval: output %dx%d planes against input %dx%d", d.n, d.c, it->shapes[0], it->shapes[1]);
    d.kh = (int32_t) cfg->kernel_shape[0]; d.kw = (int32_t) cfg->kernel_shape[1];
    d.stride_w = (int32_t) cfg->strides[0]; d.stride_h = (int32_t) cfg->strides[1];
    d.pad = (int32_t) cfg->pads[0];
    const int32_t oh = ot->shapes[2], ow = ot->shapes[3];
    const size_t cp = ((size_t) d.c + 15) / 16 * 16;
    const size_t in_bytes = s8 ? (size_t) d.n * d.h * d.w * cp : (size_t) d.n * d.c * d.h * d.w * 4;
    const size_t out_bytes = s8 ? (size_t) d.n * oh * ow * cp : (size_t) d.n * d.c * oh * ow * 4;
    const void *x;
    int rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), in_bytes, &x);
    if (rc) return rc;
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, out_bytes, &y);
        if (rc) return rc;
    }
    if (s8) rc = onhip_maxpool_s8_nhwc(&d, oh, ow, (const int8_t *) x, (int8_t *) y, g_stream);
    else rc = onhip_maxpool_f32(&d, oh, ow, (const float *) x, (float *) y, g_stream);
    if (rc) return rc;
    return finish_output(host_out, y, out_bytes, out_on_dev);
}

static int gap_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const OPERAND_S *it = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    if (!it) return set_error(ONHIP_ERR_ARG, "GlobalAveragePool eval: empty slot");
    const int n = it->shapes[0], c = it->shapes[1], h = it->shapes[2], w = it->shapes[3];
    if (n < 1 || c < 1 || h < 1 || w < 1) return set_error(ONHIP_ERR_ARG, "GlobalAveragePool eval: bad shape");
    const size_t in_bytes = (size_t) n * c * h * w * 4, out_bytes = (size_t) n * c * 4;
    const void *x;
    int rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), in_bytes, &x);
    if (rc) return rc;
    void *host_out = reinterpret_cast<void *>(outputs[0].addr);
    void *y = host_out;
    const bool out_on_dev = is_device_ptr(host_out);
    if (!out_on_dev) {
        rc = stage_buf(2, out_bytes, &y);
        if (rc) return rc;
    }
    rc = onhip_global_avgpool_f32(n, c, h, w, (const float *) x, (float *) y, g_stream);
    if (rc) return rc;
    return finish_output(host_out, y, out_bytes, out_on_dev);
}

// ---- Gelu / LayerNormalization / Softmax / Transpose ------------------------------------------------------
// shared shape of the unary operators: input 0 on the device, output staged or in place
struct UnaryIo {
    const void *x;
    void *y, *host_out;
    size_t out_bytes;
    bool out_on_dev;
};
static int unary_io(BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs, size_t in_bytes, size_t out_bytes, UnaryIo *io) {
    int rc = input_on_device(0, reinterpret_cast<const void *>(inputs[0].addr), in_bytes, &io->x);
    if (rc) return rc;
    io->host_out = reinterpret_cast<void *>(outputs[0].addr);
    io->y = io->host_out;
    io->out_bytes = out_bytes;
    io->out_on_dev = is_device_ptr(io->host_out);
    if (!io->out_on_dev) rc = stage_buf(2, out_bytes, &io->y);
    return rc;
}

static int gelu_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const OPERAND_S *t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    if (!t || !inputs[BUF_MAXNUM - 1].addr) return set_error(ONHIP_ERR_ARG, "Gelu eval: empty slot (the table is inputs[11])");
    const long long n = numel(t);
    if (n < 1 || n >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "Gelu eval: %lld elements", n);
    const void *lut;
    int rc = const_on_device(reinterpret_cast<const void *>(inputs[BUF_MAXNUM - 1].addr), 8192 * 4, &lut);
    if (rc) return rc;
    UnaryIo io;
    rc = unary_io(inputs, outputs, (size_t) n * 4, (size_t) n * 4, &io);
    if (rc) return rc;
    rc = onhip_gelu_lut_f32((const float *) io.x, (const float *) lut, (float *) io.y, n, g_stream);
    if (rc) return rc;
    return finish_output(io.host_out, io.y, io.out_bytes, io.out_on_dev);
}

static int layernorm_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const LAYERNORMALIZATION_CONFIG_S *cfg = reinterpret_cast<const LAYERNORMALIZATION_CONFIG_S *>(params[0].addr);
    const OPERAND_S *t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    if (!t || !inputs[1].addr || !inputs[2].addr) return set_error(ONHIP_ERR_ARG, "LayerNormalization eval: empty slot");
    const long long n = numel(t);
    if (n < 1 || n >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "LayerNormalization eval: %lld elements", n);
    int reduce = 1, strided = 0;
    if (cfg->axes[0] == 1) {
        reduce = t->shapes[1];                         // layer_normalization.c:28-31
        strided = 1;
    } else {
        for (int i = SHAPE_LEN - 1; i >= 0; --i)       // :63-68: the last dimension that is not 1
            if (t->shapes[i] != 1) { reduce = t->shapes[i]; break; }
    }
    if (reduce < 1) return set_error(ONHIP_ERR_ARG, "LayerNormalization eval: bad shape");
    const int rows = (int) (n / reduce);
    const void *w, *b;
    int rc = const_on_device(reinterpret_cast<const void *>(inputs[1].addr), (size_t) reduce * 4, &w);
    if (rc) return rc;
    rc = const_on_device(reinterpret_cast<const void *>(inputs[2].addr), (size_t) reduce * 4, &b);
    if (rc) return rc;
    UnaryIo io;
    rc = unary_io(inputs, outputs, (size_t) n * 4, (size_t) n * 4, &io);
    if (rc) return rc;
    rc = onhip_layernorm_f32(rows, reduce, strided, (const float *) io.x, (const float *) w, (const float *) b, (float *) io.y,
                             g_stream);
    if (rc) return rc;
    return finish_output(io.host_out, io.y, io.out_bytes, io.out_on_dev);
}

static int softmax_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const SOFTMAX_CONFIG_S *cfg = reinterpret_cast<const SOFTMAX_CONFIG_S *>(params[0].addr);
    const OPERAND_S *t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    if (!t) return set_error(ONHIP_ERR_ARG, "Softmax eval: empty slot");
    const int nd = t->dim_num_of_shapes;
    if (nd < 1 || nd > SHAPE_LEN) return set_error(ONHIP_ERR_ARG, "Softmax eval: rank %d", nd);
    long long rows = 1;
    int reduce, strided;
    if (cfg->axis == -1 || cfg->axis == nd - 1) {      // softmax.c:18-19, :36-41
        for (int i = 0; i < nd - 1; ++i) rows *= t->shapes[i];
        reduce = t->shapes[nd - 1];
        strided = 0;
    } else if (cfg->axis == 1 && t->shapes[0] == 1) {  // :20-21, :72-77
        for (int i = 2; i < nd; ++i) rows *= t->shapes[i];
        reduce = t->shapes[1];
        strided = 1;
    } else {
        return set_error(ONHIP_ERR_ARG, "Softmax eval: axis %lld of a rank-%d tensor is not supported (last axis, or axis 1 "
                                        "of a batch-1 tensor, as the reference)", (long long) cfg->axis, nd);
    }
    if (rows < 1 || reduce < 1 || rows * reduce >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "Softmax eval: bad shape");
    UnaryIo io;
    int rc = unary_io(inputs, outputs, (size_t) rows * reduce * 4, (size_t) rows * reduce * 4, &io);
    if (rc) return rc;
    rc = onhip_softmax_f32((int) rows, reduce, strided, (const float *) io.x, (float *) io.y, g_stream);
    if (rc) return rc;
    return finish_output(io.host_out, io.y, io.out_bytes, io.out_on_dev);
}

static int transpose_eval_locked(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    const TRANSPOSE_CONFIG_S *cfg = reinterpret_cast<const TRANSPOSE_CONFIG_S *>(params[0].addr);
    const OPERAND_S *t = reinterpret_cast<const OPERAND_S *>(params[1].addr);
    if (!t) return set_error(ONHIP_ERR_ARG, "Transpose eval: empty slot");
    const int pn = (int) cfg->perm_num;
    if (pn < 1 || pn > 6) return set_error(ONHIP_ERR_ARG, "Transpose eval: %d axes (up to 6 as transpose.c:18-24)", pn);
    // transpose.c works on 4 (perm_num <= 4) or 6 dimensions; trailing dimensions keep their place
    const int nd = pn <= 4 ? 4 : 6;
    onhip_transpose_desc_t d;
    memset(&d, 0, sizeof(d));
    d.ndim = nd;
    long long n = 1;
    for (int i = 0; i < nd; ++i) {
        d.in_shape[i] = t->shapes[i];
        d.perm[i] = i < pn ? (int32_t) cfg->perm[i] : i;
        n *= t->shapes[i];
    }
    if (n < 1 || n >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "Transpose eval: %lld elements", n);
    UnaryIo io;
    int rc = unary_io(inputs, outputs, (size_t) n * 4, (size_t) n * 4, &io);
    if (rc) return rc;
    rc = onhip_transpose_f32(&d, (const float *) io.x, (float *) io.y, g_stream);
    if (rc) return rc;
    return finish_output(io.host_out, io.y, io.out_bytes, io.out_on_dev);
}

template <class F>
static int guarded(const char *what, F f, BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    if (!params || !inputs || !outputs || !params[0].addr || !inputs[0].addr || !outputs[0].addr) {
        int rc = set_error(ONHIP_ERR_ARG, "%s eval: null slot array or empty slot 0", what);
        fprintf(stderr, "[onenew_hip] %s\n", onhip_last_error());
        return rc;
    }
    std::lock_guard<std::mutex> lock(g_mu);
    int rc = ensure_ready();
    if (!rc) rc = f(params, inputs, outputs);
    // the host ignores the return value (host/op.h:183): make failures visible
    if (rc) fprintf(stderr, "[onenew_hip] %s eval failed (%d): %s\n", what, rc, onhip_last_error());
    return rc;
}

}  // namespace onhip

using namespace onhip;

extern "C" {

int onhip_conv_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Conv", conv_eval_locked, params, inputs, outputs);
}
int onhip_conv_add_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Conv + Add", conv_add_eval_locked, params, inputs, outputs);
}

int onhip_conv_add_relu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Conv + Add + Relu", conv_add_relu_eval_locked, params, inputs, outputs);
}
int onhip_conv_link_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *, BUFFER_INFO_S *) {
    return params ? conv_link_takes(params) : 0;
}
int onhip_conv_link_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Conv (int8 edges)", conv_link_eval_locked, params, inputs, outputs);
}
int onhip_conv_block_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Conv -> depthwise Conv -> Conv", conv_block_eval_locked, params, inputs, outputs);
}
int onhip_conv_block_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    if (!params) return 0;
    return conv_block_eval_mode(params, inputs, outputs, true);
}

int onhip_conv_pair_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Conv -> 1x1 Conv", conv_pair_eval_locked, params, inputs, outputs);
}
int onhip_conv_pair_relu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Conv -> 1x1 Conv -> Add -> Relu", conv_pair_relu_eval_locked, params, inputs, outputs);
}
int onhip_conv_pair_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    if (!params) return 0;
    return conv_pair_eval_mode(params, inputs, outputs, true, false);
}

int onhip_matmul_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("MatMul", matmul_eval_locked, params, inputs, outputs);
}
int onhip_matmul_bias_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("MatMul (+ bias)", matmul_bias_eval_locked, params, inputs, outputs);
}
int onhip_matmul_bias_gelu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("MatMul (+ bias + Gelu)", matmul_bias_gelu_eval_locked, params, inputs, outputs);
}
int onhip_matmul_bias_add_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("MatMul (+ bias + Add)", matmul_bias_add_eval_locked, params, inputs, outputs);
}
int onhip_matmul_attention_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("MatMul (attention)", matmul_attention_eval_locked, params, inputs, outputs);
}
int onhip_gemm_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Gemm", gemm_eval_locked, params, inputs, outputs);
}

int onhip_add_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Add", add_eval_locked, params, inputs, outputs);
}

int onhip_relu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Relu", relu_eval_locked, params, inputs, outputs);
}

int onhip_maxpool_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("MaxPool", maxpool_eval_locked, params, inputs, outputs);
}

int onhip_maxpool_s8_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("MaxPool (int8)", maxpool_s8_eval_locked, params, inputs, outputs);
}

int onhip_global_avgpool_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("GlobalAveragePool", gap_eval_locked, params, inputs, outputs);
}

int onhip_gelu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Gelu", gelu_eval_locked, params, inputs, outputs);
}

int onhip_layernorm_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("LayerNormalization", layernorm_eval_locked, params, inputs, outputs);
}

int onhip_softmax_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Softmax", softmax_eval_locked, params, inputs, outputs);
}

int onhip_transpose_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs) {
    return guarded("Transpose", transpose_eval_locked, params, inputs, outputs);
}

int onhip_plugin_set_async(int on) {
    std::lock_guard<std::mutex> lock(g_mu);
    g_async = on != 0;
    return ONHIP_OK;
}

int onhip_plugin_set_stream(void *stream) {
    std::lock_guard<std::mutex> lock(g_mu);
    g_stream = reinterpret_cast<hipStream_t>(stream);
    return ONHIP_OK;
}

int onhip_plugin_forget(const void *base, size_t bytes) {
    std::lock_guard<std::mutex> lock(g_mu);
    const char *lo = static_cast<const char *>(base), *hi = lo + bytes;
    bool any = false;
    for (auto it = g_packed.begin(); it != g_packed.end();) {
        const char *k = static_cast<const char *>(it->first);
        if (k >= lo && k < hi) {
            if (!any) ONHIP_CHECK_HIP(hipDeviceSynchronize());   // a kernel may still be reading the copy
            any = true;
            (void) hipFree(it->second.dev);
            it = g_packed.erase(it);
        } else {
            ++it;
        }
    }
    return forget_quantised_tables(base, bytes);
}

int onhip_plugin_trust_weights(int on) {
    std::lock_guard<std::mutex> lock(g_mu);
    g_weight_check_sampled = on != 0;
    return ONHIP_OK;
}

int onhip_plugin_release(void) {
    std::lock_guard<std::mutex> lock(g_mu);
    ONHIP_CHECK_HIP(hipDeviceSynchronize());
    for (auto &kv : g_packed) (void) hipFree(kv.second.dev);
    g_packed.clear();
    for (auto &kv : g_const) (void) hipFree(kv.second.dev);
    g_const.clear();
    for (auto &b : g_stage) {
        if (b.ptr) (void) hipFree(b.ptr);
        b.ptr = nullptr;
        b.bytes = 0;
    }
    return ONHIP_OK;
}

}  // extern "C"
